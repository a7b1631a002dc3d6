"""Routed MoE experts (stacked EXL3 SwitchGLU) on ROCm tensors.

Mirrors ``EXL3SwitchGLU`` (ponyexl3/mlx/exl3_moe.py:425-457,770-787) and the
router / weighted sum of ``EXL3MoEBlock`` (ponyexl3/mlx/exl3_moe.py:790-839).
"""

from __future__ import annotations

import numpy as np
import torch

from . import ops
from .layer import EXL3Layer, codebook_mode_from_flags, unpack_signs_or_pass

_MOE_ACTIVATIONS = {"silu": 0, "gelu": 1}


class EXL3SwitchGLU(torch.nn.Module):
    """Stacked-expert EXL3 SwitchGLU: ``(x (B,S,D), indices (B,S,kk)) -> (B,S,kk,D)``.

    gu_trellis (D/16, E*2*H/16, 16K) laid out [all experts' gate | all experts' up],
    gu_suh (E, 2, D), gu_svh (E, 2*H), dn_trellis (H/16, E*D/16, 16K),
    dn_suh (E, H), dn_svh (E, D)."""

    def __init__(self, *, gu_trellis, gu_suh, gu_svh, dn_trellis, dn_suh, dn_svh, k, cb,
                 activation: str = "silu"):
        super().__init__()
        if activation not in _MOE_ACTIVATIONS:
            raise ValueError(f"unsupported MoE activation {activation!r}")
        self._gu_trellis = gu_trellis
        self._gu_suh = gu_suh
        self._gu_svh = gu_svh
        self._dn_trellis = dn_trellis
        self._dn_suh = dn_suh
        self._dn_svh = dn_svh
        self._k = int(k)
        self._cb = int(cb)
        self._activation = activation
        self.num_experts = int(gu_suh.shape[0])
        self.input_dims = int(gu_suh.shape[2])
        self.hidden_dims = int(dn_suh.shape[1])
        E, D, H = self.num_experts, self.input_dims, self.hidden_dims
        if D % 128 or H % 128:
            raise ValueError("MoE dims must be multiples of 128")
        expect = {
            "gu_trellis": (D // 16, E * 2 * H // 16, 16 * self._k),
            "gu_suh": (E, 2, D),
            "gu_svh": (E, 2 * H),
            "dn_trellis": (H // 16, E * D // 16, 16 * self._k),
            "dn_suh": (E, H),
            "dn_svh": (E, D),
        }
        for name, shape in expect.items():
            got = tuple(getattr(self, "_" + name).shape)
            if got != shape:
                raise ValueError(f"{name} shape {got} != expected {shape}")

    @classmethod
    def from_layers(cls, gate: list[EXL3Layer], up: list[EXL3Layer], down: list[EXL3Layer],
                    activation: str = "silu", device="cuda") -> "EXL3SwitchGLU":
        """Stack per-expert layers the way the reference's loader does
        (ponyexl3/mlx/model.py:96-122)."""
        first = gate[0]
        for l in gate + up + down:
            l.validate()
            if (l.k, l.mcg, l.mul1) != (first.k, first.mcg, first.mul1):
                raise ValueError("all expert layers must share K and codebook")
        tr = lambda ls: np.concatenate([np.asarray(l.trellis).view(np.uint16) for l in ls], axis=1)
        sg = lambda v: unpack_signs_or_pass(v).astype(np.float16)
        h = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device)
        return cls(
            gu_trellis=ops.as_trellis_tensor(np.concatenate([tr(gate), tr(up)], axis=1), device),
            gu_suh=h(np.stack([np.stack([sg(g.suh), sg(u.suh)]) for g, u in zip(gate, up)])),
            gu_svh=h(np.stack([np.concatenate([sg(g.svh), sg(u.svh)]) for g, u in zip(gate, up)])),
            dn_trellis=ops.as_trellis_tensor(tr(down), device),
            dn_suh=h(np.stack([sg(d.suh) for d in down])),
            dn_svh=h(np.stack([sg(d.svh) for d in down])),
            k=first.k,
            cb=int(codebook_mode_from_flags(mcg=first.mcg, mul1=first.mul1)),
            activation=activation,
        )

    # The sorted, segmented prefill path replaces the slot kernels once the experts see
    # a few rows each (the reference switches at 9 tokens,
    # ponyexl3/mlx/exl3_moe.py:770-787). Measured on 256 experts of 2048 x 512, top-8:
    # the slot kernels, which share one pass over an expert's weights among up to four
    # of its slots as long as the call has at most 512 slots, take 64 / 97 / 124 /
    # 158 us at 16 / 32 / 48 / 64 tokens and 255 us at 72 (576 slots, every slot on
    # its own); the prefill path takes 180-207 us from 40 to 96 tokens (every expert's
    # weights are decoded once, eight launches). So: prefill above 512 slots, and
    # below that from 2.5 rows per expert on (few experts, many rows each).
    prefill_min_tokens = 24
    prefill_min_rows_per_expert = 2.5
    grouped_max_slots = 512

    def _use_prefill(self, tokens: int, top_k: int) -> bool:
        slots = tokens * top_k
        return tokens >= self.prefill_min_tokens and (
            slots > self.grouped_max_slots
            or slots >= self.prefill_min_rows_per_expert * self.num_experts)

    def forward(self, x: torch.Tensor, indices: torch.Tensor) -> torch.Tensor:
        if indices.dim() != 3:
            raise ValueError("indices must be (B, S, top_k)")
        B, S, kk = indices.shape
        R = B * S
        D = self.input_dims
        x2d = x.reshape(R, D).to(torch.float16).contiguous()
        idx = indices.reshape(R, kk).to(torch.int32).contiguous()
        if self._use_prefill(R, kk):
            return self._prefill(x2d, idx).reshape(B, S, kk, D)
        chunk = max(1, 4096 // kk)
        outs = []
        for r0 in range(0, R, chunk):
            outs.append(
                ops.moe_forward(
                    x2d[r0 : r0 + chunk], idx[r0 : r0 + chunk], self._gu_trellis, self._gu_suh,
                    self._gu_svh, self._dn_trellis, self._dn_suh, self._dn_svh, self._k, self._cb,
                    _MOE_ACTIVATIONS[self._activation],
                )
            )
        y = outs[0] if len(outs) == 1 else torch.cat(outs, dim=0)
        return y.reshape(B, S, kk, D)

    def _prefill(self, x2d: torch.Tensor, idx: torch.Tensor) -> torch.Tensor:
        """Many tokens: sort the (token, slot) pairs by expert so that every expert's
        weights are decoded once per block of its rows, rotate with per-row sign
        vectors, run the segmented MFMA GEMM, finish per row, unsort
        (``EXL3SwitchGLU._prefill``, ponyexl3/mlx/exl3_moe.py:684-768). No host
        synchronisation: the block table is built on the device for the worst case."""
        E, D, H = self.num_experts, self.input_dims, self.hidden_dims
        R, kk = idx.shape
        N = R * kk
        per_expert = N / E
        block_rows = 64 if per_expert <= 48 else 128 if per_expert <= 112 else 256
        if E <= ops.MOE_SORT_MAX_EXPERTS:
            order32, tok32, sidx32, table = ops.moe_sort(idx, E, block_rows)  # one launch
        else:
            flat = idx.reshape(-1).long().clamp_(0, E - 1)
            order = torch.argsort(flat, stable=True)
            sidx = flat[order]
            table = ops.segment_table(sidx, E, block_rows)
            sidx32, order32 = sidx.int(), order.int()
            tok32 = torch.div(order, kk, rounding_mode="floor").int()
        k, cb = self._k, self._cb
        gt, dt = H // 16, D // 16
        # rotations read x through the token table and the signs through the expert table
        xg = ops.had128_rows(x2d, self._gu_suh[:, 0], False, in_index=tok32, scale_index=sidx32)
        xu = ops.had128_rows(x2d, self._gu_suh[:, 1], False, in_index=tok32, scale_index=sidx32)
        g = ops.gemm_grouped(xg, self._gu_trellis, k, cb, 0, gt, E, table, block_rows)
        u = ops.gemm_grouped(xu, self._gu_trellis, k, cb, E * gt, gt, E, table, block_rows)
        # finish gate and up, GLU, rotate for the down projection: one launch
        xd = ops.moe_glu_rows(g, u, sidx32, self._gu_svh, self._dn_suh,
                              _MOE_ACTIVATIONS[self._activation])
        y = ops.gemm_grouped(xd, self._dn_trellis, k, cb, 0, dt, E, table, block_rows)
        # finish and scatter back to (token, slot) order in one pass
        y = ops.had128_rows(y, self._dn_svh, True, scale_index=sidx32, out_index=order32)
        return y.reshape(R, kk, D)


def route_topk(logits: torch.Tensor, top_k: int, norm_topk_prob: bool = True):
    """softmax (fp32) -> top-k -> optional renormalisation
    (ponyexl3/mlx/exl3_moe.py:817-821). Returns (indices int32, scores fp32)."""
    gates = torch.softmax(logits.float(), dim=-1)
    scores, inds = torch.topk(gates, top_k, dim=-1)
    if norm_topk_prob:
        scores = scores / scores.sum(dim=-1, keepdim=True)
    return inds.to(torch.int32), scores


def combine_experts(y: torch.Tensor, scores: torch.Tensor) -> torch.Tensor:
    """(…, kk, D) x (…, kk) -> (…, D) (ponyexl3/mlx/exl3_moe.py:838-839)."""
    return (y * scores[..., None].to(y.dtype)).sum(dim=-2)


class EXL3MoEBlock(torch.nn.Module):
    """Router + routed experts + weighted sum (``EXL3MoEBlock``,
    ponyexl3/mlx/exl3_moe.py:790-839). With ``shared_gate`` the shared expert is
    stacked as the LAST expert of ``switch`` and always selected, its routing
    weight being ``sigmoid(shared_gate(x))``; the router only ranks the others.
    ``x (..., D) -> (..., D)``."""

    def __init__(self, gate: torch.nn.Module, shared_gate: torch.nn.Module | None,
                 switch: EXL3SwitchGLU, top_k: int, norm_topk_prob: bool = True):
        super().__init__()
        self.gate = gate
        self.shared_expert_gate = shared_gate
        self.switch_mlp = switch
        self.top_k = int(top_k)
        self.norm_topk_prob = bool(norm_topk_prob)
        self._shared_idx = switch.num_experts - 1

    def route(self, x: torch.Tensor):
        inds, scores = route_topk(self.gate(x), self.top_k, self.norm_topk_prob)
        scores = scores.to(x.dtype)
        if self.shared_expert_gate is not None:
            shared_w = torch.sigmoid(self.shared_expert_gate(x)).to(x.dtype)
            shared = torch.full(inds.shape[:-1] + (1,), self._shared_idx, dtype=inds.dtype,
                                device=inds.device)
            inds = torch.cat([inds, shared], dim=-1)
            scores = torch.cat([scores, shared_w], dim=-1)
        return inds, scores

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        lead = tuple(x.shape[:-1])
        x3 = x.reshape(1, -1, x.shape[-1])
        inds, scores = self.route(x3)
        y = self.switch_mlp(x3, inds)
        return combine_experts(y, scores).reshape(lead + (x.shape[-1],))
