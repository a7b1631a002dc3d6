#!/usr/bin/env python3
"""Benchmark of the EXL3 quantized-linear hot path on one MI355X.

A step is one pass over the linears of one 27B-class decoder layer at batch 1
(q 5120->8192 with k and v 5120->1024, o 8192->5120, gate+up 5120->17408,
down 17408->5120; K=4, 3INST; seeded random trellis words, +-1 signs, fp16
x ~ N(0,1)): 180.9 MB of packed weights. Linears that share an input run as one
sibling-fused launch (gate+up, and q+k+v as the reference does for groups above
64 MB of fp16-equivalent weights, ponyexl3/mlx/model.py:354-373), so a step is
four launches; --unfused-qkv runs q, k and v as three. Successive steps rotate over
several distinct copies of the layer so the weights come from HBM, not from the
256 MB last-level cache. ``value`` is effective weight bytes per second over the
whole step (Hadamard kernels and launch gaps included).

Prints ONE JSON line: metric, value, unit, n_gpus, steps, warmup, ms_per_step,
higher_is_better, scaling, vs_baseline, dtype, data, config, plus the objects
roofline (dominant kernel = the one-launch layer kernel, launch durations from
HIP events around batched graph replays on cold weights; next to the published
8 TB/s it carries the streaming-read rate and the decode-loop rate measured in
the same run), ceilings (those two measurements in full), cpu_baseline (the C
oracle on the host cores), batch_rows (2..128 rows), config1, prefill_gemm
(M=2048, config 3), moe (config 4), encoder, config5 (K in {2,3,5,6,8} x {3INST,
MCG} x 1/4/8 rows), eager_ms_per_step (the same steps without a graph) and
launch_plans (the host-side plan of each of the step's launches).
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_F16_PEAK_TFLOPS = 2500.0
K_BITS = 4
CB = 0
# HBM bytes moved by the four layer-kernel launches of one step, from two
# rocprofv3 --pmc runs of this script (FETCH_SIZE, then WRITE_SIZE), each scaled
# by what the same counter reads for a plain copy of known size; see
# profiles/linear_small_k4_config2_pmc.txt.
TRAFFIC_BYTES_PER_STEP = 200_702_566

# (name, in, [member out sizes]) of the config-2 layer; several members = sibling-fused
LAYER_FUSED_QKV = [
    ("qkv_proj", 5120, [8192, 1024, 1024]),
    ("o_proj", 8192, [5120]),
    ("gate_up", 5120, [17408, 17408]),
    ("down_proj", 17408, [5120]),
]
LAYER_SPLIT_QKV = [
    ("q_proj", 5120, [8192]),
    ("k_proj", 5120, [1024]),
    ("v_proj", 5120, [1024]),
] + LAYER_FUSED_QKV[1:]
LAYER = LAYER_FUSED_QKV


def weight_bytes(n_in, outs, k=K_BITS):
    return n_in * sum(outs) * k // 8


def make_linear_np(n_in, outs, seed, k=K_BITS):
    """Seeded synthetic linear(s): raw random trellis words, +-1 signs (numpy).
    Members are concatenated along the tile columns, one suh row per member."""
    rng = np.random.default_rng(seed)
    trellis = rng.integers(0, 65536, size=(n_in // 16, sum(outs) // 16, 16 * k), dtype=np.uint16)
    suh = np.where(rng.random((len(outs), n_in)) > 0.5, -1.0, 1.0).astype(np.float16)
    svh = np.where(rng.random(sum(outs)) > 0.5, -1.0, 1.0).astype(np.float16)
    return trellis, suh, svh


class DeviceLinear:
    def __init__(self, name, n_in, outs, seed, device):
        import torch

        from ponyexl3_amd import ops

        tr, suh, svh = make_linear_np(n_in, outs, seed)
        members = len(outs)
        self.name, self.n_in, self.n_out, self.members = name, n_in, sum(outs), members
        self.trellis = ops.as_trellis_tensor(tr, device)
        self.suh = torch.from_numpy(suh if members > 1 else suh[0]).to(device)
        self.svh = torch.from_numpy(svh).to(device)
        self.group_sub = None
        if members > 1:
            gs = np.repeat(np.arange(members, dtype=np.int32), [o // 128 for o in outs])
            self.group_sub = torch.from_numpy(gs).to(device)
        # member of every 256-column block (one-launch prefill GEMM of a sibling group)
        self.block_sub = (self.group_sub[::2].contiguous()
                          if members > 1 and all(o % 256 == 0 for o in outs) else None)
        self.bytes = weight_bytes(n_in, outs)
        self.outs = list(outs)

    def forward(self, x):
        from ponyexl3_amd import ops

        return ops.linear_forward(x, self.trellis, K_BITS, CB, self.suh, self.svh, None, self.group_sub,
                                  member_out=self.outs if self.members > 1 else None,
                                  block_sub=self.block_sub)


def cpu_baseline(budget_s=12.0):
    """The C oracle (decode + Hadamard-128 + matvec, ponyexl3.ref restated) on
    this host's cores over one config-2 layer; returns the JSON object."""
    from oracle import exl3_oracle as orc

    threads = int(os.environ.get("OMP_NUM_THREADS", "0")) or min(16, os.cpu_count() or 1)
    orc.set_num_threads(threads)
    layers = []
    for i, (name, n_in, outs) in enumerate(LAYER):
        tr, suh, svh = make_linear_np(n_in, outs, 20_000 + 100 * i + K_BITS)
        c0 = 0
        for m, n_out in enumerate(outs):  # the CPU runs the members one after the other
            layers.append((np.ascontiguousarray(tr[:, c0 // 16 : (c0 + n_out) // 16]), suh[m],
                           svh[c0 : c0 + n_out], n_in))
            c0 += n_out
    x = {n: np.random.default_rng(n).standard_normal(n).astype(np.float16) for n in (5120, 8192, 17408)}
    total = sum(weight_bytes(n_in, outs) for _, n_in, outs in LAYER)

    def run(seconds):
        reps, t0 = 0, time.perf_counter()
        while True:
            for tr, suh, svh, n_in in layers:
                orc.linear_forward_bs1(tr, K_BITS, CB, suh, svh, x[n_in])
            reps += 1
            dt = time.perf_counter() - t0
            if dt > seconds:
                return reps, dt

    reps, dt = run(budget_s)
    orc.set_num_threads(1)  # one pass on a single core for scale (about 4 s)
    reps1, dt1 = run(0.0)
    orc.set_num_threads(threads)
    model = "unknown"
    try:
        with open("/proc/cpuinfo", encoding="utf-8") as f:
            for line in f:
                if line.startswith("model name"):
                    model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    return {
        "value": round(total * reps / dt / 1e9, 4),
        "unit": "GB/s",
        "cores": threads,
        "kind": "port",
        "sample": f"{reps} pass(es) over one config-2 decoder layer at batch 1 "
                  f"({total / 1e6:.1f} MB of K=4 trellis, decode + Hadamard-128 + matvec), "
                  f"C oracle with OpenMP, {dt:.1f} s",
        "single_core_value": round(total * reps1 / dt1 / 1e9, 4),
        "cpu_model": model,
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--repeats", type=int, default=7,
                    help="the timed region of --steps steps is run this many times; the median is reported")
    ap.add_argument("--layers", type=int, default=4, help="distinct weight copies rotated over")
    ap.add_argument("--no-graph", action="store_true", help="launch eagerly instead of replaying HIP graphs")
    ap.add_argument("--skip-cpu", action="store_true")
    ap.add_argument("--skip-extras", action="store_true", help="skip prefill GEMM and MoE figures")
    ap.add_argument("--unfused-qkv", action="store_true", help="run q, k, v as three launches")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one 64 MiB device-to-device copy (for counter runs: FETCH_SIZE / "
                         "WRITE_SIZE of a transfer of known size)")
    args = ap.parse_args()
    global LAYER
    if args.unfused_qkv:
        LAYER = LAYER_SPLIT_QKV
    if args.gpus != 1:
        print("bench.py measures one GPU: this build uses no second GPU, collectives or sharding; "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch

    from ponyexl3_amd import _lib, ops

    assert torch.cuda.is_available(), "no HIP device visible"
    _lib.load()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.copy_calibration:
        src = torch.zeros(64 << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    n_layers = max(1, args.layers)
    layers = [
        [DeviceLinear(n, i_, o_, 20_000 + 1000 * L + 100 * j + K_BITS, dev)
         for j, (n, i_, o_) in enumerate(LAYER)]
        for L in range(n_layers)
    ]
    bytes_per_step = sum(l.bytes for l in layers[0])
    g = torch.Generator().manual_seed(1234)
    xs = {n: torch.randn((1, n), generator=g).to(torch.float16).to(dev) for n in (5120, 8192, 17408)}

    def step(L):
        outs = []
        for lin in layers[L]:
            outs.append(lin.forward(xs[lin.n_in]))
        return outs

    for L in range(n_layers):  # grows the workspace, loads code objects
        step(L)
    torch.cuda.synchronize()

    # HIP graphs as a decoder would use them: one graph holds the steps of all
    # n_layers layer copies back to back (a graph launch costs a few microseconds
    # whatever it holds); single-layer graphs cover a step count that is not a
    # multiple of n_layers.
    graphs = None
    graph_all = None
    if not args.no_graph:
        try:
            graphs = []
            for L in range(n_layers):
                gr = torch.cuda.CUDAGraph()
                with torch.cuda.graph(gr):
                    keep = step(L)
                graphs.append((gr, keep))
            gr = torch.cuda.CUDAGraph()
            with torch.cuda.graph(gr):
                keep = [step(L) for L in range(n_layers)]
            graph_all = (gr, keep)
            torch.cuda.synchronize()
        except Exception as e:  # noqa: BLE001
            print(f"HIP graph capture failed ({e!r}); timing eager launches", file=sys.stderr)
            graphs = None
            graph_all = None

    def run_steps(count):
        """Exactly `count` layer steps, layer copies in rotation."""
        i = 0
        while i < count:
            if graph_all is not None and i % n_layers == 0 and count - i >= n_layers:
                graph_all[0].replay()
                i += n_layers
            elif graphs is not None:
                graphs[i % n_layers][0].replay()
                i += 1
            else:
                step(i % n_layers)
                i += 1

    run_steps(args.warmup)
    torch.cuda.synchronize()
    # exactly --steps steps between two synchronisations, --repeats times; the
    # reported figure is the median of the repeats (a 20-step region is under 2 ms)
    samples, event_samples = [], []
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for _ in range(max(1, args.repeats)):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        ev0.record()  # HIP events on the stream the kernels are launched on
        run_steps(args.steps)
        ev1.record()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        samples.append((t1 - t0) * 1e3 / args.steps)
        event_samples.append(ev0.elapsed_time(ev1) / args.steps)
    ms_per_step = float(np.median(samples))
    event_ms_per_step = float(np.median(event_samples))
    value = bytes_per_step / (ms_per_step * 1e-3) / 1e9

    # the same steps launched eagerly through the module path (ctypes call per launch,
    # no graph): what EXL3Linear costs a caller that does not capture its decode step
    eager_samples = []
    for _ in range(3):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(args.steps):
            step(i % n_layers)
        torch.cuda.synchronize()
        eager_samples.append((time.perf_counter() - t0) * 1e3 / args.steps)
    eager_ms_per_step = float(np.median(eager_samples))

    # launch plans (box-independent host decisions): a slow box can be told from a bad plan
    import ctypes

    lib = _lib.load()
    plans = {}
    for lin in layers[0]:
        v = [ctypes.c_int() for _ in range(4)]
        _lib.check(lib.exl3_linear_plan(1, lin.n_in // 16, lin.n_out // 16, K_BITS, *[ctypes.byref(c) for c in v]),
                   "exl3_linear_plan")
        splits, tk, nw, atomic = (c.value for c in v)
        plans[lin.name] = {"grid": f"{lin.n_out // 128}x{(splits + nw - 1) // nw}", "waves_per_workgroup": nw,
                           "tile_rows_per_wave": tk, "split": {4: "half block", 8: "one block"}.get(tk, f"{tk // 8} blocks"),
                           "reduction": "accumulators" if atomic else "partial rows"}

    # ---- roofline of the dominant kernel: the one-launch layer kernel (input
    # Hadamard + decode GEMV + split reduction + output Hadamard). The timed step is
    # four launches of it and nothing else, so its average launch duration over the
    # timed region is the HIP-event time of the region / (4 * steps), and achieved =
    # weight bytes of a step / event time of a step. rocprofv3's per-dispatch durations
    # of the same four launches add up to the same figure (profiles/).
    # per_linear: each launch shape on its own, two HIP events around back-to-back
    # replays of a graph that holds at least 32 launches walking over enough seeded
    # copies of that linear (>= 320 MB) that no launch finds its weights in the 256 MB
    # last-level cache. In such a run of identical launches gate+up takes about 4 us
    # longer than inside the step (34.7 vs 30.2 us median by a kernel trace of the same
    # process; the other three shapes 0.1-0.6 us), so the sum of the per_linear figures
    # is above the step time.
    per_linear = {}
    tot_bytes = tot_ms = 0.0
    for j, (name, n_in, outs) in enumerate(LAYER):
        ms = _launch_ms(layers[0][j], xs[n_in], K_BITS, dev)
        nb = layers[0][j].bytes
        per_linear[name] = {"MB": round(nb / 1e6, 2), "us": round(ms * 1e3, 2),
                            "GBps": round(nb / ms / 1e6, 1)}
        tot_bytes += nb
        tot_ms += ms
    isolated = tot_bytes / tot_ms / 1e6
    achieved = bytes_per_step / event_ms_per_step / 1e6
    roofline = {
        "bound": "hbm",
        "kernel": "linear_small_kernel<K=4, cb=3INST, rows=1>",
        "achieved": round(achieved, 1),
        "peak": HBM_PEAK_GBS,
        "unit": "GB/s",
        "frac": round(achieved / HBM_PEAK_GBS, 4),
        "traffic": TRAFFIC_BYTES_PER_STEP,
        "traffic_per_launch": TRAFFIC_BYTES_PER_STEP // 4,
        "traffic_source": "profiles/linear_small_k4_config2_pmc.txt (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this "
                          "script, scaled by a 64 MiB copy); a constant, not measured in this run",
        "bytes_per_launch": "in*out*K/8 of the launch's linear(s): 45.2 MB on average over the four launches of a "
                            "step; achieved = weight bytes of a step / HIP-event time of a step over the timed region "
                            "(= bytes per launch / average launch duration); traffic = HBM bytes of the same four "
                            "launches (FETCH_SIZE + WRITE_SIZE)",
        "avg_launch_us": round(event_ms_per_step * 1e3 / len(LAYER), 2),
        "event_ms_per_step": round(event_ms_per_step, 5),
        "per_linear": per_linear,
        "per_linear_note": "each launch shape replayed on its own (>= 32 identical launches per graph, cold weights); "
                           "gate_up runs about 4 us longer that way than inside the step",
        "achieved_from_per_linear": round(isolated, 1),
    }

    ceilings = bench_ceilings(dev)
    roofline["measured_peak"] = ceilings["stream_read_GBps"]
    roofline["frac_of_measured_peak"] = round(achieved / ceilings["stream_read_GBps"], 4)
    roofline["decode_loop_ceiling_GBps"] = ceilings["decode_loop"]["k4_3inst_cold"]["GBps"]
    roofline["frac_of_decode_loop_ceiling"] = round(
        achieved / ceilings["decode_loop"]["k4_3inst_cold"]["GBps"], 4)
    extras = {"ceilings": ceilings}
    if not args.skip_extras:
        extras.update(bench_batch_rows(dev, layers[0]))
        extras.update(bench_config1(dev))
        extras.update(bench_prefill(dev, layers[0], xs))
        extras.update(bench_moe(dev))
        extras.update(bench_encoder(dev))
        extras.update(bench_sweep(dev, layers[0]))

    out = {
        "metric": "EXL3 GEMV effective GB/s (% HBM peak) at bs1; prefill GEMM TFLOPS at M=2048",
        "value": round(value, 1),
        "unit": "GB/s",
        "pct_hbm_peak": round(100 * value / HBM_PEAK_GBS, 2),
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "ms_per_step_samples": [round(v, 5) for v in samples],
        "eager_ms_per_step": round(eager_ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "dtype_note": "K-bit trellis codes decoded to f16 weights (u32 integer decode), f16 activations, f32 accumulate",
        "data": "synthetic (seeded random trellis words, +-1 signs, N(0,1) fp16 activations)",
        "config": {
            "workload": "configs[1]: 27B-class dense decoder linears at batch 1, K=4, 3INST; "
                        "one step = " + ", ".join(n for n, _, _ in LAYER) + " of one layer",
            "bytes_per_step": bytes_per_step,
            "weight_copies_rotated": n_layers,
            "launch": (f"hip-graph replay, {n_layers} layer steps per graph" if graph_all is not None
                       else "eager"),
        },
        "launch_plans": plans,
        "roofline": roofline,
    }
    out.update(extras)
    if not args.skip_cpu:
        out["cpu_baseline"] = cpu_baseline()
    print(json.dumps(out))


def _time_ms(fn, reps, warm=3):
    import torch

    for _ in range(warm):
        fn()
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(reps)]
    torch.cuda.synchronize()
    for a, b in evs:
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    return float(np.mean([a.elapsed_time(b) for a, b in evs]))


def _launch_ms(lin, x, k, dev, cb=CB, min_bytes=320e6, reps=20):
    """Mean duration of one layer-kernel launch of the linear `lin` (its shape,
    signs and sibling table) with K = k on cold weights: one graph that walks over
    the seeded weight copies (>= min_bytes in all, so that no launch finds its
    weights in the last-level cache) often enough to hold at least 32 launches (the
    cost of replaying a graph is then a small share of a launch), replayed back to
    back between two HIP events."""
    import torch

    from ponyexl3_amd import ops

    nbytes = lin.n_in * lin.n_out * k // 8
    copies = max(2, int(np.ceil(min_bytes / nbytes)))
    gen = torch.Generator(device=dev).manual_seed(31_000 + lin.n_in + lin.n_out + k)
    trs = [torch.randint(-32768, 32768, (lin.n_in // 16, lin.n_out // 16, 16 * k), dtype=torch.int16,
                         device=dev, generator=gen) for _ in range(copies)]
    call = lambda tr: ops.linear_forward(x, tr, k, cb, lin.suh, lin.svh, None, lin.group_sub,
                                         member_out=lin.outs if lin.members > 1 else None,
                                         block_sub=lin.block_sub)
    for tr in trs:
        call(tr)
    torch.cuda.synchronize()
    cycles = max(1, int(np.ceil(32 / copies)))
    gr = torch.cuda.CUDAGraph()
    with torch.cuda.graph(gr):
        keep = [call(tr) for _ in range(cycles) for tr in trs]
    ms = _time_batch_ms(gr.replay, reps=max(4, reps // cycles), warm=3) / (copies * cycles)
    del gr, keep, trs
    return ms


def _time_batch_ms(fn, reps, warm=10):
    """Mean time of back-to-back calls (the queue never drains, so launch latency
    of an idle device is not part of it)."""
    import torch

    for _ in range(warm):
        fn()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    a.record()
    for _ in range(reps):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / reps


def _rows_x(n, rows, dev):
    import torch

    g = torch.Generator().manual_seed(4321 + n + rows)
    return torch.randn((rows, n), generator=g).to(torch.float16).to(dev)


def bench_ceilings(dev):
    """What this GPU delivers, measured in the same run: a streaming read of cold
    memory (the denominator next to the published 8 TB/s), and the small-batch
    kernels' inner loop on its own (wave-wide load, per-lane decode of 32 codewords,
    16 matrix-pipe dot products; one workgroup of 16 waves per CU, 128 tile rows per
    wave, no Hadamard, no reduction): the rate the VALU instruction sequence of the
    bit-exact decode allows before any layer structure is added. 'cold' walks over a
    2 GiB buffer so that every launch reads memory no earlier launch of the
    measurement touched; 'cache' re-reads one 32 MiB slice."""
    import ctypes

    import torch

    from ponyexl3_amd import _lib

    lib = _lib.load_diag()
    main_lib = _lib.load()
    total = 2 << 30
    buf = torch.randint(-2**31, 2**31 - 1, (total // 4,), dtype=torch.int32, device=dev)
    out = torch.zeros(4096 * 1024, dtype=torch.float32, device=dev)
    stream = lambda: ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    ptr = lambda off: ctypes.c_void_p(buf.data_ptr() + off)
    n_cu = torch.cuda.get_device_properties(dev).multi_processor_count

    def timed(launches):
        """mean ms per launch of a list of launch thunks, run back to back twice
        (first pass warms code and TLBs) between two events"""
        for fn in launches:
            fn()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        a.record()
        for fn in launches:
            fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / len(launches)

    def timed_graph(launches):
        """mean ms per launch of the thunks captured into one HIP graph and replayed"""
        for fn in launches:
            fn()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for fn in launches:
                fn()
        g.replay()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        a.record()
        g.replay()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / len(launches)

    chunk = 512 << 20
    read = [(lambda o=o: _lib.check(lib.exl3_diag_stream_read(ptr(o), chunk, ctypes.c_void_p(out.data_ptr()), stream()),
                                    "exl3_diag_stream_read")) for o in range(0, total, chunk)]
    ms = timed(read)
    res = {"stream_read_GBps": round(chunk / ms / 1e6, 1), "stream_read_chunk_MB": chunk >> 20,
           "published_peak_GBps": HBM_PEAK_GBS}
    steps = 128
    loops = {}
    for tag, k, cb, cold in (("k4_3inst_cold", 4, 0, True), ("k4_3inst_cache", 4, 0, False),
                             ("k4_mcg_cold", 4, 1, True), ("k2_3inst_cold", 2, 0, True),
                             ("k8_3inst_cold", 8, 0, True)):
        per_launch = n_cu * 16 * steps * 256 * k  # bytes one launch walks over
        offs = list(range(0, total - per_launch + 1, per_launch)) if cold else [0] * 8
        size = per_launch if cold else 32 << 20
        calls = [(lambda o=o: _lib.check(lib.exl3_diag_decode_loop(ptr(o), size, k, cb, n_cu, steps,
                                                                     ctypes.c_void_p(out.data_ptr()), stream()),
                                         "exl3_diag_decode_loop")) for o in offs]
        ms = timed(calls)
        weights = n_cu * 16 * steps * 2048
        loops[tag] = {"us_per_launch": round(ms * 1e3, 1), "Tweights_per_s": round(weights / ms / 1e9, 2),
                      "GBps": round(weights * k / 8 / ms / 1e6, 1),
                      "frac_hbm_peak": round(weights * k / 8 / ms / 1e6 / HBM_PEAK_GBS, 4)}
    res["decode_loop"] = loops
    res["decode_loop_note"] = ("n_cu workgroups x 16 waves x 128 tile rows per launch, launch overhead included "
                               "(about 10 % of a launch)")
    # The phases of a layer-kernel launch that no decoding overlaps, on the four grids of
    # the timed step (K=4, one row): dispatch of the grid alone, and dispatch + every
    # wave's first four tile rows arriving from cold memory.
    phases = {}
    n_rows = total // (256 * K_BITS)
    grids = []
    for name, n_in, outs in LAYER:  # the grids the host plans for these launches
        v = [ctypes.c_int() for _ in range(4)]
        _lib.check(main_lib.exl3_linear_plan(1, n_in // 16, sum(outs) // 16, K_BITS, *[ctypes.byref(c) for c in v]),
                   "exl3_linear_plan")
        splits, _, nw, _ = (c.value for c in v)
        grids.append((name, sum(outs) // 128, (splits + nw - 1) // nw, nw * 64))
    for name, gx, gy, threads in grids:
        waves = gx * gy * threads // 64
        empty = [(lambda: _lib.check(lib.exl3_diag_empty_launch(gx, gy, threads, stream()),
                                     "exl3_diag_empty_launch"))] * 64
        stride = max(waves * 4, n_rows // 64)
        first = [(lambda i=i: _lib.check(lib.exl3_diag_first_rows(ptr(0), total, K_BITS, gx, gy, threads,
                                                                   (i * stride) % n_rows,
                                                                   ctypes.c_void_p(out.data_ptr()), stream()),
                                         "exl3_diag_first_rows")) for i in range(64)]
        phases[name] = {"grid": f"{gx}x{gy}x{threads}", "dispatch_us": round(timed_graph(empty) * 1e3, 2),
                        "dispatch_and_first_rows_us": round(timed_graph(first) * 1e3, 2)}
    res["launch_phases"] = phases
    res["launch_phases_note"] = "64 launches back to back inside one HIP graph (device-side rate, no host launch cost)"
    del buf, out
    return res


def bench_batch_rows(dev, layer):
    """The same layer step at 2 .. 128 rows (batched decode, speculative verify):
    sum of the launch durations on cold weights (9..32 rows: each linear is the
    input rotation launch plus the medium-batch kernel; above that the rotation, the
    prefill GEMM with every tile split and its fix-up pass)."""
    res = {}
    total = sum(l.bytes for l in layer)
    for rows in (2, 4, 8, 16, 32, 64, 128):
        ms = sum(_launch_ms(lin, _rows_x(lin.n_in, rows, dev), K_BITS, dev) for lin in layer)
        res[f"rows_{rows}"] = {"us_per_step": round(ms * 1e3, 2), "GBps": round(total / ms / 1e6, 1)}
    return {"batch_rows": res}


def bench_config1(dev):
    """config 1: one 4096 -> 4096 linear, K=4, 3INST, one row."""
    lin = DeviceLinear("cfg1", 4096, [4096], 10_004, dev)
    ms = _launch_ms(lin, _rows_x(4096, 1, dev), K_BITS, dev)
    return {"config1": {"MB": round(lin.bytes / 1e6, 2), "us": round(ms * 1e3, 2),
                        "GBps": round(lin.bytes / ms / 1e6, 1)}}


def bench_sweep(dev, layer, ks=(2, 3, 5, 6, 8), row_counts=(1, 4, 8)):
    """config 5: the config-2 layer at K in {2,3,5,6,8} x {3INST, MCG} x 1/4/8 rows."""
    res = {}
    for k in ks:
        total = sum(l.n_in * l.n_out * k // 8 for l in layer)
        for cb, cbn in ((0, "3inst"), (1, "mcg")):
            for rows in row_counts:
                ms = sum(_launch_ms(lin, _rows_x(lin.n_in, rows, dev), k, dev, cb=cb) for lin in layer)
                res[f"k{k}_{cbn}_rows{rows}"] = {"us_per_step": round(ms * 1e3, 2),
                                                 "GBps": round(total / ms / 1e6, 1)}
                print(f"sweep k={k} {cbn} rows={rows}: {ms * 1e3:.1f} us/step, {total / ms / 1e6:.0f} GB/s",
                      file=sys.stderr, flush=True)
    return {"config5": res}


def bench_prefill(dev, layer, xs):
    """config 3: M=2048 prefill GEMM on the config-2 weights (MFMA kernel alone)."""
    import torch

    from ponyexl3_amd import ops

    g = torch.Generator().manual_seed(77)
    per = {}
    flop = ms_tot = ms_layer_tot = 0.0
    for lin in layer:
        xh = torch.randn((2048, lin.n_in), generator=g).to(torch.float16).to(dev)
        # calls queued back to back (the device never waits for the host between them), as the
        # layers of a prefill chunk are
        ms = _time_batch_ms(lambda: ops.inner_gemm(xh, lin.trellis, K_BITS, CB), reps=10, warm=3)
        # the whole layer at 2048 rows: input rotation, GEMM with the output transform in its
        # epilogue (split tiles: in the pass that adds their partial tiles)
        ms_layer = _time_batch_ms(lambda: lin.forward(xh), reps=10, warm=3)
        f = 2.0 * 2048 * lin.n_in * lin.n_out
        per[lin.name] = {"ms": round(ms, 4), "TFLOPs": round(f / ms / 1e9, 1),
                         "layer_ms": round(ms_layer, 4), "layer_TFLOPs": round(f / ms_layer / 1e9, 1)}
        flop += f
        ms_tot += ms
        ms_layer_tot += ms_layer
        del xh
    tf = flop / ms_tot / 1e9
    # context: what a plain fp16 GEMM of the library reaches on this box at the gate+up shape
    a = torch.randn((2048, 5120), generator=g).to(torch.float16).to(dev)
    b = torch.randn((5120, 34816), generator=g).to(torch.float16).to(dev)
    ms_lib = _time_batch_ms(lambda: torch.matmul(a, b), reps=10, warm=3)
    lib_tf = 2.0 * 2048 * 5120 * 34816 / ms_lib / 1e9
    del a, b
    return {"prefill_gemm": {"M": 2048, "TFLOPs": round(tf, 1), "peak": MFMA_F16_PEAK_TFLOPS,
                             "layer_TFLOPs_with_hadamards": round(flop / ms_layer_tot / 1e9, 1),
                             "library_fp16_gemm_TFLOPs_gate_up_shape": round(lib_tf, 1),
                             "frac": round(tf / MFMA_F16_PEAK_TFLOPS, 4),
                             "layer_frac": round(flop / ms_layer_tot / 1e9 / MFMA_F16_PEAK_TFLOPS, 4),
                             "bound": "mfma", "kernel": "gemm_kernel<K=4, cb=3INST>",
                             "timing": "HIP events around ten calls queued back to back",
                             "per_linear": per}}


def bench_encoder(dev):
    """Encoder side: tail-biting trellis search over 4096 tiles of N(0, 1.24^2)
    targets (a 1024 x 1024 matrix) at K = 4, MCG, plus the symbol packer. Every step
    of the search evaluates all 65536 codewords, 2 x 256 steps per tile; the kernel
    spends five VALU instructions per evaluation."""
    import torch

    from ponyexl3_amd import search

    n, k = 4096, 4
    gen = torch.Generator(device=dev).manual_seed(50_004)
    tiles = torch.randn((n, 256), device=dev, generator=gen) * 1.24371088
    search.quantize_tiles(tiles[:64], k, 1)
    keep = {}

    def run():
        keep["q"], keep["idx"] = search.quantize_tiles(tiles, k, 1)

    ms = _time_ms(run, reps=3, warm=1)
    mse = float(((keep["q"] - tiles) ** 2).mean())
    evals = n * 2 * 256 * 65536
    sym = keep["idx"] & ((1 << k) - 1)
    pack_ms = _time_ms(lambda: search.pack_trellis(sym, k), reps=10, warm=2)
    return {"encoder": {"workload": f"{n} tiles, K={k}, MCG", "ms": round(ms, 2),
                        "tiles_per_s": round(n / ms * 1e3), "Mweights_per_s": round(n * 256 / ms / 1e3, 1),
                        "T_evals_per_s": round(evals / ms / 1e9, 2),
                        "T_valu_lane_ops_per_s": round(5 * evals / ms / 1e9, 1),
                        "mse": round(mse, 5), "pack_trellis_us": round(pack_ms * 1e3, 1)}}


def bench_moe(dev):
    """config 4: A3B-style routed experts, top-8 of 256, at 1, 8 and 32 tokens (from
    16 tokens on the slots of one expert share a pass over its weights) and 512
    tokens through the prefill path."""
    import torch

    from ponyexl3_amd import EXL3SwitchGLU, ops
    from ponyexl3_amd.moe import route_topk

    E, D, H, kk = 256, 2048, 512, 8
    copies = 2  # 2 x 403 MB of expert weights: more than the last-level cache
    rng = np.random.default_rng(40_004)
    moes = []
    for c in range(copies):
        gen = torch.Generator(device=dev).manual_seed(40_004 + c)
        rnd = lambda *s: torch.randint(-32768, 32768, s, dtype=torch.int16, device=dev, generator=gen)
        sgn = lambda *s: (torch.randint(0, 2, s, device=dev, generator=gen) * 2 - 1).to(torch.float16)
        moes.append(EXL3SwitchGLU(
            gu_trellis=rnd(D // 16, E * 2 * H // 16, 16 * K_BITS), gu_suh=sgn(E, 2, D), gu_svh=sgn(E, 2 * H),
            dn_trellis=rnd(H // 16, E * D // 16, 16 * K_BITS), dn_suh=sgn(E, H), dn_svh=sgn(E, D),
            k=K_BITS, cb=CB))
    res = {}
    per_graph = 32  # chains per graph, each with its own routing, alternating weight copies
    for T in (1, 8, 32):
        x = torch.from_numpy((rng.standard_normal((1, T, D)) * 0.25).astype(np.float16)).to(dev)
        # Routing differs from chain to chain so that a replay streams far more expert
        # weights than the 256 MB last-level cache holds: at one token the 32 chains
        # of a graph use 32 disjoint top-8 sets (all 256 experts of both copies,
        # 2 x 403 MB); at eight tokens every chain draws fresh router logits.
        idxs, distinct = [], []
        perm = rng.permutation(E)
        for c in range(per_graph):
            if T == 1:
                inds = torch.from_numpy(perm[(c * kk) % E:(c * kk) % E + kk].astype(np.int32)).to(dev).reshape(1, kk)
            else:
                logits = torch.from_numpy(rng.standard_normal((T, E)).astype(np.float32)).to(dev)
                inds, _ = route_topk(logits, kk)
            distinct.append(int(torch.unique(inds).numel()))
            idxs.append(inds.reshape(1, T, kk).to(torch.int32).contiguous())
        for c in range(per_graph):  # warm-up outside any capture (workspaces, counters)
            moes[c % copies](x, idxs[c])
        torch.cuda.synchronize()
        launch = "eager"
        graph = None
        try:  # device time of the chain: replay it from a HIP graph like the decode step
            gr = torch.cuda.CUDAGraph()
            with torch.cuda.graph(gr):
                keep = [moes[c % copies](x, idxs[c]) for c in range(per_graph)]
            graph = (gr, keep)
            launch = f"hip-graph replay, {per_graph} chains per graph"
        except Exception as e:  # noqa: BLE001
            print(f"MoE graph capture failed ({e!r}); timing eager launches", file=sys.stderr)

        def fn():
            if graph is not None:
                graph[0].replay()
            else:
                for c in range(per_graph):
                    moes[c % copies](x, idxs[c])

        ms = _time_batch_ms(fn, reps=20, warm=3) / per_graph
        mean_distinct = float(np.mean(distinct))
        nbytes = mean_distinct * 3 * D * H * K_BITS // 8
        res[f"tokens_{T}"] = {"us": round(ms * 1e3, 2), "launch": launch,
                              "distinct_experts": round(mean_distinct, 1),
                              "MB": round(nbytes / 1e6, 2), "GBps": round(nbytes / ms / 1e6, 1),
                              "frac_hbm": round(nbytes / ms / 1e6 / HBM_PEAK_GBS, 4)}
    # prefill: 512 tokens through the sorted, segmented GEMM path (eager launches,
    # host-side sort and table ops included)
    T = 512
    x = torch.from_numpy((rng.standard_normal((1, T, D)) * 0.25).astype(np.float16)).to(dev)
    logits = torch.from_numpy(rng.standard_normal((T, E)).astype(np.float32)).to(dev)
    inds, _ = route_topk(logits, kk)
    idx = inds.reshape(1, T, kk).to(torch.int32).contiguous()
    it = [0]

    def prefill():
        moes[it[0] % copies](x, idx)
        it[0] += 1

    ms = _time_batch_ms(prefill, reps=10, warm=3)
    flop = 2.0 * T * kk * 3 * D * H
    res["tokens_512_prefill"] = {"ms": round(ms, 4), "TFLOPs": round(flop / ms / 1e9, 1),
                                 "expert_weights_MB": round(E * 3 * D * H * K_BITS / 8 / 1e6, 1)}
    return {"moe": res}


if __name__ == "__main__":
    main()
