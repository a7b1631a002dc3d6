// Routed MoE expert chain for a handful of tokens (decode / speculative verify):
// per slot (token t, expert e) gate and up GEMVs, GLU, down GEMV, each an EXL3
// linear with its own suh/svh. Only the selected experts' tile columns of the
// stacked trellises are read: the GEMV kernel is pointed at them through
// per-group tables built on the device from the routing indices.
//
// Two launches when the caller provides zeroed counters:
//   A. moe_gateup_kernel    per (slot, gate|up, 128 columns of H): input rotation
//                           in the wave, decode GEMV over D, workgroup sum; the
//                           last workgroup of a (slot, column block) adds the
//                           partial rows of gate and up, applies post-Hadamard,
//                           svh and the GLU and rotates the block for the down
//                           projection (a Hadamard block of H is exactly one
//                           128-column group of gate/up)
//   B. moe_down_kernel      per (slot, 128 columns of D): decode GEMV over H on
//                           the rotated block, sum, post-Hadamard, svh
//   (four waves per workgroup, one Hadamard block of the reduction each; with few
//   slots eight waves on half a block each, which doubles the loads in flight)
//   With several tokens and enough slots per expert (moe_*_grouped_kernel) the slots
//   that route to one expert share a pass over its weights, four batch rows at a time.
// Without counters the same result comes from a chain of five launches:
//   1. moe_prep_kernel      rotated activations per (slot, proj) + group tables
//   2. gemv_kernel          gate/up partial sums, fp32
//   3. moe_glu_kernel       split reduction, post-Hadamard, svh, GLU, then the
//                           down projection's input rotation
//   4. gemv_kernel          down partial sums
//   5. moe_finish_kernel    split reduction, post-Hadamard, per-expert svh
//
// Semantics follow the unfused chain of ponyexl3/mlx/exl3_moe.py:648-682 with
// the casts of ponyexl3/ref/forward.py:34,41,42; the Metal A2/B2 kernels
// (ponyexl3/mlx/exl3_moe.py:345-422) are what this replaces.
#include "exl3_device.hpp"
#include "exl3_host.hpp"
#include "exl3_small.hpp"

#include <algorithm>
#include <type_traits>

#pragma clang fp contract(off)

namespace exl3 {

// Routing indices come from the caller's device memory; an out-of-range value is
// clamped so that it can never turn into an out-of-bounds read.
__device__ __forceinline__ int clamp_expert(int e, int E) { return e < 0 ? 0 : (e >= E ? E - 1 : e); }

// xh_gu[s][p][:] = fp16(had(x[t] * gu_suh[e][p])); also fills the group tables:
//   gate/up GEMV group (s, p, hg): sub = 2s+p, tile = (p*E + e)*(H/16) + 8*hg
//   down GEMV group (s, og):       sub = s,    tile = e*(D/16) + 8*og
__global__ __launch_bounds__(256) void moe_prep_kernel(
    const half_t* __restrict__ x, const int* __restrict__ indices,
    const half_t* __restrict__ gu_suh, half_t* __restrict__ xh_gu, int* __restrict__ gu_sub,
    int* __restrict__ gu_tile, int* __restrict__ dn_sub, int* __restrict__ dn_tile, int slots,
    int top_k, int E, int D, int H) {
    const int lane = threadIdx.x & 63;
    const int dblocks = D >> 7, hblocks = H >> 7;
    const int wave_id = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int gtid = blockIdx.x * 256 + threadIdx.x;
    if (gtid < slots * 2 * hblocks) {
        const int hg = gtid % hblocks, sp = gtid / hblocks;
        const int e = clamp_expert(indices[sp >> 1], E);
        gu_sub[gtid] = sp;
        gu_tile[gtid] = ((sp & 1) * E + e) * (H >> 4) + 8 * hg;
    }
    if (gtid < slots * dblocks) {
        const int og = gtid % dblocks, s = gtid / dblocks;
        dn_sub[gtid] = s;
        dn_tile[gtid] = clamp_expert(indices[s], E) * (D >> 4) + 8 * og;
    }
    if (wave_id >= slots * 2 * dblocks) return;
    const int blk = wave_id % dblocks;
    const int sp = wave_id / dblocks;
    const int s = sp >> 1, p = sp & 1;
    const int t = s / top_k;
    const int e = clamp_expert(indices[s], E);
    const half2_t xv = *reinterpret_cast<const half2_t*>(x + (size_t)t * D + blk * 128 + 2 * lane);
    const half2_t sv = *reinterpret_cast<const half2_t*>(gu_suh + ((size_t)e * 2 + p) * D +
                                                         blk * 128 + 2 * lane);
    float a = (float)xv.x * (float)sv.x, b = (float)xv.y * (float)sv.y;
    wht128_lanes(a, b, lane);
    half2_t o;
    o.x = (half_t)(a * kHadScaleF);
    o.y = (half_t)(b * kHadScaleF);
    *reinterpret_cast<half2_t*>(xh_gu + (size_t)sp * D + blk * 128 + 2 * lane) = o;
}

__device__ __forceinline__ float glu_act(float g, float u, int activation) {
    if (activation == 1) {
        const float t = 0.797884560803f * (g + 0.044715f * g * g * g);
        return 0.5f * g * (1.0f + tanhf(t)) * u;
    }
    return (g / (1.0f + expf(-g))) * u;
}

// One wave per (slot, 128-block of H): finishes gate and up, applies the GLU and
// rotates the result for the down projection.
__global__ __launch_bounds__(256) void moe_glu_kernel(
    const float* __restrict__ partial, int n_splits, size_t split_stride,
    const int* __restrict__ indices, const half_t* __restrict__ gu_svh,
    const half_t* __restrict__ dn_suh, half_t* __restrict__ xh_dn, int slots, int H, int E,
    int activation) {
    const int lane = threadIdx.x & 63;
    const int hblocks = H >> 7;
    const int wave_id = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (wave_id >= slots * hblocks) return;
    const int blk = wave_id % hblocks, s = wave_id / hblocks;
    const int e = clamp_expert(indices[s], E);
    float v[2][2];
#pragma unroll
    for (int p = 0; p < 2; p++) {
        // partial layout: [split][(s*2+p)*H + h]
        const size_t off = ((size_t)s * 2 + p) * H + blk * 128 + 2 * lane;
        float2_t acc = *reinterpret_cast<const float2_t*>(partial + off);
        for (int i = 1; i < n_splits; i++) {
            const float2_t q = *reinterpret_cast<const float2_t*>(partial + i * split_stride + off);
            acc.x = acc.x + q.x;
            acc.y = acc.y + q.y;
        }
        float a = (float)(half_t)acc.x, b = (float)(half_t)acc.y;
        wht128_lanes(a, b, lane);
        const half2_t sv = *reinterpret_cast<const half2_t*>(gu_svh + (size_t)e * 2 * H + p * H +
                                                             blk * 128 + 2 * lane);
        v[p][0] = (float)(half_t)(a * kHadScaleF * (float)sv.x);
        v[p][1] = (float)(half_t)(b * kHadScaleF * (float)sv.y);
    }
    const float h0 = (float)(half_t)glu_act(v[0][0], v[1][0], activation);
    const float h1 = (float)(half_t)glu_act(v[0][1], v[1][1], activation);
    const half2_t ds =
        *reinterpret_cast<const half2_t*>(dn_suh + (size_t)e * H + blk * 128 + 2 * lane);
    float a = h0 * (float)ds.x, b = h1 * (float)ds.y;
    wht128_lanes(a, b, lane);
    half2_t o;
    o.x = (half_t)(a * kHadScaleF);
    o.y = (half_t)(b * kHadScaleF);
    *reinterpret_cast<half2_t*>(xh_dn + (size_t)s * H + blk * 128 + 2 * lane) = o;
}

__global__ __launch_bounds__(256) void moe_finish_kernel(
    const float* __restrict__ partial, int n_splits, size_t split_stride,
    const int* __restrict__ indices, const half_t* __restrict__ dn_svh, half_t* __restrict__ y,
    int slots, int D, int E) {
    const int lane = threadIdx.x & 63;
    const int dblocks = D >> 7;
    const int wave_id = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (wave_id >= slots * dblocks) return;
    const int blk = wave_id % dblocks, s = wave_id / dblocks;
    const int e = clamp_expert(indices[s], E);
    const size_t off = (size_t)s * D + blk * 128 + 2 * lane;
    float2_t acc = *reinterpret_cast<const float2_t*>(partial + off);
    for (int i = 1; i < n_splits; i++) {
        const float2_t q = *reinterpret_cast<const float2_t*>(partial + i * split_stride + off);
        acc.x = acc.x + q.x;
        acc.y = acc.y + q.y;
    }
    float a = (float)(half_t)acc.x, b = (float)(half_t)acc.y;
    wht128_lanes(a, b, lane);
    const half2_t sv =
        *reinterpret_cast<const half2_t*>(dn_svh + (size_t)e * D + blk * 128 + 2 * lane);
    half2_t o;
    o.x = (half_t)(a * kHadScaleF * (float)sv.x);
    o.y = (half_t)(b * kHadScaleF * (float)sv.y);
    *reinterpret_cast<half2_t*>(y + off) = o;
}


// ---------------------------------------------------------------------------
// Fused chain: shared tail of both kernels. The NW waves of a workgroup are
// added through LDS in wave order; returns the two sums of this lane's columns
// (2*lane, 2*lane+1) to wave 0.
template <int NW>
__device__ __forceinline__ float2_t moe_wg_sum(float (*red)[128], const float (&acc)[1][2],
                                               int lane, int wave) {
    const int c0 = (lane >> 3) * 16 + (lane & 7);
    red[wave][c0] = acc[0][0];
    red[wave][c0 + 8] = acc[0][1];
    __syncthreads();
    float2_t v{red[0][2 * lane], red[0][2 * lane + 1]};
#pragma unroll
    for (int w = 1; w < NW; w++) {
        v.x = __fadd_rn(v.x, red[w][2 * lane]);
        v.y = __fadd_rn(v.y, red[w][2 * lane + 1]);
    }
    return v;
}

// Partial rows cross workgroups through device-scope accesses only (the XCDs'
// L2 caches are not coherent with each other): store, wait, bump the counter;
// the workgroup that sees `expected - 1` is the last one and reads them back.
__device__ __forceinline__ bool moe_publish(float* row, float2_t v, int* counter, int expected,
                                            int lane) {
    __hip_atomic_store(reinterpret_cast<uint64_t*>(row + 2 * lane),
                       __builtin_bit_cast(uint64_t, v), __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    int seen = 0;
    if (lane == 0)
        seen = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return __shfl(seen, 0, kWave) == expected - 1;
}

// Eight partial rows in flight (a batch that runs past the last row re-reads that row and
// drops it, so that every batch is one round trip); added in index order.
__device__ __forceinline__ float2_t moe_sum_rows(const float* rows, int n, int lane) {
    float a = 0.f, b = 0.f;
    for (int s = 0; s < n; s += 8) {
        uint64_t v[8];
#pragma unroll
        for (int i = 0; i < 8; i++)
            v[i] = __hip_atomic_load(
                reinterpret_cast<const uint64_t*>(rows + (size_t)min(s + i, n - 1) * 128 + 2 * lane),
                __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
        for (int i = 0; i < 8; i++) {
            if (s + i < n) {
                const float2_t f = __builtin_bit_cast(float2_t, v[i]);
                a = __fadd_rn(a, f.x);
                b = __fadd_rn(b, f.y);
            }
        }
    }
    return float2_t{a, b};
}

// fp16(had128(fp16(sum)) / sqrt(128) * sv): the finish of one EXL3 linear on one
// 128-column block (ponyexl3/ref/forward.py:41-42).
__device__ __forceinline__ void moe_finish_block(float2_t sum, half2_t sv, int lane, float& o0,
                                                 float& o1) {
    float a = (float)(half_t)sum.x, b = (float)(half_t)sum.y;
    wht128_lanes(a, b, lane);
    o0 = (float)(half_t)(a * kHadScaleF * (float)sv.x);
    o1 = (float)(half_t)(b * kHadScaleF * (float)sv.y);
}

// grid = (slots * 2 * H/128, ceil((D/128) / 4)); wave w of workgroup (gid, q) owns
// the Hadamard block 4q + w of D for slot s = gid / (2*hblocks), projection
// p = (gid / hblocks) & 1 and column block hg = gid % hblocks.
// part: fp32 [gid][n_wg][128]; counters[s*hblocks + hg] count 2*n_wg workgroups.
template <int K, int CB, int NW>
__global__ __launch_bounds__(NW * 64) void moe_gateup_kernel(
    const uint32_t* __restrict__ gu_trellis, const half_t* __restrict__ x,
    const int* __restrict__ indices, const half_t* __restrict__ gu_suh,
    const half_t* __restrict__ gu_svh, const half_t* __restrict__ dn_suh, half_t* xh_dn,
    float* part, int* counters, int top_k, int E, int D, int H, int activation) {
    __shared__ __attribute__((aligned(16))) half_t xs[NW][1][kXwLd];
    __shared__ float red[NW][128];
    __shared__ float up_val[128];
    __shared__ int last_flag;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int dblocks = D >> 7, hblocks = H >> 7;
    const int n_wg = gridDim.y;
    const int gid = blockIdx.x;
    const int hg = gid % hblocks, sp = gid / hblocks;
    const int s = sp >> 1, p = sp & 1;
    const int e = clamp_expert(indices[s], E);
    constexpr bool kHalf = NW == 8;
    const int part_idx = blockIdx.y * NW + wave;
    const int blk = kHalf ? part_idx >> 1 : part_idx;
    const int tk0 = blk * 8 + (kHalf ? (part_idx & 1) * 4 : 0);
    float acc[1][2] = {{0.f, 0.f}};
    if (blk < dblocks) {
        const size_t row_words = (size_t)E * 2 * (H >> 4) * (8 * K);
        const uint32_t* base =
            gu_trellis + ((size_t)(p * E + e) * (H >> 4) + 8 * hg) * (8 * K) + lane * K;
        stream_block_rows<K, CB, 1, true, kHalf, true>(base, row_words, tk0, tk0 + (kHalf ? 4 : 8),
                                                 x + (size_t)(s / top_k) * D, (size_t)D, 1,
                                                 gu_suh + ((size_t)e * 2 + p) * D, xs[wave], lane,
                                                 acc);
    }
    const float2_t v = moe_wg_sum<NW>(red, acc, lane, wave);
    int* counter = counters + s * hblocks + hg;
    if (wave == 0) {
        const bool last = moe_publish(part + ((size_t)gid * n_wg + blockIdx.y) * 128, v, counter,
                                      2 * n_wg, lane);
        if (lane == 0) last_flag = last;
    }
    __syncthreads();
    if (!last_flag) return;
    asm volatile("" ::: "memory");
    // waves 0 and 1 finish gate and up, wave 0 then applies the GLU and rotates
    float f0 = 0.f, f1 = 0.f;
    if (wave < 2) {
        const int gid_p = (s * 2 + wave) * hblocks + hg;
        const float2_t sum = moe_sum_rows(part + (size_t)gid_p * n_wg * 128, n_wg, lane);
        const half2_t sv = *reinterpret_cast<const half2_t*>(
            gu_svh + (size_t)e * 2 * H + wave * H + hg * 128 + 2 * lane);
        moe_finish_block(sum, sv, lane, f0, f1);
        if (wave == 1) {
            up_val[2 * lane] = f0;
            up_val[2 * lane + 1] = f1;
        }
    }
    __syncthreads();
    if (wave != 0) return;
    const float h0 = (float)(half_t)glu_act(f0, up_val[2 * lane], activation);
    const float h1 = (float)(half_t)glu_act(f1, up_val[2 * lane + 1], activation);
    const half2_t ds =
        *reinterpret_cast<const half2_t*>(dn_suh + (size_t)e * H + hg * 128 + 2 * lane);
    float a = h0 * (float)ds.x, b = h1 * (float)ds.y;
    wht128_lanes(a, b, lane);
    half2_t o;
    o.x = (half_t)(a * kHadScaleF);
    o.y = (half_t)(b * kHadScaleF);
    *reinterpret_cast<half2_t*>(xh_dn + (size_t)s * H + hg * 128 + 2 * lane) = o;
    if (lane == 0) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Gate and up of one k-chunk in ONE workgroup of eight waves, reduced through 64-bit
// accumulators with returning atomics (see fix_word): waves 0..3 stream gate, waves
// 4..7 up, over the same Hadamard blocks of D - HALF: half a block each, two blocks
// per workgroup; else a block each, four blocks per workgroup. Wave 0 adds the
// workgroup's 128 gate sums and 128 up sums to the accumulators of (slot, column
// block); the workgroup whose add completes the first gate column is the finisher: it
// holds (or polls for, if other workgroups' adds were interleaved with its own) both
// totals, so it goes on to post-Hadamard, svh, GLU and the rotation for the down
// projection without another trip through memory. One round trip instead of the
// three of store / counter / reload.
// grid = (slots * H/128, chunks); sums: uint64 [slots][2][H], zero on entry and exit.
template <int K, int CB, bool HALF>
__global__ __launch_bounds__(512) void moe_gateup_pair_kernel(
    const uint32_t* __restrict__ gu_trellis, const half_t* __restrict__ x,
    const int* __restrict__ indices, const half_t* __restrict__ gu_suh,
    const half_t* __restrict__ gu_svh, const half_t* __restrict__ dn_suh, half_t* xh_dn,
    unsigned long long* sums, int top_k, int E, int D, int H, int activation, int* status,
    int spin_limit) {
    __shared__ __attribute__((aligned(16))) half_t xs[8][1][kXwLd];
    __shared__ float red[8][128];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int dblocks = D >> 7, hblocks = H >> 7;
    const int n_chunks = gridDim.y;
    const int gid = blockIdx.x;
    const int hg = gid % hblocks, s = gid / hblocks;
    const int p = wave >> 2, j = wave & 3;
    const int e = clamp_expert(indices[s], E);
    const int blk = HALF ? blockIdx.y * 2 + (j >> 1) : blockIdx.y * 4 + j;
    const int tk0 = blk * 8 + (HALF ? (j & 1) * 4 : 0);
    float acc[1][2] = {{0.f, 0.f}};
    if (blk < dblocks) {
        const size_t row_words = (size_t)E * 2 * (H >> 4) * (8 * K);
        const uint32_t* base =
            gu_trellis + ((size_t)(p * E + e) * (H >> 4) + 8 * hg) * (8 * K) + lane * K;
        stream_block_rows<K, CB, 1, true, HALF, true>(base, row_words, tk0, tk0 + (HALF ? 4 : 8),
                                                x + (size_t)(s / top_k) * D, (size_t)D, 1,
                                                gu_suh + ((size_t)e * 2 + p) * D, xs[wave], lane,
                                                acc);
    }
    const int c0 = (lane >> 3) * 16 + (lane & 7);
    red[wave][c0] = acc[0][0];
    red[wave][c0 + 8] = acc[0][1];
    __syncthreads();
    if (wave != 0) return;
    // word q of a lane: projection q >> 1, column 2*lane + (q & 1); wave order within a projection
    unsigned long long w[4];
    unsigned long long* slot[4];
#pragma unroll
    for (int q = 0; q < 4; q++) {
        const int col = 2 * lane + (q & 1), w0 = (q >> 1) * 4;
        float v = red[w0][col];
#pragma unroll
        for (int i = 1; i < 4; i++) v = __fadd_rn(v, red[w0 + i][col]);
        slot[q] = sums + ((size_t)s * 2 + (q >> 1)) * H + hg * 128 + col;
        const unsigned long long a = fix_word(v);
        w[q] = __hip_atomic_fetch_add(slot[q], a, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + a;
    }
    if (__builtin_amdgcn_readfirstlane(fix_count(w[0])) != n_chunks) return;
    auto all_complete = [&]() {
        bool ok = true;
#pragma unroll
        for (int q = 0; q < 4; q++) ok = ok && fix_count(w[q]) == n_chunks;
        return __ballot(ok) == ~0ull;
    };
    bool complete = all_complete();
    for (int spin = 0; !complete && spin < spin_limit; spin++) {
#pragma unroll
        for (int q = 0; q < 4; q++)
            w[q] = __hip_atomic_load(slot[q], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        complete = all_complete();
    }
    if (!complete) {
        // the counts never became complete (array not zero on entry, or shared with an
        // overlapping call): NaN for this block of the down projection's input (and so
        // for the slot's output), status word set, accumulators left for the caller to zero
        if (status && lane == 0)
            __hip_atomic_fetch_or(status, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        half2_t bad;
        bad.x = bad.y = bits_to_half(0x7E00);
        *reinterpret_cast<half2_t*>(xh_dn + (size_t)s * H + hg * 128 + 2 * lane) = bad;
        return;
    }
#pragma unroll
    for (int q = 0; q < 4; q++)
        __hip_atomic_store(slot[q], 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const half_t* svh_e = gu_svh + (size_t)e * 2 * H + hg * 128 + 2 * lane;
    float g0, g1, u0, u1;
    moe_finish_block(float2_t{fix_value(w[0]), fix_value(w[1])},
                     *reinterpret_cast<const half2_t*>(svh_e), lane, g0, g1);
    moe_finish_block(float2_t{fix_value(w[2]), fix_value(w[3])},
                     *reinterpret_cast<const half2_t*>(svh_e + H), lane, u0, u1);
    const float h0 = (float)(half_t)glu_act(g0, u0, activation);
    const float h1 = (float)(half_t)glu_act(g1, u1, activation);
    const half2_t ds =
        *reinterpret_cast<const half2_t*>(dn_suh + (size_t)e * H + hg * 128 + 2 * lane);
    float a = h0 * (float)ds.x, b = h1 * (float)ds.y;
    wht128_lanes(a, b, lane);
    half2_t o;
    o.x = (half_t)(a * kHadScaleF);
    o.y = (half_t)(b * kHadScaleF);
    *reinterpret_cast<half2_t*>(xh_dn + (size_t)s * H + hg * 128 + 2 * lane) = o;
}

// grid = (slots * D/128, ceil((H/128) / 4)); slot s = gid / dblocks, column block
// og = gid % dblocks. xh_dn is already rotated. part: fp32 [gid][n_wg][128].
template <int K, int CB, int NW>
__global__ __launch_bounds__(NW * 64) void moe_down_kernel(
    const uint32_t* __restrict__ dn_trellis, const half_t* __restrict__ xh_dn,
    const int* __restrict__ indices, const half_t* __restrict__ dn_svh, half_t* __restrict__ y,
    float* part, int* counters, int E, int D, int H) {
    __shared__ __attribute__((aligned(16))) half_t xs[NW][1][kXwLd];
    __shared__ float red[NW][128];
    __shared__ int last_flag;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int dblocks = D >> 7, hblocks = H >> 7;
    const int n_wg = gridDim.y;
    const int gid = blockIdx.x;
    const int og = gid % dblocks, s = gid / dblocks;
    const int e = clamp_expert(indices[s], E);
    constexpr bool kHalf = NW == 8;
    const int part_idx = blockIdx.y * NW + wave;
    const int blk = kHalf ? part_idx >> 1 : part_idx;
    const int tk0 = blk * 8 + (kHalf ? (part_idx & 1) * 4 : 0);
    float acc[1][2] = {{0.f, 0.f}};
    if (blk < hblocks) {
        const size_t row_words = (size_t)E * (D >> 4) * (8 * K);
        const uint32_t* base = dn_trellis + ((size_t)e * (D >> 4) + 8 * og) * (8 * K) + lane * K;
        stream_block_rows<K, CB, 1, false, kHalf>(base, row_words, tk0, tk0 + (kHalf ? 4 : 8),
                                                  xh_dn + (size_t)s * H, (size_t)H, 1, nullptr,
                                                  xs[wave], lane, acc);
    }
    float2_t v = moe_wg_sum<NW>(red, acc, lane, wave);
    if (n_wg > 1) {
        int* counter = counters + gid;
        if (wave == 0) {
            const bool last = moe_publish(part + ((size_t)gid * n_wg + blockIdx.y) * 128, v,
                                          counter, n_wg, lane);
            if (lane == 0) last_flag = last;
        }
        __syncthreads();
        if (!last_flag || wave != 0) return;
        asm volatile("" ::: "memory");
        v = moe_sum_rows(part + (size_t)gid * n_wg * 128, n_wg, lane);
        if (lane == 0) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    } else if (wave != 0) {
        return;
    }
    const half2_t sv =
        *reinterpret_cast<const half2_t*>(dn_svh + (size_t)e * D + og * 128 + 2 * lane);
    float o0, o1;
    moe_finish_block(v, sv, lane, o0, o1);
    half2_t o;
    o.x = (half_t)o0;
    o.y = (half_t)o1;
    *reinterpret_cast<half2_t*>(y + (size_t)s * D + og * 128 + 2 * lane) = o;
}

// ---------------------------------------------------------------------------
// The same chain with the slots grouped by expert. With several tokens, slots that
// route to the same expert share one pass over its weights: the grid stays one
// workgroup set per slot, every workgroup finds the slots of its own expert in the
// routing table, and only the first of every four of them (in slot order) works, on up
// to four batch rows (the 4x4x4 matrix instructions carry four rows at the price of
// one). The others leave at once. Per row the arithmetic, the partial rows and the
// counters are those of the kernels above, so the results are bit-identical.

constexpr int kGroupRows = 4;       // batch rows one workgroup carries
constexpr int kGroupMaxSlots = 512; // routing table entries a workgroup scans (8 per lane)

struct SlotGroup {
    int n;               // rows of this workgroup; 0 = another workgroup carries this slot
    int expert;
    int s0, s1, s2, s3;  // the rows' slots, ascending; entries past n repeat s0
};

// Loads above stay above, work below stays below (in the optimiser, which would sink
// loads to their first use, and in the instruction scheduler): the routing table is
// requested first, the first trellis rows second, and the search of the table runs
// while the trellis rows are in flight. Emits no instruction.
__device__ __forceinline__ void pin_program_order() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
}

// The same address with its origin hidden from the optimiser: loads through a kernel
// argument that is declared free of aliases may otherwise move across pin_program_order.
__device__ __forceinline__ global_words_t opaque_pointer(const uint32_t* p) {
    asm volatile("" : "+v"(p));
    return (global_words_t)p;
}

// A wave's copy of the routing table: lane l holds entries c*64 + l (the last entry
// repeated past the end). Always the same number of loads, whatever `slots` is, so
// that the wait for them can leave younger loads in flight.
struct SlotTable {
    int idx[kGroupMaxSlots / 64];
};

__device__ __forceinline__ SlotTable load_slot_table(const int* __restrict__ indices, int slots,
                                                     int lane) {
    SlotTable t;
#pragma unroll
    for (int c = 0; c < kGroupMaxSlots / 64; c++) t.idx[c] = indices[min(c * 64 + lane, slots - 1)];
    return t;
}

// Nothing computed from the table may be placed above this point.
__device__ __forceinline__ void use_table_from_here(SlotTable& t) {
#pragma unroll
    for (int c = 0; c < kGroupMaxSlots / 64; c++) asm volatile("" : "+v"(t.idx[c]));
}

// Every wave computes the same answer (wave-uniform values). Branch-free: the matches
// of chunk c are a 64-bit ballot; the slots before s are counted, the first three
// after s extracted.
__device__ __forceinline__ SlotGroup find_slot_group(const SlotTable& t, int slots, int s,
                                                     int expert, int E, int lane) {
    constexpr int kChunks = kGroupMaxSlots / 64;
    const int sc = s >> 6, sb = s & 63;
    const uint64_t below = (1ull << sb) - 1ull;
    uint64_t after[kChunks];
    int before = 0;
#pragma unroll
    for (int c = 0; c < kChunks; c++) {
        const uint64_t m =
            __ballot(c * 64 + lane < slots && clamp_expert(t.idx[c], E) == expert);
        before += __popcll(c < sc ? m : (c == sc ? m & below : 0ull));
        after[c] = c < sc ? 0ull : (c == sc ? m & ~(below | (1ull << sb)) : m);
    }
    int n = 1, next[kGroupRows - 1];
#pragma unroll
    for (int take = 0; take < kGroupRows - 1; take++) {
        int pos = -1;
#pragma unroll
        for (int c = kChunks - 1; c >= 0; c--)
            if (after[c] != 0) pos = c;  // lowest chunk that still has a match
#pragma unroll
        for (int c = 0; c < kChunks; c++) {
            if (pos == c) {
                pos = c * 64 + (int)__builtin_ctzll(after[c]) + (1 << 20);
                after[c] &= after[c] - 1;
            }
        }
        next[take] = pos < 0 ? s : pos - (1 << 20);
        n += pos >= 0;
    }
    SlotGroup g;
    g.expert = expert;
    g.n = __builtin_amdgcn_readfirstlane((before % kGroupRows) == 0 ? n : 0);
    g.s0 = s;
    g.s1 = __builtin_amdgcn_readfirstlane(next[0]);
    g.s2 = __builtin_amdgcn_readfirstlane(next[1]);
    g.s3 = __builtin_amdgcn_readfirstlane(next[2]);
    return g;
}

__device__ __forceinline__ int group_slot(const SlotGroup& g, int r) {
    return r == 1 ? g.s1 : (r == 2 ? g.s2 : (r == 3 ? g.s3 : g.s0));
}

// The NW waves' sums of batch row r, added in wave order.
template <int NW>
__device__ __forceinline__ float2_t moe_row_sum(const float (*red)[kGroupRows][128], int r,
                                                int lane) {
    float2_t v{red[0][r][2 * lane], red[0][r][2 * lane + 1]};
#pragma unroll
    for (int w = 1; w < NW; w++) {
        v.x = __fadd_rn(v.x, red[w][r][2 * lane]);
        v.y = __fadd_rn(v.y, red[w][r][2 * lane + 1]);
    }
    return v;
}

// Same grid and arguments as moe_gateup_kernel (+ slots). Wave r of the working
// workgroup takes batch row r through the split reduction and, as the last
// contributor of (slot, column block), through gate finish, up finish, GLU and the
// rotation for the down projection.
template <int K, int CB, int NW>
__global__ __launch_bounds__(NW * 64) void moe_gateup_grouped_kernel(
    const uint32_t* __restrict__ gu_trellis, const half_t* __restrict__ x,
    const int* __restrict__ indices, const half_t* __restrict__ gu_suh,
    const half_t* __restrict__ gu_svh, const half_t* __restrict__ dn_suh, half_t* xh_dn,
    float* part, int* counters, int slots, int top_k, int E, int D, int H, int activation) {
    __shared__ __attribute__((aligned(16))) half_t xs[NW][kGroupRows][kXwLd];
    __shared__ float red[NW][kGroupRows][128];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int dblocks = D >> 7, hblocks = H >> 7;
    const int n_wg = gridDim.y;
    const int gid = blockIdx.x;
    const int hg = gid % hblocks, sp = gid / hblocks;
    const int s = sp >> 1, p = sp & 1;
    // the first trellis loads only need this slot's own expert: they are in flight
    // while the routing table is searched; workgroups that carry nothing drop them
    const int e = clamp_expert(indices[s], E);
    constexpr bool kHalf = NW == 8;
    const int part_idx = blockIdx.y * NW + wave;
    const int blk = kHalf ? part_idx >> 1 : part_idx;
    // (waves past the last block load the last block's rows and drop them, so that every
    // wave has the same loads in flight behind the table's)
    const int tk0 = min(blk, dblocks - 1) * 8 + (kHalf ? (part_idx & 1) * 4 : 0);
    const int tk1 = tk0 + (kHalf ? 4 : 8);
    const size_t row_words = (size_t)E * 2 * (H >> 4) * (8 * K);
    const uint32_t* base =
        gu_trellis + ((size_t)(p * E + e) * (H >> 4) + 8 * hg) * (8 * K) + lane * K;
    SlotTable table = load_slot_table(indices, slots, lane);
    uint32_t buf[kStreamSlots][K];
    pin_program_order();
    issue_first_rows<K, kHalf>(opaque_pointer(base), row_words, tk0, tk1, buf);
    pin_program_order();
    use_table_from_here(table);
    const SlotGroup grp = find_slot_group(table, slots, s, e, E, lane);
    if (grp.n == 0) return;
    float acc[kGroupRows][2];
#pragma unroll
    for (int m = 0; m < kGroupRows; m++) acc[m][0] = acc[m][1] = 0.f;
    if (blk < dblocks) {
        const half_t* xrow[kGroupRows];
#pragma unroll
        for (int m = 0; m < kGroupRows; m++) xrow[m] = x + (size_t)(group_slot(grp, m) / top_k) * D;
        stream_block_rows_at<K, CB, kGroupRows, true, kHalf, true, true, true>(
            base, row_words, tk0, tk1, xrow, grp.n, gu_suh + ((size_t)e * 2 + p) * D, xs[wave],
            lane, acc, buf);
    }
    const int c0 = (lane >> 3) * 16 + (lane & 7);
#pragma unroll
    for (int m = 0; m < kGroupRows; m++) {
        red[wave][m][c0] = acc[m][0];
        red[wave][m][c0 + 8] = acc[m][1];
    }
    __syncthreads();
    if (wave >= grp.n) return;
    const int sr = group_slot(grp, wave);
    const float2_t v = moe_row_sum<NW>(red, wave, lane);
    int* counter = counters + sr * hblocks + hg;
    const size_t gid_r = ((size_t)sr * 2 + p) * hblocks + hg;
    if (!moe_publish(part + (gid_r * n_wg + blockIdx.y) * 128, v, counter, 2 * n_wg, lane)) return;
    asm volatile("" ::: "memory");
    // both projections' partial rows in flight together
    const float* rows_g = part + (((size_t)sr * 2) * hblocks + hg) * n_wg * 128;
    const float* rows_u = part + (((size_t)sr * 2 + 1) * hblocks + hg) * n_wg * 128;
    float2_t sg{0.f, 0.f}, su{0.f, 0.f};
    for (int s0 = 0; s0 < n_wg; s0 += 4) {  // four rows of each projection per round trip
        uint64_t vg[4], vu[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const size_t off = (size_t)min(s0 + i, n_wg - 1) * 128 + 2 * lane;
            vg[i] = __hip_atomic_load(reinterpret_cast<const uint64_t*>(rows_g + off),
                                      __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            vu[i] = __hip_atomic_load(reinterpret_cast<const uint64_t*>(rows_u + off),
                                      __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
#pragma unroll
        for (int i = 0; i < 4; i++) {
            if (s0 + i < n_wg) {
                const float2_t fg = __builtin_bit_cast(float2_t, vg[i]);
                const float2_t fu = __builtin_bit_cast(float2_t, vu[i]);
                sg.x = __fadd_rn(sg.x, fg.x);
                sg.y = __fadd_rn(sg.y, fg.y);
                su.x = __fadd_rn(su.x, fu.x);
                su.y = __fadd_rn(su.y, fu.y);
            }
        }
    }
    const half_t* svh_e = gu_svh + (size_t)e * 2 * H + hg * 128 + 2 * lane;
    float g0, g1, u0, u1;
    moe_finish_block(sg, *reinterpret_cast<const half2_t*>(svh_e), lane, g0, g1);
    moe_finish_block(su, *reinterpret_cast<const half2_t*>(svh_e + H), lane, u0, u1);
    const float h0 = (float)(half_t)glu_act(g0, u0, activation);
    const float h1 = (float)(half_t)glu_act(g1, u1, activation);
    const half2_t ds =
        *reinterpret_cast<const half2_t*>(dn_suh + (size_t)e * H + hg * 128 + 2 * lane);
    float a = h0 * (float)ds.x, b = h1 * (float)ds.y;
    wht128_lanes(a, b, lane);
    half2_t o;
    o.x = (half_t)(a * kHadScaleF);
    o.y = (half_t)(b * kHadScaleF);
    *reinterpret_cast<half2_t*>(xh_dn + (size_t)sr * H + hg * 128 + 2 * lane) = o;
    if (lane == 0) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Same grid and arguments as moe_down_kernel (+ slots); wave r finishes batch row r.
template <int K, int CB, int NW>
__global__ __launch_bounds__(NW * 64) void moe_down_grouped_kernel(
    const uint32_t* __restrict__ dn_trellis, const half_t* __restrict__ xh_dn,
    const int* __restrict__ indices, const half_t* __restrict__ dn_svh, half_t* __restrict__ y,
    float* part, int* counters, int slots, int E, int D, int H) {
    __shared__ __attribute__((aligned(16))) half_t xs[NW][kGroupRows][kXwLd];
    __shared__ float red[NW][kGroupRows][128];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int dblocks = D >> 7, hblocks = H >> 7;
    const int n_wg = gridDim.y;
    const int gid = blockIdx.x;
    const int og = gid % dblocks, s = gid / dblocks;
    const int e = clamp_expert(indices[s], E);
    constexpr bool kHalf = NW == 8;
    const int part_idx = blockIdx.y * NW + wave;
    const int blk = kHalf ? part_idx >> 1 : part_idx;
    const int tk0 = min(blk, hblocks - 1) * 8 + (kHalf ? (part_idx & 1) * 4 : 0);
    const int tk1 = tk0 + (kHalf ? 4 : 8);
    const size_t row_words = (size_t)E * (D >> 4) * (8 * K);
    const uint32_t* base = dn_trellis + ((size_t)e * (D >> 4) + 8 * og) * (8 * K) + lane * K;
    SlotTable table = load_slot_table(indices, slots, lane);
    uint32_t buf[kStreamSlots][K];
    pin_program_order();
    issue_first_rows<K, kHalf>(opaque_pointer(base), row_words, tk0, tk1, buf);
    pin_program_order();
    use_table_from_here(table);
    const SlotGroup grp = find_slot_group(table, slots, s, e, E, lane);
    if (grp.n == 0) return;
    float acc[kGroupRows][2];
#pragma unroll
    for (int m = 0; m < kGroupRows; m++) acc[m][0] = acc[m][1] = 0.f;
    if (blk < hblocks) {
        const half_t* xrow[kGroupRows];
#pragma unroll
        for (int m = 0; m < kGroupRows; m++) xrow[m] = xh_dn + (size_t)group_slot(grp, m) * H;
        stream_block_rows_at<K, CB, kGroupRows, false, kHalf, true, true>(
            base, row_words, tk0, tk1, xrow, grp.n, nullptr, xs[wave], lane, acc, buf);
    }
    const int c0 = (lane >> 3) * 16 + (lane & 7);
#pragma unroll
    for (int m = 0; m < kGroupRows; m++) {
        red[wave][m][c0] = acc[m][0];
        red[wave][m][c0 + 8] = acc[m][1];
    }
    __syncthreads();
    if (wave >= grp.n) return;
    const int sr = group_slot(grp, wave);
    float2_t v = moe_row_sum<NW>(red, wave, lane);
    if (n_wg > 1) {
        const size_t gid_r = (size_t)sr * dblocks + og;
        int* counter = counters + gid_r;
        if (!moe_publish(part + (gid_r * n_wg + blockIdx.y) * 128, v, counter, n_wg, lane)) return;
        asm volatile("" ::: "memory");
        v = moe_sum_rows(part + gid_r * n_wg * 128, n_wg, lane);
        if (lane == 0) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    const half2_t sv =
        *reinterpret_cast<const half2_t*>(dn_svh + (size_t)e * D + og * 128 + 2 * lane);
    float o0, o1;
    moe_finish_block(v, sv, lane, o0, o1);
    half2_t o;
    o.x = (half_t)o0;
    o.y = (half_t)o1;
    *reinterpret_cast<half2_t*>(y + (size_t)sr * D + og * 128 + 2 * lane) = o;
}

struct MoeWorkspace {
    size_t xh_gu, xh_dn, tables, part_gu, part_dn;
    size_t o_xh_gu, o_xh_dn, o_tables, o_part_gu, o_part_dn, total;
    GemvPlan plan_gu, plan_dn;
    int g_gu, g_dn;
};

// Two-launch chain: below this many whole-block waves in the gate/up launch the waves
// take half blocks (4096 = four per SIMD).
static int moe_half_below() {
    static const int v = env_int("EXL3_MOE_HALF_BELOW", 4096, 0, 1 << 20);
    return v;
}

// Two-launch chain with several tokens: slots of the same expert in one workgroup (1) or
// every slot on its own (0).
static bool moe_group_slots() {
    static const int v = env_int("EXL3_MOE_GROUP", 1, 0, 1);
    return v != 0;
}

// Gate/up launches that would issue more atomics than this reduce through partial rows
// (the memory side retires about 75 000 returning atomics per microsecond).
static long long moe_max_atomics() {
    static const int v = env_int("EXL3_MOE_MAX_ATOMICS", 300000, 0, 1 << 30);
    return v;
}

static MoeWorkspace moe_workspace(int tokens, int top_k, int D, int H) {
    MoeWorkspace w{};
    const int slots = tokens * top_k;
    w.g_gu = slots * 2 * (H / 128);
    w.g_dn = slots * (D / 128);
    w.plan_gu = plan_gemv(1, D / 16, w.g_gu);
    w.plan_dn = plan_gemv(1, H / 16, w.g_dn);
    w.xh_gu = align_up((size_t)slots * 2 * D * 2, 256);
    w.xh_dn = align_up((size_t)slots * H * 2, 256);
    w.tables = align_up((size_t)2 * (w.g_gu + w.g_dn) * sizeof(int), 256);
    // partial rows per group: the chain's split plan or the fused kernels' one row per
    // workgroup of four Hadamard blocks, whichever is larger
    const int rows_gu = std::max(w.plan_gu.n_partials(), (D / 128 + 3) / 4);
    const int rows_dn = std::max(w.plan_dn.n_partials(), (H / 128 + 3) / 4);
    w.part_gu = align_up((size_t)rows_gu * w.g_gu * 128 * sizeof(float), 256);
    w.part_dn = align_up((size_t)rows_dn * w.g_dn * 128 * sizeof(float), 256);
    w.o_xh_gu = 0;
    w.o_xh_dn = w.o_xh_gu + w.xh_gu;
    w.o_tables = w.o_xh_dn + w.xh_dn;
    w.o_part_gu = w.o_tables + w.tables;
    w.o_part_dn = w.o_part_gu + w.part_gu;
    w.total = w.o_part_dn + w.part_dn;
    return w;
}

// ---------------------------------------------------------------------------
// Prefill glue: sort the (token, slot) pairs by expert and build the row-block
// table of the segmented GEMM in ONE launch of one workgroup (the pair counts are
// small: tokens * top_k), and finish gate/up + GLU + down rotation per sorted row.

constexpr int kSortThreads = 1024;
constexpr int kSortMaxExperts = 1024;

// Stable counting sort by expert id. Outputs, all indexed by sorted position:
//   order[pos] = pair index (token * top_k + slot), tok[pos] = token,
//   sidx[pos] = expert; table[b] = {expert, first row, end row of the expert, 0}
// for every block of block_rows rows, unused entries {E-1, N, N, 0} (empty).
__global__ __launch_bounds__(kSortThreads) void moe_sort_kernel(
    const int* __restrict__ indices, int n_pairs, int top_k, int E, int block_rows,
    int* __restrict__ order, int* __restrict__ tok, int* __restrict__ sidx,
    int4* __restrict__ table, int table_len) {
    __shared__ int count[kSortMaxExperts];  // pairs per expert, later the scatter cursor
    __shared__ unsigned short wave_count[kSortThreads / 64][kSortMaxExperts];  // <= 64 each
    __shared__ int scan_tmp[2][kSortThreads / 64];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    for (int e = tid; e < E; e += kSortThreads) count[e] = 0;
    for (int i = tid; i < (kSortThreads / 64) * kSortMaxExperts; i += kSortThreads)
        (&wave_count[0][0])[i] = 0;
    __syncthreads();
    for (int i = tid; i < n_pairs; i += kSortThreads) atomicAdd(&count[clamp_expert(indices[i], E)], 1);
    __syncthreads();

    // exclusive scans over the experts (E <= 1024 = one value per thread): rows and blocks
    const int c = tid < E ? count[tid] : 0;
    const int nb = (c + block_rows - 1) / block_rows;
    int inc_rows = c, inc_blk = nb;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const int r = __shfl_up(inc_rows, off, kWave), b = __shfl_up(inc_blk, off, kWave);
        if (lane >= off) {
            inc_rows += r;
            inc_blk += b;
        }
    }
    if (lane == 63) {
        scan_tmp[0][wave] = inc_rows;
        scan_tmp[1][wave] = inc_blk;
    }
    __syncthreads();
    int base_rows = 0, base_blk = 0, total_blk = 0;
    for (int w = 0; w < kSortThreads / 64; w++) {
        if (w < wave) {
            base_rows += scan_tmp[0][w];
            base_blk += scan_tmp[1][w];
        }
        total_blk += scan_tmp[1][w];
    }
    const int row0 = base_rows + inc_rows - c;  // first sorted row of expert tid
    const int blk0 = base_blk + inc_blk - nb;
    __syncthreads();
    if (tid < E) {
        count[tid] = row0;  // scatter cursor
        for (int b = 0; b < nb && blk0 + b < table_len; b++)
            table[blk0 + b] = int4{tid, row0 + b * block_rows, row0 + c, 0};
    }
    for (int b = total_blk + tid; b < table_len; b += kSortThreads)
        table[b] = int4{E - 1, n_pairs, n_pairs, 0};
    __syncthreads();

    // stable scatter, 1024 pairs at a time in pair order: rank inside the wave by
    // matching expert ids bit by bit, then across the waves of the chunk
    int ebits = 0;
    while ((1 << ebits) < E) ebits++;
    for (int i0 = 0; i0 < n_pairs; i0 += kSortThreads) {
        const int i = i0 + tid;
        const bool valid = i < n_pairs;
        const int e = valid ? clamp_expert(indices[i], E) : 0;
        unsigned long long same = __ballot(valid);
        for (int b = 0; b < ebits; b++) {
            const unsigned long long m = __ballot(valid && ((e >> b) & 1));
            same &= ((e >> b) & 1) ? m : ~m;
        }
        const int rank = __popcll(same & ((1ull << lane) - 1ull));
        if (valid && rank == 0) wave_count[wave][e] = (unsigned short)__popcll(same);
        __syncthreads();
        if (valid) {
            int pos = count[e] + rank;
            for (int w = 0; w < wave; w++) pos += wave_count[w][e];
            order[pos] = i;
            tok[pos] = i / top_k;
            sidx[pos] = e;
        }
        __syncthreads();
        for (int ee = tid; ee < E; ee += kSortThreads) {
            int add = 0;
#pragma unroll
            for (int w = 0; w < kSortThreads / 64; w++) {
                add += wave_count[w][ee];
                wave_count[w][ee] = 0;
            }
            count[ee] += add;
        }
        __syncthreads();
    }
}

// One wave per (sorted row, 128-block of H): post-Hadamard + svh of the gate and up
// GEMM outputs, GLU, and the input rotation (dn_suh) of the down projection; the
// same steps and casts as moe_glu_kernel, on fp16 GEMM outputs.
__global__ __launch_bounds__(256) void moe_glu_rows_kernel(
    const half_t* __restrict__ g, const half_t* __restrict__ u, int n_rows, int H,
    const int* __restrict__ sidx, const half_t* __restrict__ gu_svh,
    const half_t* __restrict__ dn_suh, int E, int activation, half_t* __restrict__ xh_dn) {
    const int lane = threadIdx.x & 63;
    const int hblocks = H >> 7;
    const long long wave_id = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (wave_id >= (long long)n_rows * hblocks) return;
    const int blk = (int)(wave_id % hblocks);
    const size_t r = (size_t)(wave_id / hblocks);
    const int e = clamp_expert(sidx[r], E);
    const size_t off = r * H + blk * 128 + 2 * lane;
    float v[2][2];
#pragma unroll
    for (int p = 0; p < 2; p++) {
        const half2_t in = *reinterpret_cast<const half2_t*>((p ? u : g) + off);
        float a = (float)in.x, b = (float)in.y;
        wht128_lanes(a, b, lane);
        const half2_t sv = *reinterpret_cast<const half2_t*>(gu_svh + (size_t)e * 2 * H + p * H +
                                                             blk * 128 + 2 * lane);
        v[p][0] = (float)(half_t)(a * kHadScaleF * (float)sv.x);
        v[p][1] = (float)(half_t)(b * kHadScaleF * (float)sv.y);
    }
    const float h0 = (float)(half_t)glu_act(v[0][0], v[1][0], activation);
    const float h1 = (float)(half_t)glu_act(v[0][1], v[1][1], activation);
    const half2_t ds =
        *reinterpret_cast<const half2_t*>(dn_suh + (size_t)e * H + blk * 128 + 2 * lane);
    float a = h0 * (float)ds.x, b = h1 * (float)ds.y;
    wht128_lanes(a, b, lane);
    half2_t o;
    o.x = (half_t)(a * kHadScaleF);
    o.y = (half_t)(b * kHadScaleF);
    *reinterpret_cast<half2_t*>(xh_dn + off) = o;
}

}  // namespace exl3

EXL3_EXPORT size_t exl3_moe_workspace_bytes(int tokens, int top_k, int D, int H) {
    if (tokens < 1 || top_k < 1 || D < 128 || H < 128 || D % 128 || H % 128) return 0;
    return exl3::moe_workspace(tokens, top_k, D, H).total;
}

EXL3_EXPORT int exl3_moe_forward(const uint16_t* x, int tokens, const int32_t* indices, int top_k,
                                 const uint16_t* gu_trellis, const uint16_t* gu_suh,
                                 const uint16_t* gu_svh, const uint16_t* dn_trellis,
                                 const uint16_t* dn_suh, const uint16_t* dn_svh, int num_experts,
                                 int D, int H, int K, int cb, int activation, uint16_t* y,
                                 void* workspace, size_t workspace_bytes, int32_t* counters,
                                 size_t counters_len, void* stream) {
    using namespace exl3;
    if (int rc = check_k_cb(K, cb)) return rc;
    if (!x || !indices || !gu_trellis || !gu_suh || !gu_svh || !dn_trellis || !dn_suh || !dn_svh ||
        !y || !workspace)
        return EXL3_E_NULL_POINTER;
    if (tokens < 1 || top_k < 1 || num_experts < 1 || D < 128 || H < 128 || D % 128 || H % 128 ||
        (long long)tokens * top_k > 4096)
        return EXL3_E_BAD_SHAPE;
    if (activation != 0 && activation != 1) return EXL3_E_UNSUPPORTED;
    const MoeWorkspace w = moe_workspace(tokens, top_k, D, H);
    if (workspace_bytes < w.total) return EXL3_E_WORKSPACE;
    hipStream_t s = as_stream(stream);
    char* base = reinterpret_cast<char*>(workspace);
    half_t* xh_gu = reinterpret_cast<half_t*>(base + w.o_xh_gu);
    half_t* xh_dn = reinterpret_cast<half_t*>(base + w.o_xh_dn);
    int* gu_sub = reinterpret_cast<int*>(base + w.o_tables);
    int* gu_tile = gu_sub + w.g_gu;
    int* dn_sub = gu_tile + w.g_gu;
    int* dn_tile = dn_sub + w.g_dn;
    float* part_gu = reinterpret_cast<float*>(base + w.o_part_gu);
    float* part_dn = reinterpret_cast<float*>(base + w.o_part_dn);
    const int slots = tokens * top_k;

    if (counters && !exact_weights()) {
        // two launches: gate/up + GLU + rotation, then down
        const int hblocks = H / 128, dblocks = D / 128;
        if (counters_len < (size_t)slots * (hblocks + dblocks)) return EXL3_E_WORKSPACE;
        // few slots: eight waves per workgroup, each on half a block, so that the
        // chip holds twice the loads in flight (same workgroup count, same partial rows)
        const bool half = (size_t)slots * 2 * hblocks * dblocks < (size_t)moe_half_below();
        // several tokens: slots of one expert share a pass over its weights, once enough
        // of them coincide to pay for the table search (from one slot per two experts on:
        // 16 tokens of top-8 over 256 experts, where ~20 % of the slots share an expert)
        const bool grouped = tokens > 1 && slots <= kGroupMaxSlots && 2 * slots >= num_experts &&
                             moe_group_slots();
        // every slot on its own, few enough atomics, and counters large enough to hold
        // the accumulators (uint64 [slots][2][H], then the down launch's counters): gate
        // and up of a k-chunk in one workgroup, reduced through returning atomics
        const int pair_chunks = half ? (dblocks + 1) / 2 : (dblocks + 3) / 4;
        const size_t pair_ints = (size_t)slots * 2 * H * 2;
        const bool pair = !grouped && pair_chunks <= 255 &&
                          (long long)slots * 2 * H * pair_chunks <= moe_max_atomics() &&
                          counters_len >= pair_ints + (size_t)slots * dblocks &&
                          (reinterpret_cast<uintptr_t>(counters) & 7) == 0;
        auto chain = [&](auto k, auto c, auto nw) {
            constexpr int NW = nw.value;
            if (pair) {
                moe_gateup_pair_kernel<k.value, c.value, NW == 8>
                    <<<dim3((unsigned)(slots * hblocks), (unsigned)pair_chunks), dim3(512), 0, s>>>(
                        reinterpret_cast<const uint32_t*>(gu_trellis),
                        reinterpret_cast<const half_t*>(x), indices,
                        reinterpret_cast<const half_t*>(gu_suh),
                        reinterpret_cast<const half_t*>(gu_svh),
                        reinterpret_cast<const half_t*>(dn_suh), xh_dn,
                        reinterpret_cast<unsigned long long*>(counters), top_k, num_experts, D, H,
                        activation,
                        counters_status_word(counters, counters_len,
                                             pair_ints + (size_t)slots * dblocks),
                        reduction_spin_limit());
                if (int rc = launch_status()) return rc;
                moe_down_kernel<k.value, c.value, NW>
                    <<<dim3((unsigned)(slots * dblocks), (unsigned)((hblocks + 3) / 4)),
                       dim3(NW * 64), 0, s>>>(reinterpret_cast<const uint32_t*>(dn_trellis), xh_dn,
                                              indices, reinterpret_cast<const half_t*>(dn_svh),
                                              reinterpret_cast<half_t*>(y), part_dn,
                                              counters + pair_ints, num_experts, D, H);
                return launch_status();
            }
            if (grouped) {
                moe_gateup_grouped_kernel<k.value, c.value, NW>
                    <<<dim3((unsigned)(slots * 2 * hblocks), (unsigned)((dblocks + 3) / 4)),
                       dim3(NW * 64), 0, s>>>(reinterpret_cast<const uint32_t*>(gu_trellis),
                                              reinterpret_cast<const half_t*>(x), indices,
                                              reinterpret_cast<const half_t*>(gu_suh),
                                              reinterpret_cast<const half_t*>(gu_svh),
                                              reinterpret_cast<const half_t*>(dn_suh), xh_dn,
                                              part_gu, counters, slots, top_k, num_experts, D, H,
                                              activation);
                if (int rc = launch_status()) return rc;
                moe_down_grouped_kernel<k.value, c.value, NW>
                    <<<dim3((unsigned)(slots * dblocks), (unsigned)((hblocks + 3) / 4)),
                       dim3(NW * 64), 0, s>>>(reinterpret_cast<const uint32_t*>(dn_trellis), xh_dn,
                                              indices, reinterpret_cast<const half_t*>(dn_svh),
                                              reinterpret_cast<half_t*>(y), part_dn,
                                              counters + (size_t)slots * hblocks, slots,
                                              num_experts, D, H);
                return launch_status();
            }
            moe_gateup_kernel<k.value, c.value, NW>
                <<<dim3((unsigned)(slots * 2 * hblocks), (unsigned)((dblocks + 3) / 4)),
                   dim3(NW * 64), 0, s>>>(reinterpret_cast<const uint32_t*>(gu_trellis),
                                          reinterpret_cast<const half_t*>(x), indices,
                                          reinterpret_cast<const half_t*>(gu_suh),
                                          reinterpret_cast<const half_t*>(gu_svh),
                                          reinterpret_cast<const half_t*>(dn_suh), xh_dn, part_gu,
                                          counters, top_k, num_experts, D, H, activation);
            if (int rc = launch_status()) return rc;
            moe_down_kernel<k.value, c.value, NW>
                <<<dim3((unsigned)(slots * dblocks), (unsigned)((hblocks + 3) / 4)), dim3(NW * 64),
                   0, s>>>(reinterpret_cast<const uint32_t*>(dn_trellis), xh_dn, indices,
                           reinterpret_cast<const half_t*>(dn_svh), reinterpret_cast<half_t*>(y),
                           part_dn, counters + (size_t)slots * hblocks, num_experts, D, H);
            return launch_status();
        };
        return dispatch_k_cb(K, cb, [&](auto k, auto c) {
            return half ? chain(k, c, std::integral_constant<int, 8>{})
                        : chain(k, c, std::integral_constant<int, 4>{});
        });
    }

    {
        const int waves = slots * 2 * (D / 128);
        const int threads = waves * 64 > w.g_gu ? waves * 64 : w.g_gu;
        const int need = threads > w.g_dn ? threads : w.g_dn;
        moe_prep_kernel<<<dim3((need + 255) / 256), dim3(256), 0, s>>>(
            reinterpret_cast<const half_t*>(x), indices, reinterpret_cast<const half_t*>(gu_suh),
            xh_gu, gu_sub, gu_tile, dn_sub, dn_tile, slots, top_k, num_experts, D, H);
        if (int rc = launch_status()) return rc;
    }
    // gate/up: rows = 1, n_sub = 2*slots activation rows, one group per (slot, proj, hg)
    if (int rc = launch_gemv_partials(reinterpret_cast<const uint16_t*>(xh_gu), 1, slots * 2,
                                      gu_trellis, D / 16, num_experts * 2 * (H / 16), K, cb,
                                      gu_sub, gu_tile, w.g_gu, part_gu, w.plan_gu, s))
        return rc;
    {
        const int waves = slots * (H / 128);
        moe_glu_kernel<<<dim3((waves + 3) / 4), dim3(256), 0, s>>>(
            part_gu, w.plan_gu.n_partials(), (size_t)w.g_gu * 128, indices,
            reinterpret_cast<const half_t*>(gu_svh), reinterpret_cast<const half_t*>(dn_suh), xh_dn,
            slots, H, num_experts, activation);
        if (int rc = launch_status()) return rc;
    }
    if (int rc = launch_gemv_partials(reinterpret_cast<const uint16_t*>(xh_dn), 1, slots,
                                      dn_trellis, H / 16, num_experts * (D / 16), K, cb, dn_sub,
                                      dn_tile, w.g_dn, part_dn, w.plan_dn, s))
        return rc;
    {
        const int waves = slots * (D / 128);
        moe_finish_kernel<<<dim3((waves + 3) / 4), dim3(256), 0, s>>>(
            part_dn, w.plan_dn.n_partials(), (size_t)w.g_dn * 128, indices,
            reinterpret_cast<const half_t*>(dn_svh), reinterpret_cast<half_t*>(y), slots, D,
            num_experts);
        return launch_status();
    }
}

EXL3_EXPORT int exl3_moe_sort(const int32_t* indices, int n_pairs, int top_k, int n_experts,
                              int block_rows, int32_t* order, int32_t* tok, int32_t* sidx,
                              int32_t* table, int table_len, void* stream) {
    using namespace exl3;
    if (!indices || !order || !tok || !sidx || !table) return EXL3_E_NULL_POINTER;
    if (n_pairs < 1 || top_k < 1 || n_experts < 1 || block_rows < 1 ||
        table_len < n_pairs / block_rows + n_experts)
        return EXL3_E_BAD_SHAPE;
    if (n_experts > kSortMaxExperts) return EXL3_E_UNSUPPORTED;
    if (reinterpret_cast<uintptr_t>(table) & 15) return EXL3_E_BAD_SHAPE;
    moe_sort_kernel<<<dim3(1), dim3(kSortThreads), 0, as_stream(stream)>>>(
        indices, n_pairs, top_k, n_experts, block_rows, order, tok, sidx,
        reinterpret_cast<int4*>(table), table_len);
    return launch_status();
}

EXL3_EXPORT int exl3_moe_glu_rows(const uint16_t* g, const uint16_t* u, int n_rows, int H,
                                  const int32_t* sidx, const uint16_t* gu_svh,
                                  const uint16_t* dn_suh, int n_experts, int activation,
                                  uint16_t* xh_dn, void* stream) {
    using namespace exl3;
    if (!g || !u || !sidx || !gu_svh || !dn_suh || !xh_dn) return EXL3_E_NULL_POINTER;
    if (n_rows < 0 || H < 128 || H % 128 || n_experts < 1) return EXL3_E_BAD_SHAPE;
    if (activation < 0 || activation > 1) return EXL3_E_UNSUPPORTED;
    if (n_rows == 0) return EXL3_OK;
    const long long waves = (long long)n_rows * (H / 128);
    const long long grid = (waves + 3) / 4;
    if (grid > 0x7FFFFFFFLL) return EXL3_E_BAD_SHAPE;
    moe_glu_rows_kernel<<<dim3((unsigned)grid), dim3(256), 0, as_stream(stream)>>>(
        reinterpret_cast<const half_t*>(g), reinterpret_cast<const half_t*>(u), n_rows, H, sidx,
        reinterpret_cast<const half_t*>(gu_svh), reinterpret_cast<const half_t*>(dn_suh), n_experts,
        activation, reinterpret_cast<half_t*>(xh_dn));
    return launch_status();
}
