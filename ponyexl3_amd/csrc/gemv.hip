// Small-batch fused trellis-decode GEMV (rows 1..8): y = xh @ W_inner with the
// weights decoded in registers straight from the packed bitstream.
//
// Work decomposition
//   * the unit of work is a wavefront: wave (g, s) owns the 128-column output
//     group g and split s of the tile rows, tk in [s*L, min(in_tiles, (s+1)*L));
//     the four waves of a workgroup are four consecutive splits of one group and
//     meet only once, at the end, to add their accumulators through LDS;
//   * per tile row a wave issues one wave-wide non-temporal load of 256*K
//     contiguous bytes (8 tiles) and keeps kPrefetch such loads in flight; lane
//     u of a tile decodes its 32 codewords = output columns u and u+8 over all 16
//     input rows and keeps two fp32 accumulators per batch row, so no
//     cross-lane reduction exists anywhere;
//   * activations of a tile row are wave-uniform (scalar loads) and enter
//     v_dot2_f32_f16 as SGPR operands;
//   * every workgroup writes one fp32 partial row [wg][row][128 columns]; rows
//     are added in index order by the caller (exl3_had128_post or the reduction
//     kernel below) - no atomics, so results are run-to-run deterministic.
//
// The split count is chosen so that all waves of a launch are resident at once
// (about kWavesPerSimd per SIMD) and carry equal work: no second, partly filled
// round of workgroups.
//
// Replaces the Metal kernels behind inner_gemv_mlx / inner_gemm_mlx /
// inner_gem_fused_mlx (ponyexl3/mlx/gemv_metal.py:109-232, 460-627, 1481-1515).
#include "exl3_device.hpp"
#include "exl3_host.hpp"
#include "exl3_small.hpp"

#include <stdlib.h>

namespace exl3 {

constexpr int kPrefetch = 6;  // wave-wide loads in flight per wave

template <int K, int CB, int MT>
__global__ __launch_bounds__(256) void gemv_kernel(
    const uint32_t* __restrict__ trellis, const half_t* __restrict__ xh,
    float* __restrict__ partial, const int* __restrict__ group_sub,
    const int* __restrict__ group_tile, int in_tiles, int out_tiles, int rows, int n_sub,
    int n_groups, int tk_per_split, int n_splits) {
    const int g = blockIdx.x;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int split = blockIdx.y * 4 + wave;
    const bool active = split < n_splits;  // idle waves still reach the barrier below
    const int tn0 = group_tile ? group_tile[g] : g * 8;
    const int sub = group_sub ? group_sub[g] : 0;
    const int in_features = in_tiles * 16;
    const int tk_begin = active ? split * tk_per_split : 0;
    const int tk_end = active ? min(in_tiles, tk_begin + tk_per_split) : 0;
    const size_t row_words = (size_t)out_tiles * (8 * K);
    const uint32_t* base = trellis + (size_t)tn0 * (8 * K) + lane * K;

    const half_t* xrow[MT];
#pragma unroll
    for (int m = 0; m < MT; m++) {
        const int r = m < rows ? m : 0;  // rows past the batch alias row 0 and are never stored
        xrow[m] = xh + ((size_t)r * n_sub + sub) * in_features;
    }

    float acc[MT][2];
#pragma unroll
    for (int m = 0; m < MT; m++) acc[m][0] = acc[m][1] = 0.f;

    // Software pipeline: buf[s] holds tile row tk_begin + i*kPrefetch + s. A slot
    // is refilled only after its codewords have been consumed, so the refill can
    // land in the same registers and the only wait in the loop is for the oldest
    // of the kPrefetch loads in flight.
    // One pipeline step: the neighbour dword and (for one or two batch rows) the
    // activations of the NEXT tile row are requested first, so the LDS-crossbar
    // and scalar-cache latencies hide behind this step's decode; then the current
    // slot is decoded and multiplied, then the slot is refilled from memory.
    constexpr bool kPipeX = MT <= 2;  // more rows would not fit the scalar registers
    struct XTile {
        half2_t v[MT][8];
    };
    auto load_x = [&](int tk) {
        XTile t;
#pragma unroll
        for (int m = 0; m < MT; m++) {
            const half2_t* xp = reinterpret_cast<const half2_t*>(xrow[m] + tk * 16);
#pragma unroll
            for (int j = 0; j < 8; j++) t.v[m][j] = xp[j];
        }
        return t;
    };
    auto consume = [&](const uint32_t (&words)[K], uint32_t prev, const XTile& xt) {
        const LaneWords<K> lw = make_lane_words<K>(prev, words);
        half2_t wp[16];
        decode_lane<K, CB>(lw, wp);
#pragma unroll
        for (int m = 0; m < MT; m++) {
#pragma unroll
            for (int j = 0; j < 8; j++) {
                acc[m][0] = dot2(wp[j], xt.v[m][j], acc[m][0]);
                acc[m][1] = dot2(wp[8 + j], xt.v[m][j], acc[m][1]);
            }
        }
    };

    if (active) {
        uint32_t buf[kPrefetch][K];
#pragma unroll
        for (int s = 0; s < kPrefetch; s++) {
            const int t = min(tk_begin + s, tk_end - 1);  // clamped: stays inside the split
            load_lane_words_nt<K>(base + (size_t)t * row_words, buf[s]);
        }
        uint32_t prev = neighbour_word(buf[0][K - 1], lane);
        XTile xcur = load_x(tk_begin);
        int tk0 = tk_begin;
        for (; tk0 + kPrefetch <= tk_end; tk0 += kPrefetch) {
#pragma unroll
            for (int s = 0; s < kPrefetch; s++) {
                const int tk = tk0 + s;
                // results requested one step ago (scalar loads return out of order, so
                // the only usable wait is for all of them) - long since complete
                __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
                __builtin_amdgcn_sched_barrier(0);
                const uint32_t prev_next = neighbour_word(buf[(s + 1) % kPrefetch][K - 1], lane);
                XTile xnext;
                if constexpr (kPipeX) xnext = load_x(min(tk + 1, tk_end - 1));
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (!kPipeX) xcur = load_x(tk);
                consume(buf[s], prev, xcur);
                const int tn = min(tk + kPrefetch, tk_end - 1);
                load_lane_words_nt<K>(base + (size_t)tn * row_words, buf[s]);
                __builtin_amdgcn_sched_barrier(0);
                prev = prev_next;
                if constexpr (kPipeX) xcur = xnext;
            }
        }
#pragma unroll
        for (int s = 0; s < kPrefetch - 1; s++) {
            const int tk = tk0 + s;
            if (tk < tk_end) {
                const uint32_t prev_next = neighbour_word(buf[(s + 1) % kPrefetch][K - 1], lane);
                xcur = load_x(tk);
                consume(buf[s], prev, xcur);
                prev = prev_next;
            }
        }
    }

    // the four waves are summed through LDS in wave order; one partial row per workgroup
    __shared__ float red[4][MT][128];
    const int c0 = (lane >> 3) * 16 + (lane & 7);
#pragma unroll
    for (int m = 0; m < MT; m++) {
        red[wave][m][c0] = acc[m][0];
        red[wave][m][c0 + 8] = acc[m][1];
    }
    __syncthreads();
    if (wave == 0) {
        const size_t out_total = (size_t)n_groups * 128;
#pragma unroll
        for (int m = 0; m < MT; m++) {
            if (m < rows) {
                float2_t v;
                v.x = ((red[0][m][2 * lane] + red[1][m][2 * lane]) + red[2][m][2 * lane]) +
                      red[3][m][2 * lane];
                v.y = ((red[0][m][2 * lane + 1] + red[1][m][2 * lane + 1]) +
                       red[2][m][2 * lane + 1]) + red[3][m][2 * lane + 1];
                *reinterpret_cast<float2_t*>(partial + ((size_t)blockIdx.y * rows + m) * out_total +
                                             (size_t)g * 128 + 2 * lane) = v;
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Whole small-batch layer in one launch: input Hadamard, decode GEMV, split
// reduction, output Hadamard, svh and bias.
//
//   * input side: a wave rotates the 128-wide block of x (times suh) that its
//     current tile rows need, keeps the fp16 result in its own LDS slot and reads
//     the 16 activations of a tile row back with two broadcast ds_read_b128; the
//     raw block after that is already in flight while the current one is used;
//   * output side: every workgroup adds its partial row to the accumulators of its
//     128-column group with returning atomics (fixed point, so the total is
//     independent of the arrival order); the workgroup whose add completes the group
//     rounds to fp16 (the cast at ponyexl3/ref/forward.py:41), applies the output
//     Hadamard of that one 128-column block, svh and bias, and zeroes the
//     accumulators again. No workgroup waits for another one to be scheduled.
// The counters array (accumulators uint64 [rows][out], or one int per column group)
// must be zero on entry; it is zero again when the kernel ends.
//
// HALF (one and two rows only): splits are half blocks of four tile rows.
// ATOMIC: which of the two split reductions described at the end of the kernel runs.
// NW: waves per workgroup, 4 or 8 (8 only with ATOMIC: half as many workgroups add
// to a column group's accumulators).
template <int K, int CB, int MT, bool HALF, bool ATOMIC, int NW = 4>
__global__ __launch_bounds__(NW * 64) void linear_small_kernel(
    const uint32_t* __restrict__ trellis, const half_t* __restrict__ x,
    const half_t* __restrict__ suh, const half_t* __restrict__ svh,
    const half_t* __restrict__ bias, half_t* __restrict__ y, float* partial, int* counters,
    const int* __restrict__ group_sub, int in_tiles, int out_tiles, int rows, int n_groups,
    int tk_per_split, int n_splits, int* status, int spin_limit) {
    static_assert(NW == 4 || (NW == 8 && ATOMIC), "eight-wave workgroups use the accumulators");
    // the staged activations and, once every wave has left the streaming loop, the waves'
    // sums share one LDS buffer (at eight rows the two together would cost occupancy)
    constexpr size_t kXsBytes = sizeof(half_t) * NW * MT * kXwLd;
    constexpr size_t kRedBytes = sizeof(float) * NW * MT * 128;
    __shared__ __attribute__((aligned(16))) unsigned char smem[kXsBytes > kRedBytes ? kXsBytes : kRedBytes];
    half_t (*xs)[MT][kXwLd] = reinterpret_cast<half_t (*)[MT][kXwLd]>(smem);
    float (*red)[MT][128] = reinterpret_cast<float (*)[MT][128]>(smem);
    const int g = blockIdx.x;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int split = blockIdx.y * NW + wave;
    const bool active = split < n_splits;  // idle waves still take part in the barriers below
    const int sub = group_sub ? group_sub[g] : 0;
    const int in_features = in_tiles * 16;
    const int tk_begin = active ? split * tk_per_split : 0;  // tk_per_split: multiple of 8, or 4 (HALF)
    const int tk_end = active ? min(in_tiles, tk_begin + tk_per_split) : 0;
    const size_t row_words = (size_t)out_tiles * (8 * K);
    const uint32_t* base = trellis + (size_t)g * 8 * (8 * K) + lane * K;
    const half_t* suh_row = suh ? suh + (size_t)sub * in_features : nullptr;

    float acc[MT][2];
#pragma unroll
    for (int m = 0; m < MT; m++) acc[m][0] = acc[m][1] = 0.f;

    // ---- input Hadamard (or staging) + decode/dot pipeline over this wave's blocks
    if (active)
        stream_block_rows<K, CB, MT, true, HALF>(base, row_words, tk_begin, tk_end, x,
                                                 (size_t)in_features, rows, suh_row, xs[wave], lane,
                                                 acc);

    // ---- the four waves of the workgroup are summed through LDS in wave order; the
    // workgroup's partial row then goes into the column group's accumulators with
    // returning 64-bit atomic adds, and the workgroup whose add completes the group
    // applies the output transform.
    //
    // Accumulator word of one (batch row, column): count << 56 | sum, the sum a signed
    // fixed-point number with 24 fraction bits. Integer addition is associative, so the
    // total does not depend on the order in which workgroups arrive (run-to-run
    // deterministic), and the returned old value tells a lane both how many partial
    // rows are in and what they add up to: the usual chain of store, wait, counter,
    // wait, reload (three memory round trips) becomes one round trip.
    // The eight XCDs have private L2 caches; the atomics are device-scope operations
    // that execute at the memory side, so no cache level has to be written back or
    // invalidated.
    // Finisher = the workgroup whose add brought (row 0, first column of the group) to
    // wg_splits: exactly one. Usually its other adds were last as well and it holds all
    // the totals. If another workgroup's adds were interleaved with its own, some of its
    // returned values are short; every contributor has issued all its adds by then (its
    // first one has landed), so the finisher re-reads the accumulators until all
    // counts are complete - a wait for memory operations that are already in flight,
    // not for another wave to be scheduled. Accumulators must be zero on entry; the
    // finisher zeroes them again.
    const int c0 = (lane >> 3) * 16 + (lane & 7);
    __syncthreads();  // nobody reads staged activations any more
#pragma unroll
    for (int m = 0; m < MT; m++) {
        red[wave][m][c0] = acc[m][0];
        red[wave][m][c0 + 8] = acc[m][1];
    }
    __syncthreads();
    if constexpr (ATOMIC) {
        if (wave != 0) return;
        unsigned long long* sums = reinterpret_cast<unsigned long long*>(counters);
        const size_t out_total = (size_t)n_groups * 128;
        const int wg_splits = (n_splits + NW - 1) / NW;  // partial rows per group
        const size_t col = (size_t)g * 128 + 2 * lane;
        // requested now, needed only by the finishing workgroup: by then they are here
        half2_t sv, bv;
        if (svh) sv = *reinterpret_cast<const half2_t*>(svh + col);
        if (bias) bv = *reinterpret_cast<const half2_t*>(bias + col);
        unsigned long long w0[MT], w1[MT];
#pragma unroll
        for (int m = 0; m < MT; m++) {
            w0[m] = w1[m] = 0;
            if (m < rows) {
                float vx = red[0][m][2 * lane], vy = red[0][m][2 * lane + 1];
#pragma unroll
                for (int w = 1; w < NW; w++) {  // wave order
                    vx = __fadd_rn(vx, red[w][m][2 * lane]);
                    vy = __fadd_rn(vy, red[w][m][2 * lane + 1]);
                }
                const unsigned long long ax = fix_word(vx), ay = fix_word(vy);
                unsigned long long* slot = sums + (size_t)m * out_total + col;
                w0[m] = __hip_atomic_fetch_add(slot, ax, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + ax;
                w1[m] = __hip_atomic_fetch_add(slot + 1, ay, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + ay;
            }
        }
        // lane 0's first word is (row 0, first column of the group)
        const int first_count = __builtin_amdgcn_readfirstlane(fix_count(w0[0]));
        if (first_count != wg_splits) return;
        auto all_complete = [&]() {
            bool ok = true;
#pragma unroll
            for (int m = 0; m < MT; m++)
                if (m < rows) ok = ok && fix_count(w0[m]) == wg_splits && fix_count(w1[m]) == wg_splits;
            return __ballot(ok) == ~0ull;
        };
        bool complete = all_complete();
        for (int spin = 0; !complete && spin < spin_limit; spin++) {
#pragma unroll
            for (int m = 0; m < MT; m++) {
                if (m < rows) {
                    const unsigned long long* slot = sums + (size_t)m * out_total + col;
                    w0[m] = __hip_atomic_load(slot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    w1[m] = __hip_atomic_load(slot + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            }
            complete = all_complete();
        }
        if (!complete) {
            // The counts never became complete (the array was not zero on entry, or it is
            // shared with an overlapping call). No total can be trusted: the group's
            // outputs become NaN, the status word is set and the accumulators are left
            // as they are - the caller has to zero the array again.
            if (status && lane == 0)
                __hip_atomic_fetch_or(status, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            half2_t bad;
            bad.x = bad.y = bits_to_half(0x7E00);
#pragma unroll
            for (int m = 0; m < MT; m++)
                if (m < rows) *reinterpret_cast<half2_t*>(y + (size_t)m * out_total + col) = bad;
            return;
        }
#pragma unroll
        for (int m = 0; m < MT; m++) {
            if (m < rows) {
                unsigned long long* slot = sums + (size_t)m * out_total + col;
                __hip_atomic_store(slot, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store(slot + 1, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                // the cast at ponyexl3/ref/forward.py:41, then the output Hadamard of this one
                // 128-column block, svh and bias (forward.py:42-45)
                float a = (float)(half_t)fix_value(w0[m]);
                float b = (float)(half_t)fix_value(w1[m]);
                wht128_lanes(a, b, lane);
                a = __fmul_rn(a, kHadScaleF);
                b = __fmul_rn(b, kHadScaleF);
                if (svh) {
                    a = __fmul_rn(a, (float)sv.x);
                    b = __fmul_rn(b, (float)sv.y);
                }
                half2_t o;
                o.x = (half_t)a;
                o.y = (half_t)b;
                if (bias) {
                    o.x = o.x + bv.x;
                    o.y = o.y + bv.y;
                }
                *reinterpret_cast<half2_t*>(y + (size_t)m * out_total + col) = o;
            }
        }
    } else {
        // Few, large launches (many column groups x partial rows x batch rows): the
        // memory side retires about 75 000 such atomics per microsecond, which costs
        // more than the round trips it saves. There the partial row is stored, the
        // group counter bumped, and the workgroup that brings it to wg_splits reloads
        // the partial rows in index order. Partial rows and counters only ever move
        // through device-scope accesses (the XCDs have private L2s; a release/acquire
        // fence per workgroup would write back / invalidate a whole L2), and the
        // stores are waited for (s_waitcnt vmcnt(0)) before the counter is bumped.
        __shared__ int last_flag;
        const size_t out_total = (size_t)n_groups * 128;
        const int wg_splits = (n_splits + 3) >> 2;  // partial rows per group
        const size_t col = (size_t)g * 128 + 2 * lane;
        if (wave == 0) {
#pragma unroll
            for (int m = 0; m < MT; m++) {
                if (m < rows) {
                    float2_t v;
                    v.x = ((red[0][m][2 * lane] + red[1][m][2 * lane]) + red[2][m][2 * lane]) +
                          red[3][m][2 * lane];
                    v.y = ((red[0][m][2 * lane + 1] + red[1][m][2 * lane + 1]) +
                           red[2][m][2 * lane + 1]) + red[3][m][2 * lane + 1];
                    uint64_t* dst = reinterpret_cast<uint64_t*>(
                        partial + ((size_t)blockIdx.y * rows + m) * out_total + col);
                    __hip_atomic_store(dst, __builtin_bit_cast(uint64_t, v), __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
                }
            }
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            int seen = 0;
            if (lane == 0) {
                seen = __hip_atomic_fetch_add(&counters[g], 1, __ATOMIC_RELAXED,
                                              __HIP_MEMORY_SCOPE_AGENT);
                last_flag = seen == wg_splits - 1;
            }
        }
        __syncthreads();
        if (!last_flag) return;
        asm volatile("" ::: "memory");
        half2_t sv, bv;
        if (svh) sv = *reinterpret_cast<const half2_t*>(svh + col);
        if (bias) bv = *reinterpret_cast<const half2_t*>(bias + col);
        for (int m = wave; m < rows; m += 4) {  // the finishing workgroup splits the batch rows
            // device-scope loads, sixteen partial rows in flight, added in split order
            const float* src = partial + (size_t)m * out_total + col;
            const size_t stride = (size_t)rows * out_total;
            float a = 0.f, b = 0.f;
            // (a batch that runs past the last partial row re-reads that row and drops
            // it: every batch is one round trip, whatever wg_splits is)
            for (int s = 0; s < wg_splits; s += 16) {
                uint64_t v[16];
#pragma unroll
                for (int i = 0; i < 16; i++)
                    v[i] = __hip_atomic_load(
                        reinterpret_cast<const uint64_t*>(src + (size_t)min(s + i, wg_splits - 1) * stride),
                        __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    if (s + i < wg_splits) {
                        const float2_t f = __builtin_bit_cast(float2_t, v[i]);
                        a = __fadd_rn(a, f.x);
                        b = __fadd_rn(b, f.y);
                    }
                }
            }
            a = (float)(half_t)a;
            b = (float)(half_t)b;
            wht128_lanes(a, b, lane);
            a = __fmul_rn(a, kHadScaleF);
            b = __fmul_rn(b, kHadScaleF);
            if (svh) {
                a = __fmul_rn(a, (float)sv.x);
                b = __fmul_rn(b, (float)sv.y);
            }
            half2_t o;
            o.x = (half_t)a;
            o.y = (half_t)b;
            if (bias) {
                o.x = o.x + bv.x;
                o.y = o.y + bv.y;
            }
            *reinterpret_cast<half2_t*>(y + (size_t)m * out_total + col) = o;
        }
        if (threadIdx.x == 0)
            __hip_atomic_store(&counters[g], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

// y[i] = sum over the partial rows, index order.
__global__ __launch_bounds__(256) void reduce_partials_kernel(const float* __restrict__ partial,
                                                              float* __restrict__ y, size_t n,
                                                              int n_splits) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    float s = partial[i];
    for (int k = 1; k < n_splits; k++) s = s + partial[(size_t)k * n + i];
    y[i] = s;
}

// Tuning knobs read once from the environment (the reference selects kernel
// variants the same way, ponyexl3/mlx/gemv_metal.py:1017-1020).
GemvPlan plan_gemv(int rows, int in_tiles, int n_groups) {
    (void)rows;
    // Aim for kWavesPerSimd waves per SIMD over the 256*4 SIMDs, but never fewer
    // than kMinTileRows tile rows per wave (pipeline depth, partial-sum traffic).
    // Measured on gate+up (272 groups): 4 waves/SIMD leaves workgroup counts like
    // 4.25 per CU, and the CUs that draw 5 set the kernel time; 12 dilutes that.
    static const int kWavesPerSimd = env_int("EXL3_GEMV_WAVES_PER_SIMD", 12, 1, 16);
    static const int kMinTileRows = env_int("EXL3_GEMV_MIN_TILE_ROWS", 8, 1, 4096);
    const int target_waves = 256 * 4 * kWavesPerSimd;
    int n_splits = target_waves / (n_groups > 0 ? n_groups : 1);
    if (n_splits < 1) n_splits = 1;
    int tk_per_split = (in_tiles + n_splits - 1) / n_splits;
    if (tk_per_split < kMinTileRows) tk_per_split = kMinTileRows;
    if (tk_per_split > in_tiles) tk_per_split = in_tiles;
    n_splits = (in_tiles + tk_per_split - 1) / tk_per_split;
    return GemvPlan{n_splits, tk_per_split};
}

// Plan of the one-launch layer kernel: splits are whole Hadamard blocks (8 tile
// rows) and every wave gets the same number of blocks where that divides.
GemvPlan plan_linear_small(int rows, int in_tiles, int n_groups, int K) {
    static const int kWavesPerSimd = env_int("EXL3_LINEAR_WAVES_PER_SIMD", 12, 1, 16);
    // From this K on a wave takes at least two blocks where that still leaves two waves
    // per SIMD. The kernel holds 7 waves per SIMD up to K = 4, 6 at K = 5..7 and 5 at
    // K = 8 (VGPRs), so one-block waves come in two to three rounds there; measured at
    // one row on 5120 -> 34816 / 17408 -> 5120: K = 5 38.4 -> 35.6 / 21.3 -> 21.0 us,
    // K = 6 43.3 -> 40.1 / 23.5 -> 22.2, K = 8 52.7 -> 47.5 / 29.0 -> 25.4 (K <= 4: no
    // gain or a loss).
    static const int kDeepFromK = env_int("EXL3_LINEAR_DEEP_FROM_K", 5, 1, 9);
    // one and two rows: when even one block per wave leaves fewer than this many waves
    // (four per SIMD), the waves take half blocks
    static const int kHalfBelow = env_int("EXL3_LINEAR_HALF_BELOW", 4096, 0, 1 << 20);
    const int target_waves = 256 * 4 * kWavesPerSimd;
    const int n_blocks = in_tiles / 8;
    // Half blocks double the waves, which evens out the load of the SIMDs when whole
    // blocks leave only a few waves on each (8192 -> 5120: 2560 whole-block waves are
    // two on half of the 1024 SIMDs and three on the others; 5120 half-block waves are
    // five everywhere), at the price of rotating every block twice. Cost per SIMD in
    // issue slots: (most waves on a SIMD) x (tile rows x 118 + 60 for the rotation).
    // The accumulator reduction has to be able to take the partial sums (eight-bit
    // count, atomics limit); with partial rows, 100+ rows per column group would cost
    // the finishing workgroup more than the balance gains.
    if (rows <= 2 && (long long)n_blocks * n_groups < kHalfBelow) {
        const long long whole = (long long)n_blocks * n_groups, n_simd = 1024;
        const long long cost_whole = ((whole + n_simd - 1) / n_simd) * (8 * 118 + 60);
        const long long cost_half = ((2 * whole + n_simd - 1) / n_simd) * (4 * 118 + 60);
        const GemvPlan half{n_blocks * 2, 4};
        if ((n_blocks <= 48 || linear_small_uses_atomics(rows, n_groups, half)) &&
            (n_blocks <= 48 || cost_half < cost_whole))
            return half;
    }
    int max_splits = target_waves / (n_groups > 0 ? n_groups : 1);
    if (max_splits < 1) max_splits = 1;
    if (max_splits > n_blocks) max_splits = n_blocks;
    int blocks_per_split = (n_blocks + max_splits - 1) / max_splits;
    const int n_splits = (n_blocks + blocks_per_split - 1) / blocks_per_split;
    blocks_per_split = (n_blocks + n_splits - 1) / n_splits;
    if (K >= kDeepFromK && blocks_per_split == 1 && n_blocks >= 2 &&
        (long long)n_groups * ((n_blocks + 1) / 2) >= 2048)
        return GemvPlan{(n_blocks + 1) / 2, 16};
    return GemvPlan{n_splits, blocks_per_split * 8};
}

// The atomic-accumulator reduction pays off while the launch issues few atomics:
// (column groups x partial rows per group x 128 columns x batch rows). Measured on
// the 27B-class shapes at one row: 33 k (4096 -> 4096) 9.1 -> 6.8 us, q+k+v
// 15.0 -> 13.2 us (205 k with half-block splits), 174 k (down) 20.7 -> 19.2 us, 348 k (gate+up) no gain; at 8 rows
// (2.8 M) the step got 13 % slower. At two rows the partial-row reduction is the
// more expensive one up to 8/3 of that limit (down 348 k: 20.6 -> 18.9 us, o_proj as
// half blocks 327 k: 11.7 -> 11.2 us, gate+up 696 k: no loss; the step 83.0 -> 79.8 us);
// at four rows neither limit gains (86.0 / 86.6 / 90.4 us at 300 k / 800 k / 1.6 M).
bool linear_small_uses_atomics(int rows, int n_groups, GemvPlan plan) {
    static const int kMaxAtomics = env_int("EXL3_LINEAR_MAX_ATOMICS", 300000, 0, 1 << 30);
    if (plan.n_partials() > 255) return false;  // the count field has eight bits
    const long long limit = rows == 2 ? (long long)kMaxAtomics * 8 / 3 : kMaxAtomics;
    return (long long)n_groups * plan.n_partials() * 128 * rows <= limit;
}

GemvPlan plan_linear_small_launch(int rows, int in_tiles, int n_groups, int K) {
    GemvPlan plan = plan_linear_small(rows, in_tiles, n_groups, K);
    if (rows == 1 && plan.tk_per_split >= 8 && !linear_small_uses_atomics(rows, n_groups, plan)) {
        GemvPlan wide = plan;
        wide.wg_waves = 8;
        if (linear_small_uses_atomics(rows, n_groups, wide)) plan = wide;
    }
    return plan;
}

int launch_gemv_partials(const uint16_t* xh, int rows, int n_sub, const uint16_t* trellis,
                         int in_tiles, int out_tiles, int K, int cb, const int32_t* group_sub,
                         const int32_t* group_tile, int n_groups, float* partial, GemvPlan plan,
                         hipStream_t stream) {
    if (int rc = check_k_cb(K, cb)) return rc;
    if (!xh || !trellis || !partial) return EXL3_E_NULL_POINTER;
    if (rows < 1 || rows > kGemvMaxRows || n_sub < 1 || in_tiles < 1 || out_tiles < 1 ||
        n_groups < 1 || in_tiles % 8 || out_tiles % 8)
        return EXL3_E_BAD_SHAPE;
    if (!group_tile && n_groups * 8 != out_tiles) return EXL3_E_BAD_SHAPE;
    if (n_sub > 1 && !group_sub) return EXL3_E_BAD_INDEX;
    if (plan.n_splits < 1 || plan.n_splits > 4 * 65535 || plan.tk_per_split < 1 ||
        (long long)plan.n_splits * plan.tk_per_split < in_tiles)
        return EXL3_E_BAD_SHAPE;
    const dim3 grid((unsigned)n_groups, (unsigned)((plan.n_splits + 3) / 4));
    const int mt = rows <= 1 ? 1 : rows <= 2 ? 2 : rows <= 4 ? 4 : 8;
    return dispatch_k_cb(K, cb, [&](auto k, auto c) {
        auto go = [&](auto mtc) {
            gemv_kernel<k.value, c.value, mtc.value><<<grid, dim3(256), 0, stream>>>(
                reinterpret_cast<const uint32_t*>(trellis), reinterpret_cast<const half_t*>(xh),
                partial, group_sub, group_tile, in_tiles, out_tiles, rows, n_sub, n_groups,
                plan.tk_per_split, plan.n_splits);
        };
        switch (mt) {
            case 1: go(std::integral_constant<int, 1>{}); break;
            case 2: go(std::integral_constant<int, 2>{}); break;
            case 4: go(std::integral_constant<int, 4>{}); break;
            default: go(std::integral_constant<int, 8>{}); break;
        }
        return launch_status();
    });
}

int launch_linear_small(const uint16_t* x, int rows, const uint16_t* trellis, int in_tiles,
                        int out_tiles, int K, int cb, const uint16_t* suh, int n_sub,
                        const int32_t* group_sub, const uint16_t* svh, const uint16_t* bias,
                        uint16_t* y, float* partial, int* counters, GemvPlan plan,
                        hipStream_t stream, int* status) {
    if (int rc = check_k_cb(K, cb)) return rc;
    if (!x || !trellis || !y || !counters) return EXL3_E_NULL_POINTER;
    const int spin_limit = reduction_spin_limit();
    const bool atomic = linear_small_uses_atomics(rows, out_tiles / 8, plan);
    if (atomic && (reinterpret_cast<uintptr_t>(counters) & 7)) return EXL3_E_BAD_SHAPE;
    if (!atomic && !partial) return EXL3_E_NULL_POINTER;
    if (rows < 1 || rows > kLinearSmallMaxRows || n_sub < 1 || in_tiles < 8 || out_tiles < 8 ||
        in_tiles % 8 || out_tiles % 8)
        return EXL3_E_BAD_SHAPE;
    if (n_sub > 1 && (!group_sub || !suh)) return EXL3_E_BAD_INDEX;
    const bool half = plan.tk_per_split == 4 && rows <= 2;
    if (plan.n_splits < 1 || plan.n_splits > 4 * 65535 ||
        (!half && (plan.tk_per_split < 8 || plan.tk_per_split % 8)) ||
        (long long)plan.n_splits * plan.tk_per_split < in_tiles)
        return EXL3_E_BAD_SHAPE;
    const int n_groups = out_tiles / 8;
    if (plan.wg_waves != 4 && !(plan.wg_waves == 8 && rows == 1 && !half && atomic))
        return EXL3_E_UNSUPPORTED;
    const dim3 grid((unsigned)n_groups, (unsigned)plan.n_partials());
    const int mt = rows <= 1 ? 1 : rows <= 2 ? 2 : rows <= 4 ? 4 : 8;
    return dispatch_k_cb(K, cb, [&](auto k, auto c) {
        auto go = [&](auto mtc, auto halfc) {
            auto launch = [&](auto atomicc) {
                linear_small_kernel<k.value, c.value, mtc.value, halfc.value, atomicc.value>
                    <<<grid, dim3(256), 0, stream>>>(
                        reinterpret_cast<const uint32_t*>(trellis),
                        reinterpret_cast<const half_t*>(x), reinterpret_cast<const half_t*>(suh),
                        reinterpret_cast<const half_t*>(svh), reinterpret_cast<const half_t*>(bias),
                        reinterpret_cast<half_t*>(y), partial, counters, group_sub, in_tiles,
                        out_tiles, rows, n_groups, plan.tk_per_split, plan.n_splits, status,
                        spin_limit);
            };
            if (atomic) launch(std::true_type{});
            else launch(std::false_type{});
        };
        if (plan.wg_waves == 8) {  // one row, whole blocks, accumulators (checked above)
            linear_small_kernel<k.value, c.value, 1, false, true, 8>
                <<<grid, dim3(512), 0, stream>>>(
                    reinterpret_cast<const uint32_t*>(trellis), reinterpret_cast<const half_t*>(x),
                    reinterpret_cast<const half_t*>(suh), reinterpret_cast<const half_t*>(svh),
                    reinterpret_cast<const half_t*>(bias), reinterpret_cast<half_t*>(y), partial,
                    counters, group_sub, in_tiles, out_tiles, rows, n_groups, plan.tk_per_split,
                    plan.n_splits, status, spin_limit);
            return launch_status();
        }
        using T = std::true_type;
        using F = std::false_type;
        switch (mt) {
            case 1:
                if (half) go(std::integral_constant<int, 1>{}, T{});
                else go(std::integral_constant<int, 1>{}, F{});
                break;
            case 2:
                if (half) go(std::integral_constant<int, 2>{}, T{});
                else go(std::integral_constant<int, 2>{}, F{});
                break;
            case 4: go(std::integral_constant<int, 4>{}, F{}); break;
            default: go(std::integral_constant<int, 8>{}, F{}); break;
        }
        return launch_status();
    });
}

}  // namespace exl3

EXL3_EXPORT int exl3_gemv_max_rows(void) { return exl3::kGemvMaxRows; }

EXL3_EXPORT int exl3_linear_small_max_rows(void) {
    // the medium-batch kernel continues where the small-batch one ends
    const int mid = exl3::linear_mid_max_rows();
    return mid > exl3::kLinearSmallMaxRows ? mid : exl3::kLinearSmallMaxRows;
}

EXL3_EXPORT size_t exl3_gemv_workspace_bytes(int rows, int in_tiles, int n_groups) {
    if (rows < 1 || in_tiles < 1 || n_groups < 1) return 0;
    const exl3::GemvPlan plan = exl3::plan_gemv(rows, in_tiles, n_groups);
    return (size_t)plan.n_partials() * rows * n_groups * 128 * sizeof(float);
}

EXL3_EXPORT int exl3_gemv_plan(int rows, int in_tiles, int n_groups, int* n_splits,
                               int* tile_rows_per_split) {
    if (rows < 1 || rows > exl3::kGemvMaxRows || in_tiles < 1 || n_groups < 1)
        return EXL3_E_BAD_SHAPE;
    const exl3::GemvPlan plan = exl3::plan_gemv(rows, in_tiles, n_groups);
    if (n_splits) *n_splits = plan.n_partials();
    if (tile_rows_per_split) *tile_rows_per_split = plan.tk_per_split;
    return EXL3_OK;
}

EXL3_EXPORT int exl3_linear_plan(int rows, int in_tiles, int out_tiles, int K, int* n_splits,
                                 int* tile_rows_per_split, int* waves_per_workgroup, int* atomic) {
    using namespace exl3;
    if (rows < 1 || rows > kLinearSmallMaxRows || in_tiles < 8 || out_tiles < 8 || in_tiles % 8 ||
        out_tiles % 8 || K < 1 || K > 8)
        return EXL3_E_BAD_SHAPE;
    const GemvPlan plan = plan_linear_small_launch(rows, in_tiles, out_tiles / 8, K);
    if (n_splits) *n_splits = plan.n_splits;
    if (tile_rows_per_split) *tile_rows_per_split = plan.tk_per_split;
    if (waves_per_workgroup) *waves_per_workgroup = plan.wg_waves;
    if (atomic) *atomic = linear_small_uses_atomics(rows, out_tiles / 8, plan) ? 1 : 0;
    return EXL3_OK;
}

EXL3_EXPORT int exl3_gemv_partials(const uint16_t* xh, int rows, int n_sub, const uint16_t* trellis,
                                   int in_tiles, int out_tiles, int K, int cb,
                                   const int32_t* group_sub, const int32_t* group_tile,
                                   int n_groups, float* partial, size_t partial_bytes,
                                   void* stream) {
    using namespace exl3;
    if (rows < 1 || rows > kGemvMaxRows || in_tiles < 1 || n_groups < 1) return EXL3_E_BAD_SHAPE;
    const GemvPlan plan = plan_gemv(rows, in_tiles, n_groups);
    if (partial_bytes < (size_t)plan.n_partials() * rows * n_groups * 128 * sizeof(float))
        return EXL3_E_WORKSPACE;
    return launch_gemv_partials(xh, rows, n_sub, trellis, in_tiles, out_tiles, K, cb, group_sub,
                                group_tile, n_groups, partial, plan, as_stream(stream));
}

EXL3_EXPORT int exl3_gemv(const uint16_t* xh, int rows, int n_sub, const uint16_t* trellis,
                          int in_tiles, int out_tiles, int K, int cb, const int32_t* group_sub,
                          const int32_t* group_tile, int n_groups, float* y_out, void* workspace,
                          size_t workspace_bytes, void* stream) {
    using namespace exl3;
    if (!y_out) return EXL3_E_NULL_POINTER;
    if (rows < 1 || rows > kGemvMaxRows || in_tiles < 1 || n_groups < 1) return EXL3_E_BAD_SHAPE;
    const GemvPlan plan = plan_gemv(rows, in_tiles, n_groups);
    hipStream_t s = as_stream(stream);
    if (plan.n_partials() == 1)
        return launch_gemv_partials(xh, rows, n_sub, trellis, in_tiles, out_tiles, K, cb, group_sub,
                                    group_tile, n_groups, y_out, plan, s);
    if (!workspace) return EXL3_E_NULL_POINTER;
    if (workspace_bytes < exl3_gemv_workspace_bytes(rows, in_tiles, n_groups))
        return EXL3_E_WORKSPACE;
    float* partial = reinterpret_cast<float*>(workspace);
    if (int rc = launch_gemv_partials(xh, rows, n_sub, trellis, in_tiles, out_tiles, K, cb,
                                      group_sub, group_tile, n_groups, partial, plan, s))
        return rc;
    const size_t n = (size_t)rows * n_groups * 128;
    reduce_partials_kernel<<<dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s>>>(partial, y_out, n,
                                                                                 plan.n_partials());
    return launch_status();
}
