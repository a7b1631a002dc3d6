// Small-batch fused trellis-decode GEMV (rows 1..8): y = xh @ W_inner with the
// weights decoded in registers straight from the packed bitstream.
//
// Work decomposition
//   * the unit of work is a wavefront: wave (g, s) owns the 128-column output
//     group g and split s of the tile rows, tk in [s*L, min(in_tiles, (s+1)*L));
//     the four waves of a workgroup are four consecutive splits of one group and
//     never talk to each other (no LDS, no barrier);
//   * per tile row a wave issues one wave-wide non-temporal load of 256*K
//     contiguous bytes (8 tiles) and keeps kPrefetch such loads in flight; lane
//     u of a tile decodes its 32 codewords = output columns u and u+8 over all 16
//     input rows and keeps two fp32 accumulators per batch row, so no
//     cross-lane reduction exists anywhere;
//   * activations of a tile row are wave-uniform (scalar loads) and enter
//     v_dot2_f32_f16 as SGPR operands;
//   * every wave writes one fp32 partial row [split][row][128 columns]; splits
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

#include <stdlib.h>

namespace exl3 {

constexpr int kPrefetch = 4;  // wave-wide loads in flight per wave

template <int K>
__device__ __forceinline__ void load_lane_words_nt(const uint32_t* __restrict__ p,
                                                   uint32_t (&own)[K]) {
#pragma unroll
    for (int i = 0; i < K; i++) own[i] = __builtin_nontemporal_load(p + i);
}

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
    if (split >= n_splits) return;
    const int tn0 = group_tile ? group_tile[g] : g * 8;
    const int sub = group_sub ? group_sub[g] : 0;
    const int in_features = in_tiles * 16;
    const int tk_begin = split * tk_per_split;
    const int tk_end = min(in_tiles, tk_begin + tk_per_split);
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
    auto consume = [&](const uint32_t (&words)[K], int tk) {
        const LaneWords<K> lw = finish_lane_words<K>(words, lane);
        half2_t wp[16];
        decode_lane<K, CB>(lw, wp);
#pragma unroll
        for (int m = 0; m < MT; m++) {
            const half2_t* xp = reinterpret_cast<const half2_t*>(xrow[m] + tk * 16);
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const half2_t xv = xp[j];
                acc[m][0] = dot2(wp[j], xv, acc[m][0]);
                acc[m][1] = dot2(wp[8 + j], xv, acc[m][1]);
            }
        }
    };

    uint32_t buf[kPrefetch][K];
#pragma unroll
    for (int s = 0; s < kPrefetch; s++) {
        const int t = min(tk_begin + s, tk_end - 1);  // clamped: stays inside the split
        load_lane_words_nt<K>(base + (size_t)t * row_words, buf[s]);
    }
    int tk0 = tk_begin;
    for (; tk0 + kPrefetch <= tk_end; tk0 += kPrefetch) {
#pragma unroll
        for (int s = 0; s < kPrefetch; s++) {
            consume(buf[s], tk0 + s);
            const int tn = min(tk0 + s + kPrefetch, tk_end - 1);
            load_lane_words_nt<K>(base + (size_t)tn * row_words, buf[s]);
        }
    }
#pragma unroll
    for (int s = 0; s < kPrefetch - 1; s++)
        if (tk0 + s < tk_end) consume(buf[s], tk0 + s);

    const int c0 = (lane >> 3) * 16 + (lane & 7);
    const size_t out_total = (size_t)n_groups * 128;
#pragma unroll
    for (int m = 0; m < MT; m++) {
        if (m < rows) {
            float* dst = partial + ((size_t)split * rows + m) * out_total + (size_t)g * 128 + c0;
            dst[0] = acc[m][0];
            dst[8] = acc[m][1];
        }
    }
}

// y[i] = sum over splits, index order.
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
static int env_int(const char* name, int dflt, int lo, int hi) {
    const char* v = getenv(name);
    if (!v || !*v) return dflt;
    const int x = atoi(v);
    return x < lo ? lo : (x > hi ? hi : x);
}

GemvPlan plan_gemv(int rows, int in_tiles, int n_groups) {
    (void)rows;
    // All waves of a launch should be resident together and carry equal work:
    // aim for kWavesPerSimd waves on each of the 256*4 SIMDs, but never fewer
    // than kMinTileRows tile rows per wave (pipeline depth, partial-sum traffic).
    static const int kWavesPerSimd = env_int("EXL3_GEMV_WAVES_PER_SIMD", 4, 1, 16);
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

}  // namespace exl3

EXL3_EXPORT int exl3_gemv_max_rows(void) { return exl3::kGemvMaxRows; }

EXL3_EXPORT size_t exl3_gemv_workspace_bytes(int rows, int in_tiles, int n_groups) {
    if (rows < 1 || in_tiles < 1 || n_groups < 1) return 0;
    const exl3::GemvPlan plan = exl3::plan_gemv(rows, in_tiles, n_groups);
    return (size_t)plan.n_splits * rows * n_groups * 128 * sizeof(float);
}

EXL3_EXPORT int exl3_gemv_plan(int rows, int in_tiles, int n_groups, int* n_splits,
                               int* tile_rows_per_split) {
    if (rows < 1 || rows > exl3::kGemvMaxRows || in_tiles < 1 || n_groups < 1)
        return EXL3_E_BAD_SHAPE;
    const exl3::GemvPlan plan = exl3::plan_gemv(rows, in_tiles, n_groups);
    if (n_splits) *n_splits = plan.n_splits;
    if (tile_rows_per_split) *tile_rows_per_split = plan.tk_per_split;
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
    if (partial_bytes < (size_t)plan.n_splits * rows * n_groups * 128 * sizeof(float))
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
    if (plan.n_splits == 1)
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
                                                                                 plan.n_splits);
    return launch_status();
}
