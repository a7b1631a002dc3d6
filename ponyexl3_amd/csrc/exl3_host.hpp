// Host-side plumbing shared by the translation units of libexl3_hip.so:
// argument checks, (K, codebook) template dispatch and the internal launchers
// that the composite entry points (exl3_linear_forward, exl3_moe_forward) chain.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>

#include "../../include/exl3_hip.h"

#define EXL3_EXPORT extern "C" __attribute__((visibility("default")))

namespace exl3 {

inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }

inline int launch_status() { return hipGetLastError() == hipSuccess ? EXL3_OK : EXL3_E_LAUNCH; }

inline int check_k_cb(int K, int cb) {
    if (K < 1 || K > 8) return EXL3_E_BAD_K;
    if (cb < 0 || cb > 2) return EXL3_E_BAD_CODEBOOK;
    return EXL3_OK;
}

// Calls f(integral_constant<int,K>, integral_constant<int,CB>) for runtime K, cb.
template <typename F>
inline int dispatch_k_cb(int K, int cb, F&& f) {
#define EXL3_CASE_CB(KV)                                                                   \
    switch (cb) {                                                                          \
        case 0: return f(std::integral_constant<int, KV>{}, std::integral_constant<int, 0>{}); \
        case 1: return f(std::integral_constant<int, KV>{}, std::integral_constant<int, 1>{}); \
        case 2: return f(std::integral_constant<int, KV>{}, std::integral_constant<int, 2>{}); \
        default: return EXL3_E_BAD_CODEBOOK;                                               \
    }
    switch (K) {
        case 1: EXL3_CASE_CB(1)
        case 2: EXL3_CASE_CB(2)
        case 3: EXL3_CASE_CB(3)
        case 4: EXL3_CASE_CB(4)
        case 5: EXL3_CASE_CB(5)
        case 6: EXL3_CASE_CB(6)
        case 7: EXL3_CASE_CB(7)
        case 8: EXL3_CASE_CB(8)
        default: return EXL3_E_BAD_K;
    }
#undef EXL3_CASE_CB
}

constexpr int kGemvMaxRows = 8;

// Split-K plan of the small-batch kernel: the tile rows [0, in_tiles) are cut
// into n_splits ranges of tk_per_split rows; every (128-column group, split)
// pair is one workgroup.
struct GemvPlan {
    int n_splits;      // wave-level splits of the tile rows
    int tk_per_split;  // tile rows per split
    int wg_waves = 4;  // waves per workgroup (4; the one-launch layer kernel also has 8)
    // the waves of a workgroup are summed in LDS: partial rows per group
    int n_partials() const { return (n_splits + wg_waves - 1) / wg_waves; }
};
GemvPlan plan_gemv(int rows, int in_tiles, int n_groups);
GemvPlan plan_linear_small(int rows, int in_tiles, int n_groups, int K = 4);

// partial: fp32 [plan.n_partials()][rows][128*n_groups]
int launch_gemv_partials(const uint16_t* xh, int rows, int n_sub, const uint16_t* trellis,
                         int in_tiles, int out_tiles, int K, int cb, const int32_t* group_sub,
                         const int32_t* group_tile, int n_groups, float* partial, GemvPlan plan,
                         hipStream_t stream);

// One-launch small-batch layer (rows <= kLinearSmallMaxRows). The kernel rotates x
// itself. Its split reduction is one of two: 64-bit fixed-point accumulators
// (uint64 [rows][16*out_tiles], living in `counters`, 8-byte aligned; `partial`
// unused) when linear_small_uses_atomics(), else fp32 partial rows
// [plan.n_partials()][rows][out] in `partial` plus counters[out_tiles/8]. Either way
// the counters array must be zero on entry and is zero again on exit;
// linear_small_counter_ints() is the length that serves both.
constexpr int kLinearSmallMaxRows = kGemvMaxRows;
bool linear_small_uses_atomics(int rows, int n_groups, GemvPlan plan);
// plan_linear_small with the reduction in mind: one row on a large layer takes
// workgroups of eight waves when that brings the launch under the atomics limit.
GemvPlan plan_linear_small_launch(int rows, int in_tiles, int n_groups, int K = 4);
inline size_t linear_small_counter_ints(int rows, int out_features) {
    return 2 * (size_t)rows * out_features;  // >= out_features / 128
}
int launch_linear_small(const uint16_t* x, int rows, const uint16_t* trellis, int in_tiles,
                        int out_tiles, int K, int cb, const uint16_t* suh, int n_sub,
                        const int32_t* group_sub, const uint16_t* svh, const uint16_t* bias,
                        uint16_t* y, float* partial, int* counters, GemvPlan plan,
                        hipStream_t stream, int* status = nullptr);
// `status` (device, may be NULL): set to non-zero by a finishing workgroup of the
// accumulator reduction whose bounded wait for the other contributors ran out.

// Medium-batch layer (rows <= kLinearMidMaxRows) on rotated activations xh, fp16
// [rows][n_sub][in]: weights decoded once and fed to 16x16x16 MFMA from registers;
// partial: fp32 [plan.n_splits][rows][out]; counters as for launch_linear_small.
constexpr int kLinearMidMaxRows = 32;
struct MidPlan {
    int n_splits;          // workgroups per 128-column group
    int blocks_per_split;  // 128-row blocks of the reduction per workgroup
};
MidPlan plan_linear_mid(int rows, int in_tiles, int n_groups);
// Largest row count that exl3_linear_forward sends to it (it starts above
// kLinearSmallMaxRows; a value below that switches it off).
int linear_mid_max_rows();
int launch_linear_mid(const uint16_t* xh, int rows, const uint16_t* trellis, int in_tiles,
                      int out_tiles, int K, int cb, int n_sub, const int32_t* group_sub,
                      const uint16_t* svh, const uint16_t* bias, uint16_t* y, float* partial,
                      int* counters, MidPlan plan, hipStream_t stream);

int launch_had_pre(const uint16_t* x, int rows, int n, const uint16_t* suh, int n_sub,
                   uint16_t* xh, hipStream_t stream);

int launch_had_post(const void* y, int y_is_fp32, int n_sum, size_t sum_stride, int rows, int n,
                    const uint16_t* svh, const uint16_t* bias, uint16_t* out, hipStream_t stream);

// Tile schedule of the prefill GEMM: block tiles of (32*mi) rows x 256 columns are
// dealt to the CUs in rounds; the `split_tiles` tiles of a partly filled last round
// are cut along the reduction into `split_runs` runs of `split_per` 64-deep steps,
// one workgroup each, whose fp32 partial tiles a second kernel adds up: either
// `split_runs_per_tile` runs per tile, or (0) the tiles' steps end to end in equally
// long runs that may cross from one tile into the next (`split_pitch`: positions from
// one tile's first step to the next tile's).
struct GemmPlan {
    int mi;  // 16-row accumulator tiles per wave: 8, 4 or 2 (256-, 128- or 64-row blocks)
    int n_row_blocks, n_col_blocks;
    int full_tiles, split_tiles;
    int split_runs, split_per, split_pitch, split_runs_per_tile;
};
GemmPlan plan_gemm(int rows, int in_tiles, int tn_count, bool allow_split);
size_t gemm_workspace_bytes(int rows, int in_tiles, int tn_count);

// Output transform the GEMM may fold into its fix-up pass: when every tile of the
// launch is split along the reduction dimension (few rows), the kernel that adds
// the partial tiles also applies the output Hadamard, svh and bias and writes
// `out` [rows][ldo] directly (tn_offset must be 0 and tn_count the whole width).
struct GemmPost {
    const uint16_t* svh;   // fp16 [16*tn_count] or NULL
    const uint16_t* bias;  // fp16 [16*tn_count] or NULL
    uint16_t* out;
    size_t ldo;
};

// workspace may be NULL (or too small): then no tile is split. If `post` is given
// and could be applied, *post_done is set and y_out is left untouched; otherwise
// y_out holds the plain product and the caller runs the output transform.
int launch_gemm(const uint16_t* xh, int rows, size_t ldx, const uint16_t* trellis, int in_tiles,
                int out_tiles, int K, int cb, int tn_offset, int tn_count, uint16_t* y_out,
                size_t ldy, void* workspace, size_t workspace_bytes, hipStream_t stream,
                const GemmPost* post = nullptr, bool* post_done = nullptr,
                const int32_t* block_sub = nullptr, size_t sub_stride = 0);
// block_sub (device, one entry per 256-column block of the slice, or NULL): the
// block multiplies xh + block_sub[g] * sub_stride instead of xh (stacked rotations
// of a sibling-fused layer).

int launch_gemm_grouped(const uint16_t* xh, int n_rows, size_t ldx, const uint16_t* trellis,
                        int in_tiles, int out_tiles, int K, int cb, int tn_base, int group_tiles,
                        int n_groups, const int32_t* group_tab, int n_row_blocks, int block_rows,
                        uint16_t* y_out, size_t ldy, hipStream_t stream);

int launch_had_rows(const uint16_t* x, int n_in_rows, int rows, int n, const int32_t* in_index,
                    const uint16_t* scale, int n_scale_rows, const int32_t* scale_index,
                    size_t scale_ld, int post, uint16_t* out, int n_out_rows,
                    const int32_t* out_index, hipStream_t stream);

inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

// Integer tuning knob from the environment, clamped to [lo, hi].
inline int env_int(const char* name, int dflt, int lo, int hi) {
    const char* v = getenv(name);
    if (!v || !*v) return dflt;
    const int x = atoi(v);
    return x < lo ? lo : (x > hi ? hi : x);
}

// EXL3_EXACT_WEIGHTS=1: every product uses the weight rounded to fp16, as the reference
// defines it. The one-launch layer kernel and the down projection of the MoE chain
// multiply by the exact sum of the weight's two fp16 halves instead (one VALU instruction
// less per weight; 4-5e-4 rel-L2 on a layer's output, against 5-7e-5); with the knob set
// the entry points take their multi-launch chains, whose kernels round first.
inline bool exact_weights() {
    static const int v = env_int("EXL3_EXACT_WEIGHTS", 0, 0, 1);
    return v != 0;
}

// Polls a finishing workgroup spends on accumulators whose counts are not complete yet
// before it gives up (EXL3_SPIN_LIMIT; read at every launch so that a test can lower it).
inline int reduction_spin_limit() { return env_int("EXL3_SPIN_LIMIT", 1 << 22, 1, 1 << 30); }

// Where the status word of a counters array lives: its last int, if the array is at
// least two ints longer than the launch needs (so that no accumulator shares it).
inline int* counters_status_word(int32_t* counters, size_t counters_len, size_t needed) {
    return counters && counters_len >= needed + 2 ? counters + (counters_len - 1) : nullptr;
}

}  // namespace exl3
