/*
 * C ABI of the MI355X (gfx950) EXL3 quantized-linear library, libexl3_hip.so.
 *
 * Every entry point takes raw device pointers, sizes and a HIP stream
 * (hipStream_t passed as void*, NULL = the default stream) and returns an int
 * status: 0 on success, a negative EXL3_E_* code otherwise. Nothing throws
 * across the boundary and nothing is allocated or freed by the library: the
 * caller owns every buffer, including the workspace. All launches are
 * asynchronous on the given stream. Argument checks happen on the host before
 * any launch, mirroring the reference, whose kernels have no error channel and
 * whose host wrappers raise ValueError first
 * (ponyexl3/ref/layer.py:35-44, ponyexl3/mlx/gemv_metal.py:1354-1372).
 *
 * Tensor contract (ponyexl3/ref/layer.py:12-44):
 *   trellis  uint16 [in_tiles][out_tiles][16*K], in_tiles = in/16, out_tiles = out/16
 *   suh/svh  fp16 per-channel multipliers [in] / [out] (general scales, not only +-1)
 *   K        bits per weight, 1..8
 *   cb       codebook id: 0 = 3INST (default), 1 = MCG, 2 = MUL1
 *            (ponyexl3/ref/codebook.py:9-12)
 *   W_inner  fp16 [in][out] row-major; y = xh @ W_inner
 * fp16 buffers are passed as uint16_t* (bit patterns).
 */
#ifndef EXL3_HIP_H
#define EXL3_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define EXL3_OK 0
#define EXL3_E_BAD_K (-1)         /* K outside 1..8 */
#define EXL3_E_BAD_CODEBOOK (-2)  /* cb outside 0..2 */
#define EXL3_E_BAD_SHAPE (-3)     /* sizes not multiples of 16 / 128, slice out of range, rows out of range */
#define EXL3_E_NULL_POINTER (-4)  /* a required pointer is NULL */
#define EXL3_E_WORKSPACE (-5)     /* workspace smaller than exl3_workspace_bytes() reports */
#define EXL3_E_LAUNCH (-6)        /* hipGetLastError() was not hipSuccess after a launch */
#define EXL3_E_BAD_INDEX (-7)     /* tile_sub / expert index table inconsistent */
#define EXL3_E_UNSUPPORTED (-8)   /* valid request this build has no kernel for */
#define EXL3_E_STATIC_LIMIT (-9)  /* exl3_linear_forward_static: beyond its built-in scratch */
#define EXL3_E_INCOMPLETE (-10)   /* exl3_counters_status: a split reduction gave up waiting */

/* Library version (major*10000 + minor*100 + patch). */
int exl3_version(void);

/* Human-readable text for a status code; never NULL. */
const char *exl3_status_string(int status);

/* Largest row count the small-batch kernel (exl3_gemv) accepts per call. */
int exl3_gemv_max_rows(void);

/* Largest row count exl3_linear_forward serves with its small- and medium-batch
 * kernels when given counters (stacked suh included; above exl3_gemv_max_rows()
 * the input rotation runs as a launch of its own first). Beyond it the prefill
 * GEMM takes over. */
int exl3_linear_small_max_rows(void);

/*
 * Trellis -> fp16 W_inner for a slice of tile columns.
 * Replaces decode_full_mlx (ponyexl3/mlx/gemv_metal.py:717-743) and the CPU
 * decode_packed_trellis (ponyexl3/ref/decode.py:32-81). Bit-exact with both.
 *   w_out   fp16 [16*in_tiles][16*tn_count] row-major
 */
int exl3_decode_full(const uint16_t *trellis, int in_tiles, int out_tiles, int K, int cb,
                     int tn_offset, int tn_count, uint16_t *w_out, void *stream);

/*
 * Stacked-expert trellis -> contiguous per-expert matrices: tile column t goes to
 * expert t / tiles_per_e. Replaces decode_full_eg_mlx
 * (ponyexl3/mlx/gemv_metal.py:746-774). out_tiles must be a multiple of tiles_per_e.
 *   w_out   fp16 [out_tiles/tiles_per_e][16*in_tiles][16*tiles_per_e]
 */
int exl3_decode_full_eg(const uint16_t *trellis, int in_tiles, int out_tiles, int K, int cb,
                        int tiles_per_e, uint16_t *w_out, void *stream);

/*
 * Trellis -> fp16 W_inner transposed, for a slice of tile columns. Replaces
 * decode_full_t_mlx (ponyexl3/mlx/gemv_metal.py:841-866).
 *   w_out_t fp16 [16*tn_count][16*in_tiles] row-major
 */
int exl3_decode_full_t(const uint16_t *trellis, int in_tiles, int out_tiles, int K, int cb,
                       int tn_offset, int tn_count, uint16_t *w_out_t, void *stream);

/*
 * Input-side Hadamard-128 with per-channel multipliers, fp32 butterflies:
 *   xh[r][s][:] = fp16( H128/sqrt(128) applied per 128-block to (x[r][:] * suh[s][:]) )
 * Replaces EXL3LayerRuntime.prepare_xh (ponyexl3/mlx/layer_state.py:133-136),
 * the stacked-suh _fused_prep (ponyexl3/mlx/exl3_fused.py:44-60) and the
 * pre_scale half of had_r_128 (ponyexl3/ref/hadamard.py:50-80, used at
 * ponyexl3/ref/forward.py:34).
 *   x     fp16 [rows][n]
 *   suh   fp16 [n_sub][n], or NULL (then n_sub must be 1 and no multiply happens)
 *   xh    fp16 [rows][n_sub][n]
 */
int exl3_had128_pre(const uint16_t *x, int rows, int n, const uint16_t *suh, int n_sub,
                    uint16_t *xh, void *stream);

/*
 * Hadamard-128 with one scale vector per row (rows routed to different experts),
 * with the row gathers and the final scatter of the sorted MoE prefill folded in:
 *   post == 0: out[o(r)] = fp16(had128(x[i(r)] * scale[s(r)]))  (_rows_prep,
 *              ponyexl3/mlx/exl3_moe.py:105-119, with the x_pairs / suh gathers of :706-709)
 *   post != 0: out[o(r)] = fp16(had128(x[i(r)]) * scale[s(r)])  (_rows_finish,
 *              ponyexl3/mlx/exl3_moe.py:122-136, with the unsort of :768)
 *   i = in_index, s = scale_index, o = out_index: device int32[rows], or NULL for
 *   the identity; scale rows are scale_ld elements apart (a multiple of 8).
 * x has n_in_rows rows, scale n_scale_rows, out n_out_rows: a table entry outside its
 * range (negative included) makes the kernel skip that row - nothing is read or
 * written for it - and with a NULL table `rows` must not exceed the buffer's rows
 * (EXL3_E_BAD_SHAPE).
 * x, out fp16 rows of n elements (n a multiple of 128); x, scale, out 16-byte aligned.
 */
int exl3_had128_rows(const uint16_t *x, int n_in_rows, int rows, int n, const int32_t *in_index,
                     const uint16_t *scale, int n_scale_rows, const int32_t *scale_index,
                     size_t scale_ld, int post, uint16_t *out, int n_out_rows,
                     const int32_t *out_index, void *stream);

/*
 * Output-side Hadamard-128: optional split-K reduction, the fp16 cast of the
 * matmul result, the transform, svh and bias:
 *   t   = fp16( sum_{i < n_sum} y[i][r][:] )      (ponyexl3/ref/forward.py:41)
 *   out = fp16( had128(t) * svh ) (+ bias, fp16 add)  (ponyexl3/ref/forward.py:42-45)
 * Replaces EXL3LayerRuntime.finish_y (ponyexl3/mlx/layer_state.py:138-141),
 * _fused_finish (ponyexl3/mlx/exl3_fused.py:63-76) and the partial-sum
 * reduction of ponyexl3/mlx/gemv_metal.py:1454-1457. Slices are added in index
 * order, so the result is deterministic.
 *   y           fp32 [n_sum][rows][n] (y_is_fp32 = 1, slice stride sum_stride
 *               elements) or fp16 [rows][n] (y_is_fp32 = 0, n_sum must be 1)
 *   svh, bias   fp16 [n] or NULL
 *   out         fp16 [rows][n]; may alias y when y is fp16
 */
int exl3_had128_post(const void *y, int y_is_fp32, int n_sum, size_t sum_stride, int rows, int n,
                     const uint16_t *svh, const uint16_t *bias, uint16_t *out, void *stream);

/*
 * Small-batch fused trellis-decode GEMV/GEMM: y[m] = xh[m, sub(g)] @ W_inner,
 * fp32 accumulation, rows <= exl3_gemv_max_rows().
 * Replaces inner_gemv_mlx / inner_gemm_mlx / inner_gem_fused_mlx
 * (ponyexl3/mlx/gemv_metal.py:1495-1515, 1481-1492) including the split-K
 * chooser (:1405-1414) and the host-side partial sum (:1454-1457).
 *
 *   xh          fp16 [rows][n_sub][in] rotated activations
 *   group_sub   int32 [out_tiles/8] or NULL: which of the n_sub activation rows
 *               the 128-column group g multiplies (tile_sub of
 *               ponyexl3/mlx/exl3_fused.py:107-125 at 128-column granularity)
 *   group_tile  int32 [n_groups] or NULL: first tile column of each 128-column
 *               group inside the trellis (tile_map of
 *               ponyexl3/mlx/exl3_moe.py:139-171 at 128-column granularity);
 *               NULL = groups 0..out_tiles/8-1 in order
 *   n_groups    number of 128-column output groups produced (out = 128*n_groups)
 *   y_out       fp32 [rows][128*n_groups]; partial sums are reduced in a fixed
 *               order, so results are run-to-run deterministic
 *   workspace   device scratch of at least exl3_gemv_workspace_bytes(...)
 */
int exl3_gemv(const uint16_t *xh, int rows, int n_sub, const uint16_t *trellis, int in_tiles,
              int out_tiles, int K, int cb, const int32_t *group_sub, const int32_t *group_tile,
              int n_groups, float *y_out, void *workspace, size_t workspace_bytes, void *stream);

size_t exl3_gemv_workspace_bytes(int rows, int in_tiles, int n_groups);

/*
 * The split-K plan exl3_gemv uses for a shape, and the decode-GEMV kernel on
 * its own: writes the per-split fp32 partial sums without reducing them, the
 * form the reference's launcher returns before its host-side sum
 * ((n_splits, out) at ponyexl3/mlx/gemv_metal.py:1431-1457). The caller adds
 * the slices in index order (exl3_had128_post does, fused with the output
 * transform). One kernel launch, so it can be timed in isolation.
 *   partial   fp32 [n_splits][rows][128*n_groups], n_splits from exl3_gemv_plan
 */
int exl3_gemv_plan(int rows, int in_tiles, int n_groups, int *n_splits, int *tile_rows_per_split);

int exl3_gemv_partials(const uint16_t *xh, int rows, int n_sub, const uint16_t *trellis,
                       int in_tiles, int out_tiles, int K, int cb, const int32_t *group_sub,
                       const int32_t *group_tile, int n_groups, float *partial,
                       size_t partial_bytes, void *stream);

/*
 * Prefill GEMM: y = xh @ W_inner for rows > exl3_gemv_max_rows(), trellis tiles
 * decoded into LDS and contracted on fp16 MFMA with fp32 accumulation.
 * Replaces the rows > 16 branches of EXL3Linear.__call__
 * (ponyexl3/mlx/exl3_linear.py:137-161: staged fused GEMM, decode_full + matmul,
 * striped matmul).
 *   xh      fp16 [rows][ldx] (ldx >= in, elements)
 *   y_out   fp16 [rows][ldy] written at column offset 0 (ldy >= out); the fp32
 *           accumulator is rounded once (the cast at ponyexl3/ref/forward.py:41)
 *   workspace  device scratch of exl3_gemm_workspace_bytes(rows, in_tiles, tn_count)
 *           bytes, 16-byte aligned, for the fp32 partial tiles of block tiles that
 *           are split along the reduction dimension to fill the last round of
 *           CUs (the reference's small-batch kernels split K for the same reason,
 *           ponyexl3/mlx/gemv_metal.py:1405-1414).
 *           NULL or too small: no tile is split (slower on some shapes, same result
 *           up to the order of fp32 additions).
 */
int exl3_gemm(const uint16_t *xh, int rows, size_t ldx, const uint16_t *trellis, int in_tiles,
              int out_tiles, int K, int cb, int tn_offset, int tn_count, uint16_t *y_out,
              size_t ldy, void *workspace, size_t workspace_bytes, void *stream);

/*
 * Prefill GEMM over rows that are sorted into groups (experts), each group
 * multiplying its own tile columns of a stacked trellis: the segmented GEMM of
 * the MoE prefill path (inner_mm_seg_mlx, ponyexl3/mlx/gemv_metal.py:1685-1741,
 * called from EXL3SwitchGLU._prefill, ponyexl3/mlx/exl3_moe.py:684-768).
 *   xh         fp16 [n_rows][ldx], rows of one group contiguous
 *   group g multiplies tile columns [tn_base + g*group_tiles, + group_tiles)
 *   group_tab  device int32 [n_row_blocks][4] = {group, first row, end row, 0}: row
 *              blocks of at most block_rows (64, 128 or 256) rows that never span
 *              two groups; first row == end row marks an unused entry (the
 *              reference builds the same table on the device and sizes it for
 *              the worst case, ponyexl3/mlx/exl3_moe.py:79-98, 722-723)
 *   y_out      fp16 [n_rows][ldy] (ldy >= 16*group_tiles), same row order as xh
 * The table comes from device memory and is checked by the kernel: an entry whose
 * group is outside [0, n_groups) or whose first row is negative is skipped, and its
 * end row is clamped to n_rows.
 */
int exl3_gemm_grouped(const uint16_t *xh, int n_rows, size_t ldx, const uint16_t *trellis,
                      int in_tiles, int out_tiles, int K, int cb, int tn_base, int group_tiles,
                      int n_groups, const int32_t *group_tab, int n_row_blocks, int block_rows,
                      uint16_t *y_out, size_t ldy, void *stream);

/* Scratch bytes exl3_gemm can use for this shape (0 when no tile would be split). */
size_t exl3_gemm_workspace_bytes(int rows, int in_tiles, int tn_count);

/*
 * Whole layer forward (ponyexl3/ref/forward.py:14-49, EXL3Linear.__call__ at
 * ponyexl3/mlx/exl3_linear.py:98-165, FusedEXL3Group.forward_all at
 * ponyexl3/mlx/exl3_fused.py:136-202):
 *   xh = fp16(had(x * suh_s)); y = fp16(xh @ W); y = fp16(had(y) * svh) (+ bias)
 *   x        fp16 [rows][in]
 *   suh      fp16 [n_sub][in] or NULL (n_sub = 1 for a plain layer)
 *   svh      fp16 [out] or NULL
 *   group_sub int32 [out/128] or NULL (required when n_sub > 1)
 *   y        fp16 [rows][out]
 *   workspace at least exl3_linear_workspace_bytes(rows, in, out, n_sub)
 *   counters int32 [counters_len], 8-byte aligned, or NULL. With counters and
 *            rows <= exl3_gemv_max_rows() the whole layer is ONE kernel launch;
 *            counters_len >= 2*rows*out. The workgroups that share a 128-column
 *            group combine their partial rows in one of two ways, chosen by the
 *            size of the launch: 64-bit fixed-point accumulators in this array,
 *            one per (row, output column), updated with returning atomics (the
 *            total does not depend on the arrival order; the workgroup whose add
 *            completes the group applies the output transform), or fp32 partial
 *            rows in the workspace plus one counter per group in this array (the
 *            workgroup that brings the counter to its final value adds the partial
 *            rows in index order). Either way the array must be all zero on entry
 *            and is all zero again when the launch has finished, so a caller
 *            zeroes it once and reuses it (calls that overlap on one array race),
 *            and results are run-to-run deterministic. Above that and up to
 *            exl3_linear_small_max_rows() rows the array serves the medium-batch
 *            kernel as group counters (counters_len >= out/128; two launches: input
 *            rotation, then everything else). NULL selects the three-launch chain
 *            (exl3_had128_pre, exl3_gemv_partials, exl3_had128_post) resp. the
 *            prefill GEMM.
 *            Status word: when counters_len is at least two ints more than the call
 *            needs, the LAST int of the array is a sticky status word (see
 *            exl3_counters_status below).
 */
int exl3_linear_forward(const uint16_t *x, int rows, const uint16_t *trellis, int in_tiles,
                        int out_tiles, int K, int cb, const uint16_t *suh, int n_sub,
                        const int32_t *group_sub, const uint16_t *svh, const uint16_t *bias,
                        uint16_t *y, void *workspace, size_t workspace_bytes, int32_t *counters,
                        size_t counters_len, void *stream);

size_t exl3_linear_workspace_bytes(int rows, int in_features, int out_features, int n_sub);

/*
 * The launch plan the one-launch layer kernel takes for a shape (rows <=
 * exl3_gemv_max_rows()), for logs and benchmarks: wave-level splits of the tile rows,
 * tile rows per split (4 = half a Hadamard block per wave, 8 = one block, 16 = two),
 * waves per workgroup (4 or 8) and whether the split reduction goes through the 64-bit
 * accumulators (1) or through partial rows (0). The counterpart of the reference's
 * split chooser (ponyexl3/mlx/gemv_metal.py:1405-1414). Any output pointer may be NULL.
 */
int exl3_linear_plan(int rows, int in_tiles, int out_tiles, int K, int *n_splits,
                     int *tile_rows_per_split, int *waves_per_workgroup, int *atomic);

/*
 * Error channel of the accumulator reductions (exl3_linear_forward, exl3_moe_forward,
 * exl3_linear_forward_static); no counterpart in the reference, whose kernels have no
 * split state that outlives a launch. The workgroup that finishes a 128-column group
 * may have to wait for atomic adds of other workgroups that are already in flight; that
 * wait is bounded (EXL3_SPIN_LIMIT polls, default 2^22). It can only run out when the
 * contract of the counters array was broken (not all zero on entry, or shared by calls
 * that overlap). Then no total can be trusted: the workgroup writes NaN to the outputs
 * of its group (for the MoE chain: to that block of the down projection's input, hence
 * to the slot's output), sets the status word - the last int of the counters array as
 * passed to the call, provided the array is at least two ints longer than the call
 * needs - to a non-zero value and leaves the accumulators as they are. The caller
 * must zero the whole array before using it again.
 * exl3_counters_status waits for `stream`, reads that word (counters_len as passed to
 * the forward call; counters == NULL: the array of exl3_linear_forward_static on the
 * current device) and returns EXL3_OK or EXL3_E_INCOMPLETE.
 */
int exl3_counters_status(const int32_t *counters, size_t counters_len, void *stream);

/*
 * exl3_linear_forward for callers that cannot allocate device memory or carry a
 * workspace: code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc. It has no counterpart in the reference. Same arguments and
 * results as exl3_linear_forward with counters (the one-launch kernel), minus
 * workspace and counters: the kernel's split-K state (fp32 partial rows and group
 * counters, or 64-bit accumulators, whichever reduction the launch uses) lives in a
 * device array inside the library: exl3_linear_static_scratch_bytes() = 16 MiB for
 * the partial rows plus as much for the counters / accumulators; every GPU the
 * library runs on holds its copy until the process ends. No hipMalloc, hipFree or
 * other allocating call is made.
 *   rows <= exl3_gemv_max_rows(), otherwise EXL3_E_UNSUPPORTED;
 *   exl3_linear_static_need_bytes(rows, in, out) (the largest of what the launch
 *   plans of the different K keep in either half) must not exceed the scratch size;
 *   a launch whose own plan needs more returns EXL3_E_STATIC_LIMIT (nothing is
 *   launched).
 * All calls on one GPU share that GPU's array: calls that overlap there (two
 * streams, two threads) race. The counter half is all zero whenever no call is
 * running. The first call on a device clears the counter half on `stream` and waits
 * for that to complete before it launches anything else; it must not be made while
 * `stream` is being captured into a graph (EXL3_E_UNSUPPORTED, nothing is launched):
 * call once eagerly before capturing.
 */
size_t exl3_linear_static_scratch_bytes(void);
size_t exl3_linear_static_need_bytes(int rows, int in_features, int out_features);
int exl3_linear_forward_static(const uint16_t *x, int rows, const uint16_t *trellis, int in_tiles,
                               int out_tiles, int K, int cb, const uint16_t *suh, int n_sub,
                               const int32_t *group_sub, const uint16_t *svh, const uint16_t *bias,
                               uint16_t *y, void *stream);

/*
 * Routed MoE expert chain for a handful of tokens, tokens*top_k <= 4096 slots
 * (EXL3SwitchGLU.__call__ at rows <= 8 in the reference,
 * ponyexl3/mlx/exl3_moe.py:770-787; unfused definition :648-682):
 * per slot (token t, expert e = indices[t][s]):
 *   g = L_gate,e(x_t); u = L_up,e(x_t); h = fp16(act(g) * u); y = L_down,e(h)
 *   gu_trellis  uint16 [D/16][E*2*H/16][16K], tile columns laid out
 *               [all experts' gate | all experts' up] (ponyexl3/mlx/model.py:96-122)
 *   gu_suh      fp16 [E][2][D];   gu_svh fp16 [E][2*H]
 *   dn_trellis  uint16 [H/16][E*D/16][16K]
 *   dn_suh      fp16 [E][H];      dn_svh fp16 [E][D]
 *   x           fp16 [tokens][D]; indices int32 [tokens][top_k]
 *   activation  0 = silu (SwiGLU), 1 = tanh-gelu (GeGLU) (ponyexl3/mlx/exl3_moe.py:62-75)
 *   y           fp16 [tokens][top_k][D]
 *   workspace   at least exl3_moe_workspace_bytes(tokens, top_k, D, H)
 *   counters    NULL, or int32[counters_len], 8-byte aligned, with counters_len >=
 *               tokens*top_k*(H/128 + D/128), zero on entry and zero again on
 *               exit. With counters the chain is two launches, the reference's
 *               A2/B2 pair (ponyexl3/mlx/exl3_moe.py:345-422: gate/up, then
 *               GLU + rotation + down); without, five launches that need no
 *               state between calls. Calls that overlap on one counters array race.
 *               With counters_len >= tokens*top_k*(4*H + D/128) the gate/up launch
 *               may reduce through 64-bit fixed-point accumulators held there (one
 *               memory round trip instead of three; chosen when every slot runs on
 *               its own and the launch issues at most EXL3_MOE_MAX_ATOMICS = 300000
 *               atomics); the result can differ from the partial-row reduction by
 *               an fp16 ulp, and is bit-identical from call to call either way.
 *               Two more ints than that make the last int the status word of
 *               exl3_counters_status.
 * Only the selected experts' trellis blocks are read. In the two-launch chain, with
 * 2 <= tokens, at most 512 slots and at least one slot per two experts, the slots that
 * route to one expert share a pass over its weights (four batch rows per pass; same
 * arithmetic per row, bit-identical results); EXL3_MOE_GROUP=0 switches that off.
 */
int exl3_moe_forward(const uint16_t *x, int tokens, const int32_t *indices, int top_k,
                     const uint16_t *gu_trellis, const uint16_t *gu_suh, const uint16_t *gu_svh,
                     const uint16_t *dn_trellis, const uint16_t *dn_suh, const uint16_t *dn_svh,
                     int num_experts, int D, int H, int K, int cb, int activation, uint16_t *y,
                     void *workspace, size_t workspace_bytes, int32_t *counters,
                     size_t counters_len, void *stream);

size_t exl3_moe_workspace_bytes(int tokens, int top_k, int D, int H);

/*
 * Prefill of one layer on activations that exl3_had128_pre already rotated:
 * the MFMA trellis GEMM and the output transform (Hadamard-128, svh, bias), for a
 * plain layer (n_sub = 1) or a sibling-fused one whose members all have
 * out_features % 256 == 0. What FusedEXL3Group.forward_all does above the
 * small-batch row counts (ponyexl3/mlx/exl3_fused.py:136-202) in one GEMM launch.
 *   xh        fp16 [rows][n_sub][16*in_tiles]
 *   block_sub i32 [out_tiles/16 rounded up] member index of every 256-column block
 *             (required when n_sub > 1)
 *   y         fp16 [rows][16*out_tiles]
 *   workspace exl3_linear_prefill_workspace_bytes(rows, in, out) bytes
 */
size_t exl3_linear_prefill_workspace_bytes(int rows, int in_features, int out_features);
int exl3_linear_prefill(const uint16_t *xh, int rows, int n_sub, const uint16_t *trellis,
                        int in_tiles, int out_tiles, int K, int cb, const int32_t *block_sub,
                        const uint16_t *svh, const uint16_t *bias, uint16_t *y, void *workspace,
                        size_t workspace_bytes, void *stream);

/*
 * MoE prefill glue, one launch each.
 * exl3_moe_sort: stable counting sort of the (token, slot) pairs by expert plus the
 * row-block table exl3_gemm_grouped takes. Replaces the argsort / segment-table
 * host code of EXL3SwitchGLU._prefill (ponyexl3/mlx/exl3_moe.py:79-98, 700-716).
 *   indices i32 [n_pairs] expert per pair (pair = token*top_k + slot; clamped)
 *   order, tok, sidx  i32 [n_pairs], by sorted position: pair index, token, expert
 *   table   i32 [table_len][4] = {expert, first row, end row, 0}, 16-byte aligned,
 *           table_len >= n_pairs / block_rows + n_experts; unused entries are empty
 * n_experts <= 1024 (EXL3_E_UNSUPPORTED above that).
 * exl3_moe_glu_rows: per sorted row r with expert e = sidx[r]:
 *   xh_dn[r] = fp16(had(fp16(act(G) * U) * dn_suh[e])), G = fp16(had(g[r]) * gu_svh[e][:H]),
 *   U likewise from u and gu_svh[e][H:]; activation 0 = SiLU, 1 = tanh-GELU. Replaces
 *   _rows_finish x2, the GLU and _rows_prep (ponyexl3/mlx/exl3_moe.py:105-136, 62-75).
 *   g, u, xh_dn fp16 [n_rows][H]; gu_svh fp16 [E][2*H]; dn_suh fp16 [E][H]
 */
int exl3_moe_sort(const int32_t *indices, int n_pairs, int top_k, int n_experts, int block_rows,
                  int32_t *order, int32_t *tok, int32_t *sidx, int32_t *table, int table_len,
                  void *stream);
int exl3_moe_glu_rows(const uint16_t *g, const uint16_t *u, int n_rows, int H, const int32_t *sidx,
                      const uint16_t *gu_svh, const uint16_t *dn_suh, int n_experts,
                      int activation, uint16_t *xh_dn, void *stream);

/*
 * Packed tiles -> their 256 sliding-window codewords per tile, kernel order.
 * Replaces unpack_trellis (ponyexl3/ref/trellis.py:153-214); the inverse of
 * exl3_pack_trellis on the low K bits. K in 1..8.
 *   trellis u16 [n_tiles][16*K]   codewords u16 [n_tiles][256] (16-byte aligned)
 */
int exl3_unpack_trellis(const uint16_t *trellis, long long n_tiles, int K, uint16_t *codewords,
                        void *stream);

/*
 * Encoder side: tail-biting Viterbi search over the bitshift trellis, one 16x16
 * tile (256 fp32 targets in kernel order) per workgroup. Replaces
 * quantize_tiles_mlx (ponyexl3/convert/metal_search.py:63-196, 254-303) and
 * follows its arithmetic (fp16 path costs, fp32 fma, warm-up pass + pinned pass),
 * so the same path is chosen; the exact float64 search
 * (ponyexl3/convert/reference_search.py:59-87) is the quality yardstick.
 * K must be in 2..8 (the reference rejects K = 1 too): EXL3_E_BAD_K otherwise.
 *   tiles     fp32 [n_tiles][256]
 *   q_tiles   fp32 [n_tiles][256]   decoded value of the chosen codeword
 *   indices   u16  [n_tiles][256]   full 16-bit codewords; indices & (2^K - 1) are
 *                                   the symbols exl3_pack_trellis takes
 *   workspace backpointer slots, exl3_quantize_slot_bytes(K) each. At least one
 *             slot is required (EXL3_E_WORKSPACE); exl3_quantize_workspace_bytes()
 *             is what keeps every CU busy; more than that is not used. A tile
 *             batch larger than the slot count is walked by the same launch.
 */
size_t exl3_quantize_slot_bytes(int K);
size_t exl3_quantize_workspace_bytes(int n_tiles, int K);
int exl3_quantize_tiles(const float *tiles, int n_tiles, int K, int cb, float *q_tiles,
                        uint16_t *indices, void *workspace, size_t workspace_bytes, void *stream);

/*
 * K-bit symbols (low K bits of each u16) -> packed tiles, bit-exact with
 * pack_trellis (ponyexl3/ref/trellis.py:13-49, 144-150) and pack_trellis_mlx
 * (ponyexl3/convert/mlx_trellis.py:66-84). K in 1..8.
 *   encoded u16 [n_tiles][256]   packed u16 [n_tiles][16*K] (4-byte aligned)
 */
int exl3_pack_trellis(const uint16_t *encoded, long long n_tiles, int K, uint16_t *packed,
                      void *stream);

#ifdef __cplusplus
}
#endif

#endif /* EXL3_HIP_H */
