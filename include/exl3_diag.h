/*
 * C ABI of libexl3_diag.so: measurement probes for the MI355X (gfx950) EXL3 kernels.
 * Not part of the product library (libexl3_hip.so, include/exl3_hip.h): these entry
 * points compute nothing a caller needs; bench.py uses them to report the ceilings its
 * roofline figures are read against. Same conventions: raw device pointers, a HIP
 * stream passed as void*, int status (0 = ok, negative EXL3_E_* codes of exl3_hip.h).
 */
#ifndef EXL3_DIAG_H
#define EXL3_DIAG_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/*
 * Diagnostics for measured ceilings (no counterpart in the reference; its kernel
 * benches quote Gw/s only, tools/bench/gemv_split_bench.py:51,84).
 * exl3_diag_stream_read: reads `bytes` (16-byte aligned buffer) once with streaming
 *   loads; out: 4 bytes of device memory, practically never written.
 * exl3_diag_decode_loop: n_wg workgroups of 16 waves run `steps` (a multiple of 4)
 *   iterations of the small-batch kernels' inner loop (one wave-wide load of 256*K
 *   bytes, per-lane decode of 32 codewords, 16 matrix-pipe dot products) over
 *   consecutive 256*K-byte rows of buf, wrapping at the largest power-of-two row
 *   count that fits in `bytes`; weights per launch = n_wg*16*steps*2048. cb 0 or 1.
 *   out: float [n_wg*1024].
 * exl3_diag_empty_launch: a kernel that does nothing on a grid of grid_x * grid_y
 *   workgroups of `threads` lanes (a multiple of 64, at most 1024): what the dispatch of
 *   such a grid costs.
 * exl3_diag_first_rows: on the same kind of grid every wave requests its first four
 *   tile rows (wave-wide loads of 256*K bytes, rows row_base + 4*wave .. +3 of buf,
 *   wrapping like above), waits for them and leaves: the time before a small-batch
 *   launch can decode anything. out: 4 bytes of device memory, practically never written.
 */
int exl3_diag_stream_read(const void *buf, size_t bytes, void *out, void *stream);
int exl3_diag_decode_loop(const void *buf, size_t bytes, int K, int cb, int n_wg, int steps,
                          float *out, void *stream);
int exl3_diag_empty_launch(int grid_x, int grid_y, int threads, void *stream);
int exl3_diag_first_rows(const void *buf, size_t bytes, int K, int grid_x, int grid_y,
                         int threads, unsigned row_base, void *out, void *stream);

#ifdef __cplusplus
}
#endif

#endif /* EXL3_DIAG_H */
