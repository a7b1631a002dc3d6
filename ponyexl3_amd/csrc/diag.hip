// Diagnostic kernels behind bench.py's measured ceilings: what this GPU delivers
// for (a) a plain streaming read and (b) the per-lane trellis decode + matrix-pipe
// dot product loop of the small-batch kernels with nothing else around it (no
// Hadamard, no split reduction, no launch-bound phases). They compute nothing a
// caller needs; they exist so that roofline fractions can be quoted against
// measured as well as published peaks.
#include "../../include/exl3_diag.h"
#include "exl3_device.hpp"
#include "exl3_host.hpp"
#include "exl3_small.hpp"

namespace exl3 {

// Every workgroup streams its contiguous share of the buffer with 16-byte
// non-temporal loads, four in flight per lane.
__global__ __launch_bounds__(256) void diag_stream_read_kernel(const uint4_t* __restrict__ p,
                                                               size_t n_vec, uint32_t* out) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * 256;
    uint4_t acc = {0, 0, 0, 0};
    for (; i + 3 * stride < n_vec; i += 4 * stride) {
        const uint4_t a = __builtin_nontemporal_load(p + i);
        const uint4_t b = __builtin_nontemporal_load(p + i + stride);
        const uint4_t c = __builtin_nontemporal_load(p + i + 2 * stride);
        const uint4_t d = __builtin_nontemporal_load(p + i + 3 * stride);
        acc ^= a ^ b ^ c ^ d;
    }
    for (; i < n_vec; i += stride) acc ^= __builtin_nontemporal_load(p + i);
    const uint32_t r = acc.x ^ acc.y ^ acc.z ^ acc.w;
    if (r == 0x9E3779B9u) out[0] = r;  // keeps the loads alive; practically never taken
}

// One workgroup of 16 waves per CU; every wave runs `steps` tile rows of the
// decode + dot loop over its own contiguous slice of the buffer (wave-wide loads
// of 256*K bytes, kSlots in flight), exactly the inner loop of the layer kernels.
template <int K, int CB>
__global__ __launch_bounds__(1024) void diag_decode_kernel(const uint32_t* __restrict__ buf,
                                                           uint32_t rows_mask, int steps,
                                                           float* __restrict__ out) {
    // 64 tile rows of activations, each value stored twice as the layer kernels stage them
    __shared__ __attribute__((aligned(16))) half_t xs[2048];
    constexpr int kSlots = 4;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const half_t xval = (half_t)(float)((int)(threadIdx.x * 37 % 17) - 8);  // small integers, -8..8
    xs[2 * threadIdx.x] = xs[2 * threadIdx.x + 1] = xval;
    __syncthreads();
    const uint32_t wave_global = blockIdx.x * 16 + wave;
    float4_t accv[2][1] = {{float4_t{0, 0, 0, 0}}, {float4_t{0, 0, 0, 0}}};
    uint32_t w[kSlots][K];
    auto row_ptr = [&](int s) {
        const uint32_t r = (wave_global * (uint32_t)steps + (uint32_t)s) & rows_mask;
        return buf + (size_t)r * (64 * K) + lane * K;
    };
#pragma unroll
    for (int s = 0; s < kSlots; s++) load_lane_words_nt<K>(row_ptr(s), w[s]);
    uint32_t prev = neighbour_word(w[0][K - 1], lane);
    for (int s0 = 0; s0 < steps; s0 += kSlots) {
#pragma unroll
        for (int s = 0; s < kSlots; s++) {
            const uint32_t prev_next = neighbour_word(w[(s + 1) % kSlots][K - 1], lane);
            const uint4_t* xp = reinterpret_cast<const uint4_t*>(xs + ((s0 + s) & 63) * 32);
            __builtin_amdgcn_sched_barrier(0);
            dot_tile_row<K, CB, 1>(make_lane_words<K>(prev, w[s]), [&](int c) {
                XChunk<1> t;
                t.v[0] = xp[c];
                return t;
            }, accv);
            load_lane_words_nt<K>(row_ptr(s0 + s + kSlots), w[s]);
            __builtin_amdgcn_sched_barrier(0);
            prev = prev_next;
        }
    }
    const float total = accv[0][0][0] + accv[1][0][0];
    out[(size_t)wave_global * 64 + lane] = total;
}

// The fixed phases of a small-batch launch, measured on a grid of the caller's choice:
// (a) nothing but the dispatch of the grid; (b) every wave requests its first
// kStreamSlots tile rows (wave-wide loads of 256*K bytes from its own slice of the
// buffer, as the layer kernels do before they can decode anything), waits for them and
// leaves.
__global__ void diag_empty_kernel() {}

template <int K>
__global__ void diag_first_rows_kernel(const uint32_t* __restrict__ buf, uint32_t rows_mask,
                                       uint32_t row_base, uint32_t* out) {
    const int lane = threadIdx.x & 63;
    const uint32_t waves_per_wg = blockDim.x >> 6;
    const uint32_t wave_global =
        (blockIdx.y * gridDim.x + blockIdx.x) * waves_per_wg + (threadIdx.x >> 6);
    uint32_t w[kStreamSlots][K];
#pragma unroll
    for (int s = 0; s < kStreamSlots; s++) {
        const uint32_t r = (row_base + wave_global * kStreamSlots + s) & rows_mask;
        load_lane_words_nt<K>(buf + (size_t)r * (64 * K) + lane * K, w[s]);
    }
    uint32_t acc = 0;
#pragma unroll
    for (int s = 0; s < kStreamSlots; s++)
#pragma unroll
        for (int i = 0; i < K; i++) acc ^= w[s][i];
    if (acc == 0x9E3779B9u) out[0] = acc;  // keeps the loads alive; practically never taken
}

}  // namespace exl3

static bool diag_grid_ok(int grid_x, int grid_y, int threads) {
    return grid_x >= 1 && grid_y >= 1 && grid_y <= 65535 && (long long)grid_x * grid_y <= (1 << 22) &&
           threads >= 64 && threads <= 1024 && threads % 64 == 0;
}

EXL3_EXPORT int exl3_diag_empty_launch(int grid_x, int grid_y, int threads, void* stream) {
    using namespace exl3;
    if (!diag_grid_ok(grid_x, grid_y, threads)) return EXL3_E_BAD_SHAPE;
    diag_empty_kernel<<<dim3((unsigned)grid_x, (unsigned)grid_y), dim3((unsigned)threads), 0,
                        as_stream(stream)>>>();
    return launch_status();
}

EXL3_EXPORT int exl3_diag_first_rows(const void* buf, size_t bytes, int K, int grid_x, int grid_y,
                                     int threads, unsigned row_base, void* out, void* stream) {
    using namespace exl3;
    if (int rc = check_k_cb(K, 0)) return rc;
    if (!buf || !out) return EXL3_E_NULL_POINTER;
    const size_t rows = bytes / ((size_t)256 * K);
    size_t pow2 = 1;
    while (pow2 * 2 <= rows) pow2 *= 2;  // the row index wraps on a power of two
    if (rows < 1 || pow2 > 0x80000000ull || !diag_grid_ok(grid_x, grid_y, threads) ||
        (reinterpret_cast<uintptr_t>(buf) & 15))
        return EXL3_E_BAD_SHAPE;
    return dispatch_k_cb(K, 0, [&](auto k, auto) {
        diag_first_rows_kernel<k.value>
            <<<dim3((unsigned)grid_x, (unsigned)grid_y), dim3((unsigned)threads), 0,
               as_stream(stream)>>>(reinterpret_cast<const uint32_t*>(buf), (uint32_t)(pow2 - 1),
                                    row_base, reinterpret_cast<uint32_t*>(out));
        return launch_status();
    });
}

EXL3_EXPORT int exl3_diag_stream_read(const void* buf, size_t bytes, void* out, void* stream) {
    using namespace exl3;
    if (!buf || !out) return EXL3_E_NULL_POINTER;
    if (bytes < 16 || (reinterpret_cast<uintptr_t>(buf) & 15)) return EXL3_E_BAD_SHAPE;
    diag_stream_read_kernel<<<dim3(8192), dim3(256), 0, as_stream(stream)>>>(
        reinterpret_cast<const uint4_t*>(buf), bytes / 16, reinterpret_cast<uint32_t*>(out));
    return launch_status();
}

EXL3_EXPORT int exl3_diag_decode_loop(const void* buf, size_t bytes, int K, int cb, int n_wg,
                                      int steps, float* out, void* stream) {
    using namespace exl3;
    if (int rc = check_k_cb(K, cb)) return rc;
    if (!buf || !out) return EXL3_E_NULL_POINTER;
    if (cb == CB_MUL1) return EXL3_E_UNSUPPORTED;
    const size_t row_bytes = (size_t)256 * K;
    size_t rows = bytes / row_bytes, pow2 = 1;
    while (pow2 * 2 <= rows) pow2 *= 2;  // the slice index wraps on a power of two
    if (rows < 1 || n_wg < 1 || n_wg > 4096 || steps < 4 || steps % 4 || pow2 > 0x80000000ull ||
        (reinterpret_cast<uintptr_t>(buf) & 15))
        return EXL3_E_BAD_SHAPE;
    return dispatch_k_cb(K, cb, [&](auto k, auto c) {
        if constexpr (c.value == CB_MUL1) {
            return (int)EXL3_E_UNSUPPORTED;
        } else {
            diag_decode_kernel<k.value, c.value><<<dim3((unsigned)n_wg), dim3(1024), 0, as_stream(stream)>>>(
                reinterpret_cast<const uint32_t*>(buf), (uint32_t)(pow2 - 1), steps, out);
            return launch_status();
        }
    });
}
