// Hadamard-128 regularisation kernels (input side with suh, output side with
// split-K reduction + svh + bias).
//
// Narrow form (few rows, fp32 partial sums): one wavefront owns one 128-wide
// block, lane l holds elements 2l and 2l+1 in fp32. The Sylvester transform
// factors into 7 butterfly stages that commute; the stage on element bit 0 is
// in-lane, the other six exchange with lane l ^ (1 << b).
// Wide form (prefill, fp16 in and out): lane l of a 16-lane group holds the 8
// consecutive elements 8l..8l+7 of a block (one 16-byte load), the stages on
// element bits 0..2 are in-lane and the other four exchange inside the group, so
// a wavefront transforms four blocks per 1 KiB load and a workgroup walks along
// one row. Same stage order and the same a+b / a-b per stage as the narrow form,
// hence the same bits. No LDS, no barriers. Arithmetic follows
// ponyexl3/ref/hadamard.py:50-80: multiply by the pre vector in fp32,
// transform, scale by 1/sqrt(128), multiply by the post vector in fp32, and the
// caller-visible casts of ponyexl3/ref/forward.py:34,41,42,45.
#include "exl3_device.hpp"
#include "exl3_host.hpp"

#pragma clang fp contract(off)

namespace exl3 {

constexpr float kHadScale = 0.088388347648318440550f;  // 1/sqrt(128)

__device__ __forceinline__ void wht128(float& a, float& b, int lane) { wht128_lanes(a, b, lane); }

// Optional row gathers / scatter of the wide kernels: kernel row r reads input row
// in_index[r], scale vector scale_index[r] (scale_ld elements apart) and writes
// output row out_index[r]; a NULL table is the identity. The tables come from the
// caller's memory: a row whose input, scale or output index falls outside
// [0, n_in) / [0, n_scale) / [0, n_out) is skipped (nothing is read or written for it).
struct RowMap {
    int per_row;
    const int32_t* in_index;
    const int32_t* scale_index;
    const int32_t* out_index;
    size_t scale_ld;
    unsigned n_in, n_scale, n_out;  // rows behind x, scale and out (per_row mode only)
    __device__ size_t in_row(size_t r) const { return in_index ? (size_t)in_index[r] : r; }
    __device__ size_t scale_row(size_t r) const { return scale_index ? (size_t)scale_index[r] : r; }
    __device__ size_t out_row(size_t r) const { return out_index ? (size_t)out_index[r] : r; }
    __device__ bool row_ok(size_t r, bool uses_scale) const {
        if (!per_row) return true;
        // negative entries wrap to huge unsigned values and fail the same test
        return in_row(r) < (size_t)n_in && out_row(r) < (size_t)n_out &&
               (!uses_scale || scale_row(r) < (size_t)n_scale);
    }
};

// v[j] = element 8*(lane & 15) + j of the lane group's block, unnormalised WHT in place.
__device__ __forceinline__ void wht128_wide(float (&v)[8], int lane) {
#pragma unroll
    for (int h = 1; h < 8; h <<= 1) {
#pragma unroll
        for (int j = 0; j < 8; j++) {
            if ((j & h) == 0) {
                const float lo = v[j], hi = v[j + h];
                v[j] = lo + hi;
                v[j + h] = lo - hi;
            }
        }
    }
    // lanes 1, 2, 4, 8 apart: DPP operands, no LDS
    static_for<0, 4>([&](auto bit) {
        const uint32_t sign = lane_sign_mask(lane, bit.value);
#pragma unroll
        for (int j = 0; j < 8; j++) v[j] = butterfly_dpp<bit.value>(v[j], sign);
    });
}

__device__ __forceinline__ void halfs_to_floats(uint4_t q, float (&v)[8]) {
    const uint32_t w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const half2_t h = bits_to_half2(w[i]);
        v[2 * i] = (float)h.x;
        v[2 * i + 1] = (float)h.y;
    }
}

// Wide forms: grid.x = number of output rows ((row, sub) pairs for the input side);
// the four waves of a workgroup take consecutive 512-element chunks of the row,
// and grid.y workgroups share a row when there are too few rows to fill the chip.
// All pointers 16-byte aligned, n a multiple of 128.
__global__ __launch_bounds__(256) void had_pre_wide_kernel(const half_t* __restrict__ x,
                                                           const half_t* __restrict__ suh,
                                                           half_t* __restrict__ xh, int n,
                                                           int n_sub, RowMap map) {
    const int lane = threadIdx.x & 63;
    // One workgroup per source row: per-row tables (rows sorted by expert) give its
    // source, scale vector and destination; otherwise the row is rotated once per stacked
    // sibling (scale vector s, destination row r * n_sub + s) from a single read.
    const size_t r = blockIdx.x;
    if (!map.row_ok(r, suh != nullptr)) return;
    const half_t* xr = x + (map.per_row ? map.in_row(r) : r) * (size_t)n;
    const int subs = map.per_row ? 1 : n_sub;
    // up to four 16-byte chunks of the row in flight per lane
    const int c0 = (blockIdx.y * 256 + threadIdx.x) * 8, cstep = 2048 * gridDim.y;
    for (int cb = c0; cb < n; cb += 4 * cstep) {
        uint4_t raw[4];
#pragma unroll
        for (int i = 0; i < 4; i++)
            if (cb + i * cstep < n) raw[i] = *reinterpret_cast<const uint4_t*>(xr + cb + i * cstep);
        for (int s = 0; s < subs; s++) {
            const half_t* sr =
                suh ? suh + (map.per_row ? map.scale_row(r) * map.scale_ld : s * (size_t)n) : nullptr;
            half_t* orow = xh + (map.per_row ? map.out_row(r) : r * n_sub + s) * (size_t)n;
            uint4_t sraw[4];
            if (sr) {
#pragma unroll
                for (int i = 0; i < 4; i++)
                    if (cb + i * cstep < n)
                        sraw[i] = *reinterpret_cast<const uint4_t*>(sr + cb + i * cstep);
            }
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int c = cb + i * cstep;
                if (c >= n) break;
                float v[8], sv[8];
                halfs_to_floats(raw[i], v);
                if (sr) {
                    halfs_to_floats(sraw[i], sv);
#pragma unroll
                    for (int j = 0; j < 8; j++) v[j] = v[j] * sv[j];
                }
                wht128_wide(v, lane);
                uint4_t o;
                uint32_t* ow = reinterpret_cast<uint32_t*>(&o);
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    half2_t h;
                    h.x = (half_t)(v[2 * k] * kHadScale);
                    h.y = (half_t)(v[2 * k + 1] * kHadScale);
                    ow[k] = half2_to_bits(h);
                }
                *reinterpret_cast<uint4_t*>(orow + c) = o;
            }
        }
    }
}

__global__ __launch_bounds__(256) void had_post_wide_kernel(const half_t* __restrict__ y,
                                                            const half_t* __restrict__ svh,
                                                            const half_t* __restrict__ bias,
                                                            half_t* out, int n, RowMap map) {
    const int lane = threadIdx.x & 63;
    const size_t rs = blockIdx.x;
    if (!map.row_ok(rs, svh != nullptr)) return;
    if (svh && map.per_row) svh += map.scale_row(rs) * map.scale_ld;
    const half_t* yr = y + map.in_row(rs) * (size_t)n;
    half_t* orow = out + map.out_row(rs) * (size_t)n;
    // up to four 16-byte chunks of the row in flight per lane
    const int c0 = (blockIdx.y * 256 + threadIdx.x) * 8, cstep = 2048 * gridDim.y;
    for (int cb = c0; cb < n; cb += 4 * cstep) {
        uint4_t raw[4];
#pragma unroll
        for (int i = 0; i < 4; i++)
            if (cb + i * cstep < n) raw[i] = *reinterpret_cast<const uint4_t*>(yr + cb + i * cstep);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int c = cb + i * cstep;
            if (c >= n) break;
            float v[8], sv[8];
            halfs_to_floats(raw[i], v);
            wht128_wide(v, lane);
            if (svh) halfs_to_floats(*reinterpret_cast<const uint4_t*>(svh + c), sv);
            uint4_t bq = {0u, 0u, 0u, 0u};
            if (bias) bq = *reinterpret_cast<const uint4_t*>(bias + c);
            const uint32_t* bw = reinterpret_cast<const uint32_t*>(&bq);
            uint4_t o;
            uint32_t* ow = reinterpret_cast<uint32_t*>(&o);
#pragma unroll
            for (int k = 0; k < 4; k++) {
                float a = v[2 * k] * kHadScale, b = v[2 * k + 1] * kHadScale;
                if (svh) {
                    a = a * sv[2 * k];
                    b = b * sv[2 * k + 1];
                }
                half2_t h;
                h.x = (half_t)a;
                h.y = (half_t)b;
                if (bias) {
                    const half2_t bv = bits_to_half2(bw[k]);
                    h.x = h.x + bv.x;
                    h.y = h.y + bv.y;
                }
                ow[k] = half2_to_bits(h);
            }
            *reinterpret_cast<uint4_t*>(orow + c) = o;
        }
    }
}

// xh[r][s][blk] = fp16(wht(x[r][blk] * suh[s][blk]) / sqrt(128))
__global__ __launch_bounds__(256) void had_pre_kernel(const half_t* __restrict__ x,
                                                      const half_t* __restrict__ suh,
                                                      half_t* __restrict__ xh, int rows, int n,
                                                      int n_sub) {
    const int lane = threadIdx.x & 63;
    const int blocks = n >> 7;
    const long long wave_id = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
    const long long total = (long long)rows * n_sub * blocks;
    if (wave_id >= total) return;
    const int blk = (int)(wave_id % blocks);
    const long long rs = wave_id / blocks;
    const int s = (int)(rs % n_sub);
    const long long r = rs / n_sub;
    const half2_t xv = *reinterpret_cast<const half2_t*>(x + r * n + blk * 128 + 2 * lane);
    float a = (float)xv.x, b = (float)xv.y;
    if (suh) {
        const half2_t sv =
            *reinterpret_cast<const half2_t*>(suh + (size_t)s * n + blk * 128 + 2 * lane);
        a = a * (float)sv.x;
        b = b * (float)sv.y;
    }
    wht128(a, b, lane);
    half2_t o;
    o.x = (half_t)(a * kHadScale);
    o.y = (half_t)(b * kHadScale);
    *reinterpret_cast<half2_t*>(xh + rs * n + blk * 128 + 2 * lane) = o;
}

// out[r][blk] = fp16(wht(fp16(sum_i y[i][r][blk])) / sqrt(128) * svh[blk]) (+ bias)
template <bool kFp32In>
__global__ __launch_bounds__(256) void had_post_kernel(const void* __restrict__ yv, int n_sum,
                                                       size_t sum_stride,
                                                       const half_t* __restrict__ svh,
                                                       const half_t* __restrict__ bias,
                                                       half_t* out, int rows, int n) {
    const int lane = threadIdx.x & 63;
    const int blocks = n >> 7;
    const long long wave_id = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (wave_id >= (long long)rows * blocks) return;
    const int blk = (int)(wave_id % blocks);
    const long long r = wave_id / blocks;
    const size_t off = (size_t)r * n + blk * 128 + 2 * lane;
    float a, b;
    if constexpr (kFp32In) {
        const float* y = reinterpret_cast<const float*>(yv);
        // slices are loaded eight at a time and added strictly in index order
        float2_t acc = {0.f, 0.f};
        int i = 0;
        for (; i + 8 <= n_sum; i += 8) {
            float2_t v[8];
#pragma unroll
            for (int j = 0; j < 8; j++)
                v[j] = *reinterpret_cast<const float2_t*>(y + (size_t)(i + j) * sum_stride + off);
#pragma unroll
            for (int j = 0; j < 8; j++) {
                acc.x = acc.x + v[j].x;
                acc.y = acc.y + v[j].y;
            }
        }
        for (; i < n_sum; i++) {
            const float2_t v = *reinterpret_cast<const float2_t*>(y + (size_t)i * sum_stride + off);
            acc.x = acc.x + v.x;
            acc.y = acc.y + v.y;
        }
        a = (float)(half_t)acc.x;  // the matmul result is stored as fp16 before the transform
        b = (float)(half_t)acc.y;
    } else {
        const half2_t v = *reinterpret_cast<const half2_t*>(reinterpret_cast<const half_t*>(yv) + off);
        a = (float)v.x;
        b = (float)v.y;
    }
    wht128(a, b, lane);
    a = a * kHadScale;
    b = b * kHadScale;
    if (svh) {
        const half2_t sv = *reinterpret_cast<const half2_t*>(svh + blk * 128 + 2 * lane);
        a = a * (float)sv.x;
        b = b * (float)sv.y;
    }
    half2_t o;
    o.x = (half_t)a;
    o.y = (half_t)b;
    if (bias) {
        const half2_t bv = *reinterpret_cast<const half2_t*>(bias + blk * 128 + 2 * lane);
        o.x = o.x + bv.x;
        o.y = o.y + bv.y;
    }
    *reinterpret_cast<half2_t*>(out + off) = o;
}

// From this many rows on the wide kernels (one workgroup per row) fill the device
// better than one wave per 128-element block.
constexpr int kWideMinRows = 16;
static inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// Workgroups per row of the wide kernels: about four workgroups per CU in total,
// never more than the row has 2048-element chunks.
static unsigned wide_row_parts(long long rows, int n) {
    const long long chunks = (n + 2047) / 2048;
    long long want = (1024 + rows - 1) / rows;
    if (want > chunks) want = chunks;
    return (unsigned)(want < 1 ? 1 : want);
}

int launch_had_pre(const uint16_t* x, int rows, int n, const uint16_t* suh, int n_sub,
                   uint16_t* xh, hipStream_t stream) {
    if (!x || !xh) return EXL3_E_NULL_POINTER;
    if (rows < 0 || n <= 0 || n % 128 || n_sub < 1) return EXL3_E_BAD_SHAPE;
    if (!suh && n_sub != 1) return EXL3_E_BAD_SHAPE;
    if (rows == 0) return EXL3_OK;
    const long long waves = (long long)rows * n_sub * (n / 128);
    const long long grid = (waves + 3) / 4;
    if (grid > 0x7FFFFFFFLL) return EXL3_E_BAD_SHAPE;
    if ((long long)rows * n_sub >= kWideMinRows && aligned16(x) && aligned16(xh) &&
        (!suh || aligned16(suh))) {
        had_pre_wide_kernel<<<dim3((unsigned)rows, wide_row_parts((long long)rows, n)),
                              dim3(256), 0, stream>>>(
            reinterpret_cast<const half_t*>(x), reinterpret_cast<const half_t*>(suh),
            reinterpret_cast<half_t*>(xh), n, n_sub, RowMap{});
        return launch_status();
    }
    had_pre_kernel<<<dim3((unsigned)grid), dim3(256), 0, stream>>>(
        reinterpret_cast<const half_t*>(x), reinterpret_cast<const half_t*>(suh),
        reinterpret_cast<half_t*>(xh), rows, n, n_sub);
    return launch_status();
}

int launch_had_post(const void* y, int y_is_fp32, int n_sum, size_t sum_stride, int rows, int n,
                    const uint16_t* svh, const uint16_t* bias, uint16_t* out, hipStream_t stream) {
    if (!y || !out) return EXL3_E_NULL_POINTER;
    if (rows < 0 || n <= 0 || n % 128 || n_sum < 1) return EXL3_E_BAD_SHAPE;
    if (!y_is_fp32 && n_sum != 1) return EXL3_E_BAD_SHAPE;
    if (rows == 0) return EXL3_OK;
    const long long waves = (long long)rows * (n / 128);
    const long long grid = (waves + 3) / 4;
    if (grid > 0x7FFFFFFFLL) return EXL3_E_BAD_SHAPE;
    const half_t* s = reinterpret_cast<const half_t*>(svh);
    const half_t* b = reinterpret_cast<const half_t*>(bias);
    half_t* o = reinterpret_cast<half_t*>(out);
    if (!y_is_fp32 && rows >= kWideMinRows && aligned16(y) && aligned16(out) &&
        (!svh || aligned16(svh)) && (!bias || aligned16(bias))) {
        had_post_wide_kernel<<<dim3((unsigned)rows, wide_row_parts(rows, n)), dim3(256), 0, stream>>>(
            reinterpret_cast<const half_t*>(y), s, b, o, n, RowMap{});
        return launch_status();
    }
    if (y_is_fp32)
        had_post_kernel<true><<<dim3((unsigned)grid), dim3(256), 0, stream>>>(y, n_sum, sum_stride,
                                                                              s, b, o, rows, n);
    else
        had_post_kernel<false><<<dim3((unsigned)grid), dim3(256), 0, stream>>>(y, 1, 0, s, b, o,
                                                                               rows, n);
    return launch_status();
}

// Per-row scale vectors (rows that belong to different experts): wide kernels only.
int launch_had_rows(const uint16_t* x, int n_in_rows, int rows, int n, const int32_t* in_index,
                    const uint16_t* scale, int n_scale_rows, const int32_t* scale_index,
                    size_t scale_ld, int post, uint16_t* out, int n_out_rows,
                    const int32_t* out_index, hipStream_t stream) {
    if (!x || !out || !scale) return EXL3_E_NULL_POINTER;
    if (rows < 0 || n <= 0 || n % 128 || scale_ld % 8 || n_in_rows < 0 || n_scale_rows < 0 ||
        n_out_rows < 0)
        return EXL3_E_BAD_SHAPE;
    // identity maps must stay inside their buffers as well
    if ((!in_index && rows > n_in_rows) || (!scale_index && rows > n_scale_rows) ||
        (!out_index && rows > n_out_rows))
        return EXL3_E_BAD_SHAPE;
    if (!aligned16(x) || !aligned16(out) || !aligned16(scale)) return EXL3_E_BAD_SHAPE;
    if (rows == 0) return EXL3_OK;
    const RowMap map{1, in_index, scale_index, out_index, scale_ld, (unsigned)n_in_rows,
                     (unsigned)n_scale_rows, (unsigned)n_out_rows};
    if (post)
        had_post_wide_kernel<<<dim3((unsigned)rows, wide_row_parts(rows, n)), dim3(256), 0, stream>>>(
            reinterpret_cast<const half_t*>(x), reinterpret_cast<const half_t*>(scale), nullptr,
            reinterpret_cast<half_t*>(out), n, map);
    else
        had_pre_wide_kernel<<<dim3((unsigned)rows, wide_row_parts(rows, n)), dim3(256), 0, stream>>>(
            reinterpret_cast<const half_t*>(x), reinterpret_cast<const half_t*>(scale),
            reinterpret_cast<half_t*>(out), n, 1, map);
    return launch_status();
}

}  // namespace exl3

EXL3_EXPORT int exl3_had128_rows(const uint16_t* x, int n_in_rows, int rows, int n,
                                 const int32_t* in_index, const uint16_t* scale, int n_scale_rows,
                                 const int32_t* scale_index, size_t scale_ld, int post,
                                 uint16_t* out, int n_out_rows, const int32_t* out_index,
                                 void* stream) {
    return exl3::launch_had_rows(x, n_in_rows, rows, n, in_index, scale, n_scale_rows, scale_index,
                                 scale_ld, post, out, n_out_rows, out_index,
                                 exl3::as_stream(stream));
}

EXL3_EXPORT int exl3_had128_pre(const uint16_t* x, int rows, int n, const uint16_t* suh, int n_sub,
                                uint16_t* xh, void* stream) {
    return exl3::launch_had_pre(x, rows, n, suh, n_sub, xh, exl3::as_stream(stream));
}

EXL3_EXPORT int exl3_had128_post(const void* y, int y_is_fp32, int n_sum, size_t sum_stride,
                                 int rows, int n, const uint16_t* svh, const uint16_t* bias,
                                 uint16_t* out, void* stream) {
    return exl3::launch_had_post(y, y_is_fp32, n_sum, sum_stride, rows, n, svh, bias, out,
                                 exl3::as_stream(stream));
}
