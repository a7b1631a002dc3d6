// Hadamard-128 regularisation kernels (input side with suh, output side with
// split-K reduction + svh + bias).
//
// One wavefront owns one 128-wide block: lane l holds elements 2l and 2l+1 in
// fp32. The Sylvester transform factors into 7 butterfly stages that commute;
// the stage on element bit 0 is in-lane, the other six exchange with lane
// l ^ (1 << b). No LDS, no barriers. Arithmetic follows
// ponyexl3/ref/hadamard.py:50-80: multiply by the pre vector in fp32,
// transform, scale by 1/sqrt(128), multiply by the post vector in fp32, and the
// caller-visible casts of ponyexl3/ref/forward.py:34,41,42,45.
#include "exl3_device.hpp"
#include "exl3_host.hpp"

#pragma clang fp contract(off)

namespace exl3 {

constexpr float kHadScale = 0.088388347648318440550f;  // 1/sqrt(128)

__device__ __forceinline__ void wht128(float& a, float& b, int lane) {
    const float s = a + b, d = a - b;
    a = s;
    b = d;
#pragma unroll
    for (int bit = 0; bit < 6; bit++) {
        const int mask = 1 << bit;
        const float pa = __shfl_xor(a, mask, kWave);
        const float pb = __shfl_xor(b, mask, kWave);
        const bool upper = (lane & mask) != 0;
        a = upper ? pa - a : a + pa;
        b = upper ? pb - b : b + pb;
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

int launch_had_pre(const uint16_t* x, int rows, int n, const uint16_t* suh, int n_sub,
                   uint16_t* xh, hipStream_t stream) {
    if (!x || !xh) return EXL3_E_NULL_POINTER;
    if (rows < 0 || n <= 0 || n % 128 || n_sub < 1) return EXL3_E_BAD_SHAPE;
    if (!suh && n_sub != 1) return EXL3_E_BAD_SHAPE;
    if (rows == 0) return EXL3_OK;
    const long long waves = (long long)rows * n_sub * (n / 128);
    const long long grid = (waves + 3) / 4;
    if (grid > 0x7FFFFFFFLL) return EXL3_E_BAD_SHAPE;
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
    if (y_is_fp32)
        had_post_kernel<true><<<dim3((unsigned)grid), dim3(256), 0, stream>>>(y, n_sum, sum_stride,
                                                                              s, b, o, rows, n);
    else
        had_post_kernel<false><<<dim3((unsigned)grid), dim3(256), 0, stream>>>(y, 1, 0, s, b, o,
                                                                               rows, n);
    return launch_status();
}

}  // namespace exl3

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
