// Prefill GEMM: y = xh @ W_inner with the trellis decoded into LDS and
// contracted on fp16 MFMA (v_mfma_f32_16x16x32_f16), fp32 accumulation.
//
// Tiling (one workgroup = 4 wavefronts, two workgroups fit a CU so the decode
// phase of one overlaps the MFMA phase of the other):
//   block tile   BM x BN = 256 rows x 128 columns, BK = 64 (four tile rows)
//   wave tile    128 x 64 -> 8 x 4 accumulator tiles of 16x16 (128 VGPRs)
//   per BK step  wave w decodes tile row k0/16 + w of the block's 8 tile columns
//                (one 256*K-byte wave-wide load, 32 codewords per lane) and
//                writes fp16 columns into the B tile; all threads copy the
//                256 x 64 activation tile into the A tile.
// LDS rows (64 halfs) are padded to 72 halfs so that 16-byte fragment reads of
// 8 consecutive rows touch all 32 banks once.
//
// The MFMA is issued as D^T = B^T A^T (weights as the first operand), so a lane
// ends up with 4 consecutive output columns of one row and stores 8 bytes.
//
// Replaces the rows > 16 ladder of EXL3Linear.__call__
// (ponyexl3/mlx/exl3_linear.py:137-161) and the decode-into-threadgroup-memory
// GEMM of ponyexl3/mlx/gemv_metal.py:1518-1741.
#include "exl3_device.hpp"
#include "exl3_host.hpp"

namespace exl3 {

constexpr int BM = 256, BN = 128, BK = 64;
constexpr int LDS_LD = BK + 8;  // halfs per padded LDS row

template <int K, int CB>
__global__ __launch_bounds__(256, 2) void gemm_kernel(const uint32_t* __restrict__ trellis,
                                                      const half_t* __restrict__ xh,
                                                      half_t* __restrict__ y, int rows,
                                                      size_t ldx, size_t ldy, int in_tiles,
                                                      int out_tiles, int tn_offset) {
    __shared__ __attribute__((aligned(16))) half_t a_s[BM * LDS_LD];
    __shared__ __attribute__((aligned(16))) half_t b_s[BN * LDS_LD];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;  // wave tile origin: rows wm*128, cols wn*64
    const int m0 = blockIdx.y * BM;
    const int g = blockIdx.x;  // 128-column group inside the slice
    const int tn0 = tn_offset + g * 8;

    float4_t acc[8][4];
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = float4_t{0.f, 0.f, 0.f, 0.f};

    const size_t row_words = (size_t)out_tiles * (8 * K);
    const uint32_t* tbase = trellis + (size_t)tn0 * (8 * K) + lane * K;

    // A-tile copy assignment: chunk c = tid + 256*i covers row c/8, halfs (c%8)*8..+7
    uint4_t a_reg[8];
    uint32_t w_reg[K];

    auto load_global = [&](int kstep) {
        const uint32_t* p = tbase + (size_t)(kstep * 4 + wave) * row_words;
#pragma unroll
        for (int i = 0; i < K; i++) w_reg[i] = p[i];
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int c = tid + 256 * i;
            const int r = m0 + (c >> 3);
            if (r < rows)
                a_reg[i] = *reinterpret_cast<const uint4_t*>(xh + (size_t)r * ldx +
                                                             (size_t)kstep * BK + (c & 7) * 8);
            else
                a_reg[i] = uint4_t{0u, 0u, 0u, 0u};
        }
    };

    auto store_lds = [&]() {
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int c = tid + 256 * i;
            *reinterpret_cast<uint4_t*>(&a_s[(c >> 3) * LDS_LD + (c & 7) * 8]) = a_reg[i];
        }
        const LaneWords<K> lw = finish_lane_words<K>(w_reg, lane);
        half2_t wp[16];
        decode_lane<K, CB>(lw, wp);
        const int col = (lane >> 3) * 16 + (lane & 7);
#pragma unroll
        for (int cs = 0; cs < 2; cs++) {
            half_t* dst = &b_s[(col + 8 * cs) * LDS_LD + wave * 16];
            uint4_t v0, v1;
            v0.x = half2_to_bits(wp[8 * cs + 0]);
            v0.y = half2_to_bits(wp[8 * cs + 1]);
            v0.z = half2_to_bits(wp[8 * cs + 2]);
            v0.w = half2_to_bits(wp[8 * cs + 3]);
            v1.x = half2_to_bits(wp[8 * cs + 4]);
            v1.y = half2_to_bits(wp[8 * cs + 5]);
            v1.z = half2_to_bits(wp[8 * cs + 6]);
            v1.w = half2_to_bits(wp[8 * cs + 7]);
            *reinterpret_cast<uint4_t*>(dst) = v0;
            *reinterpret_cast<uint4_t*>(dst + 8) = v1;
        }
    };

    const int ksteps = in_tiles / 4;
    load_global(0);
    store_lds();
    __syncthreads();

    const int fr = lane & 15, fk = (lane >> 4) * 8;
    for (int ks = 0; ks < ksteps; ks++) {
        if (ks + 1 < ksteps) load_global(ks + 1);
        // MFMA phase. Fragment reads are software-pipelined by hand: the A
        // fragments of the next pair of 16-row tiles are requested before the
        // eight MFMAs of the current pair are issued, so LDS latency hides
        // behind 128 cycles of matrix work instead of stalling every 4 MFMAs.
#pragma unroll
        for (int kk = 0; kk < 2; kk++) {
            half8_t bf[4];
            half8_t af[2][2];
            auto load_a = [&](int i) {
                return *reinterpret_cast<const half8_t*>(
                    &a_s[(wm * 128 + i * 16 + fr) * LDS_LD + kk * 32 + fk]);
            };
#pragma unroll
            for (int j = 0; j < 4; j++)
                bf[j] = *reinterpret_cast<const half8_t*>(
                    &b_s[(wn * 64 + j * 16 + fr) * LDS_LD + kk * 32 + fk]);
            af[0][0] = load_a(0);
            af[0][1] = load_a(1);
            __builtin_amdgcn_sched_group_barrier(0x100, 6, 0);  // 4 B + 2 A fragment reads
#pragma unroll
            for (int ip = 0; ip < 4; ip++) {
                if (ip < 3) {
                    af[(ip + 1) & 1][0] = load_a(2 * ip + 2);
                    af[(ip + 1) & 1][1] = load_a(2 * ip + 3);
                }
#pragma unroll
                for (int h = 0; h < 2; h++)
#pragma unroll
                    for (int j = 0; j < 4; j++)
                        acc[2 * ip + h][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                            bf[j], af[ip & 1][h], acc[2 * ip + h][j], 0, 0, 0);
                // pin the order: next pair's two reads first, then this pair's eight MFMAs
                if (ip < 3) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
                __builtin_amdgcn_sched_group_barrier(0x008, 8, 0);
            }
        }
        __syncthreads();
        if (ks + 1 < ksteps) {
            store_lds();
            __syncthreads();
        }
    }

    // acc[i][j] is D^T: lane holds columns n = 4*(lane/16)+0..3 of row m = lane%16
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const int r = m0 + wm * 128 + i * 16 + fr;
        if (r < rows) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int c = g * 128 + wn * 64 + j * 16 + (lane >> 4) * 4;
                half4_t o;
                o.x = (half_t)acc[i][j].x;
                o.y = (half_t)acc[i][j].y;
                o.z = (half_t)acc[i][j].z;
                o.w = (half_t)acc[i][j].w;
                *reinterpret_cast<half4_t*>(y + (size_t)r * ldy + c) = o;
            }
        }
    }
}

int launch_gemm(const uint16_t* xh, int rows, size_t ldx, const uint16_t* trellis, int in_tiles,
                int out_tiles, int K, int cb, int tn_offset, int tn_count, uint16_t* y_out,
                size_t ldy, hipStream_t stream) {
    if (int rc = check_k_cb(K, cb)) return rc;
    if (!xh || !trellis || !y_out) return EXL3_E_NULL_POINTER;
    if (rows < 1 || in_tiles < 4 || in_tiles % 4 || tn_offset < 0 || tn_count < 8 ||
        tn_count % 8 || tn_offset + tn_count > out_tiles || ldx < (size_t)in_tiles * 16 ||
        ldy < (size_t)tn_count * 16 || ldx % 8 || ldy % 4)
        return EXL3_E_BAD_SHAPE;
    if ((reinterpret_cast<uintptr_t>(xh) & 15) || (reinterpret_cast<uintptr_t>(y_out) & 7))
        return EXL3_E_BAD_SHAPE;
    const long long gy = ((long long)rows + BM - 1) / BM;
    if (gy > 65535) return EXL3_E_BAD_SHAPE;
    const dim3 grid((unsigned)(tn_count / 8), (unsigned)gy);
    return dispatch_k_cb(K, cb, [&](auto k, auto c) {
        gemm_kernel<k.value, c.value><<<grid, dim3(256), 0, stream>>>(
            reinterpret_cast<const uint32_t*>(trellis), reinterpret_cast<const half_t*>(xh),
            reinterpret_cast<half_t*>(y_out), rows, ldx, ldy, in_tiles, out_tiles, tn_offset);
        return launch_status();
    });
}

}  // namespace exl3

EXL3_EXPORT int exl3_gemm(const uint16_t* xh, int rows, size_t ldx, const uint16_t* trellis,
                          int in_tiles, int out_tiles, int K, int cb, int tn_offset, int tn_count,
                          uint16_t* y_out, size_t ldy, void* stream) {
    return exl3::launch_gemm(xh, rows, ldx, trellis, in_tiles, out_tiles, K, cb, tn_offset,
                             tn_count, y_out, ldy, exl3::as_stream(stream));
}
