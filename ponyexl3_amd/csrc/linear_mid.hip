// Medium-batch layer kernel (rows 9..32): the regime where every weight should
// still be decoded exactly once per launch (the decode sets the pace) but the dot
// products no longer fit the 4x4x4 matrix instruction of the small-batch kernel.
//
// The trellis format was laid out for a 16x8x16 tensor-core fragment
// (ponyexl3/ref/perm.py:8-25): "thread" t = 0..31 of a tile owns the eight
// codewords 8t..8t+7, which are input rows {2g, 2g+1, 2g+8, 2g+9} (g = t & 3) of
// the output columns c and c + 8 (c = t >> 2). Four such values are one lane's
// share of a B operand of the 16x16 matrix instructions: lane l supplies
// consecutive k-slots (group l >> 4) of column l & 15. So here a lane does not own
// 32 consecutive codewords as in the small-batch kernels; lane l of a wave owns
// thread t = 4*(l & 7) + (l >> 4) of tile (l >> 3) & 1 of a tile pair, decodes
// its eight codewords and feeds them to the matrix pipe straight from registers;
// two tile rows fill the eight k-slots of v_mfma_f32_16x16x32_f16. The order of
// the k-slots is free as long as the activations use the same one, so the
// rotated activations are staged in LDS already in operand order (one
// conflict-free ds_read_b128 per lane and 16-row fragment). No weight ever
// passes through LDS; the only exchange is inside the wave: the tile pair is
// loaded with consecutive lanes on consecutive dwords (lanes a tile thread's
// stride apart would cost one cache access each) and every lane then picks the
// dwords of its bit window from the lanes that hold them (ds_bpermute).
//
// Workgroup = one 128-column group (one block of the output Hadamard) over the
// 128-row blocks of one split. Wave w takes tile rows 2w and 2w + 1 of every
// block, on all four tile pairs, so that one activation operand serves eight
// matrix instructions; a wave stages exactly the activations it reads, so the
// main loop has no workgroup barrier. The waves' sums are added through LDS as
// (wave 0 + wave 1) + (wave 2 + wave 3); splits meet through fp32 partial rows
// and a per-group counter exactly as in the small-batch layer kernel: the
// workgroup that arrives last adds the partial rows in split order, rounds to fp16 (ponyexl3/ref/forward.py:41), applies the output
// Hadamard, svh and bias. Counters must be zero on entry and are zero again on
// exit.
//
// x is already rotated: fp16 [rows][n_sub][in] (the Hadamard kernel's output).
#include "exl3_device.hpp"
#include "exl3_host.hpp"
#include "exl3_small.hpp"

#include <type_traits>

namespace exl3 {

// Dwords of the tile stream a lane needs for its eight codewords: the window
// ends at the dword boundary at or after the end of codeword 8t+7 and must hold
// 7K + 16 bits above the (at most 31, for K = 4 and 8 zero) bits of slack.
template <int K>
constexpr int mid_window_words() {
    return K <= 4 ? 2 : 3;
}

// The lane's window, shifted right by its slack so that codeword j ends at bit
// (7 - j) * K of the 96-bit value (top : hi : lo).
struct MidWindow {
    uint32_t lo, hi, top;
};

template <int K>
__device__ __forceinline__ MidWindow mid_align(const uint32_t (&w)[mid_window_words<K>()],
                                               int slack) {
    constexpr int NW = mid_window_words<K>();
    MidWindow a;
    if constexpr (K % 4 == 0) {  // slack is zero for every lane
        a.lo = w[NW - 1];
        a.hi = w[NW - 2];
        a.top = NW == 3 ? w[0] : 0u;
    } else {
        a.lo = __builtin_amdgcn_alignbit(w[NW - 2], w[NW - 1], slack);
        if constexpr (NW == 3) {
            a.hi = __builtin_amdgcn_alignbit(w[0], w[1], slack);
            a.top = w[0] >> slack;
        } else {
            a.hi = w[0] >> slack;
            a.top = 0u;
        }
    }
    return a;
}

// Codeword J (0..7) of the lane's thread.
template <int K, int J>
__device__ __forceinline__ uint32_t mid_codeword(const MidWindow& a) {
    constexpr int s = (7 - J) * K;
    if constexpr (s + 16 <= 32) {
        return (a.lo >> s) & 0xFFFFu;
    } else if constexpr (s < 32) {
        const uint32_t mid = __builtin_amdgcn_alignbit(a.hi, a.lo, 16);
        return (mid >> (s - 16)) & 0xFFFFu;
    } else if constexpr (s - 32 + 16 <= 32) {
        return (a.hi >> (s - 32)) & 0xFFFFu;
    } else {
        const uint32_t mid = __builtin_amdgcn_alignbit(a.top, a.hi, 16);
        return (mid >> (s - 48)) & 0xFFFFu;
    }
}

template <int K, int CB, int MF>
__global__ __launch_bounds__(256, 2) void linear_mid_kernel(
    const uint32_t* __restrict__ trellis, const half_t* __restrict__ xh,
    const half_t* __restrict__ svh, const half_t* __restrict__ bias, half_t* __restrict__ y,
    float* partial, int* counters, const int* __restrict__ group_sub, int in_tiles, int out_tiles,
    int rows, int n_groups, int blocks_per_split, int n_splits, int n_sub) {
    constexpr int M = 16 * MF;
    constexpr int NW = mid_window_words<K>();
    constexpr int NL = (16 * K + 63) / 64;  // wave-wide loads that cover one tile pair
    constexpr int kDepth = 2;  // blocks ahead that a wave has its loads out for
    // Activations of one 128-row block, two buffers, laid out as the A operands of
    // the matrix instruction: [buffer][fragment][row pair of the block][lane][8 halfs].
    // After the main loop the same memory holds the fp32 sums of the workgroup: two
    // [M][kRedLd] arrays (waves 0+1 and waves 2+3). kRedLd = 130 puts the four row
    // groups of a lane quartet eight banks apart, so a wave's accesses are two per
    // bank, the minimum for 64 lanes.
    constexpr int kRedLd = 130;
    constexpr size_t kStageBytes = (size_t)2 * MF * 4 * 64 * 8 * sizeof(half_t);
    constexpr size_t kRedBytes = (size_t)2 * M * kRedLd * sizeof(float);
    __shared__ __attribute__((aligned(16))) char lds_raw[kStageBytes > kRedBytes ? kStageBytes : kRedBytes];
    half_t(*xs)[MF][4][64][8] = reinterpret_cast<half_t(*)[MF][4][64][8]>(lds_raw);
    __shared__ int last_flag;
    const int g = blockIdx.x;
    const int split = blockIdx.y;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int sub = group_sub ? group_sub[g] : 0;
    const int in_features = in_tiles * 16;
    const int n_blocks = in_tiles >> 3;
    const int blk_begin = split * blocks_per_split;
    const int blk_end = min(n_blocks, blk_begin + blocks_per_split);

    // the lane's place in the matrix instruction and in its tile
    const int col16 = lane & 15, kgroup = lane >> 4;
    const int thread_t = 4 * (col16 & 7) + kgroup;
    const int end_bit = (8 * thread_t + 8) * K;
    const int end_word = (end_bit + 31) >> 5;  // exclusive
    const int slack = end_word * 32 - end_bit;
    const size_t row_words = (size_t)out_tiles * (8 * K);
    // A tile pair is 16K consecutive dwords of a tile row. The lanes load them in
    // order (NL wave-wide loads of consecutive dwords; lanes whose addresses are a
    // tile thread's stride apart would cost one cache access each) and each lane
    // then fetches the NW dwords of its window from the lanes that hold them.
    const uint32_t* group_base = trellis + (size_t)g * 8 * (8 * K) + lane;
    int src_word[NW];  // index of the wanted dword within the pair: load (index >> 6), lane (index & 63)
#pragma unroll
    for (int i = 0; i < NW; i++)
        src_word[i] = (col16 >> 3) * (8 * K) + (end_word - NW + i + 8 * K) % (8 * K);

    // Wave w works on row pair w (tile rows 2w, 2w + 1) of every block of the split,
    // on all four tile pairs of the group: one A operand serves eight matrix
    // instructions per fragment.
    struct PairRows {
        uint32_t raw[2][NL];
    };
    auto load_pairs = [&](int blk, PairRows (&dst)[4]) {
        const int b = min(blk, blk_end - 1);
        const uint32_t* p = group_base + (size_t)(b * 8 + 2 * wave) * row_words;
#pragma unroll
        for (int q = 0; q < 4; q++)
#pragma unroll
            for (int r = 0; r < 2; r++)
#pragma unroll
                for (int i = 0; i < NL; i++) {
                    const uint32_t* src = p + (size_t)r * row_words + q * (16 * K) + 64 * i;
                    if (64 * (i + 1) <= 16 * K || lane < 16 * K - 64 * i)
                        dst[q].raw[r][i] = __builtin_nontemporal_load(src);
                    else
                        dst[q].raw[r][i] = 0u;
                }
    };
    auto decode_row = [&](const uint32_t (&raw)[NL], uint32_t& lo0, uint32_t& lo1, uint32_t& hi0,
                          uint32_t& hi1) {
        uint32_t w[NW];
#pragma unroll
        for (int i = 0; i < NW; i++) {
            const int a = __builtin_amdgcn_ds_bpermute((src_word[i] & 63) << 2, (int)raw[0]);
            if constexpr (NL == 2) {
                const int b = __builtin_amdgcn_ds_bpermute((src_word[i] & 63) << 2, (int)raw[1]);
                w[i] = (uint32_t)(src_word[i] < 64 ? a : b);
            } else {
                w[i] = (uint32_t)a;
            }
        }
        const MidWindow win = mid_align<K>(w, slack);
        half2_t w00, w01, w10, w11;
        decode_pair2<CB>(mid_codeword<K, 0>(win), mid_codeword<K, 1>(win), mid_codeword<K, 2>(win),
                         mid_codeword<K, 3>(win), w00, w01);
        decode_pair2<CB>(mid_codeword<K, 4>(win), mid_codeword<K, 5>(win), mid_codeword<K, 6>(win),
                         mid_codeword<K, 7>(win), w10, w11);
        lo0 = half2_to_bits(w00);
        lo1 = half2_to_bits(w01);
        hi0 = half2_to_bits(w10);
        hi1 = half2_to_bits(w11);
    };

    // staging of the activations: 16-byte chunks of a row (input rows 2j, 2j+1 of one
    // half of a tile row), MF per thread and block; the four dwords of a chunk go
    // to the four k-groups' operands. Wave w stages row pair w: lane -> batch row
    // lane >> 2 of a fragment, chunk lane & 3 of the pair, which spreads a store
    // instruction over all LDS banks (two lanes per bank).
    const half_t* x_rows = xh + (size_t)sub * in_features;
    const size_t x_stride = (size_t)n_sub * in_features;
    uint4_t xr[MF];
    auto fetch_x = [&](int blk) {
#pragma unroll
        for (int f = 0; f < MF; f++) {
            const int r = min(16 * f + (lane >> 2), rows - 1);
            xr[f] = *reinterpret_cast<const uint4_t*>(x_rows + (size_t)r * x_stride + blk * 128 +
                                                      (4 * wave + (lane & 3)) * 8);
        }
    };
    auto stage_x = [&](int which) {
        const int odd = (lane >> 1) & 1, hi = lane & 1;  // tile row 2w + odd, upper half hi
#pragma unroll
        for (int f = 0; f < MF; f++) {
            const uint32_t d[4] = {xr[f].x, xr[f].y, xr[f].z, xr[f].w};
#pragma unroll
            for (int kg = 0; kg < 4; kg++)
                *reinterpret_cast<uint32_t*>(
                    &xs[which][f][wave][16 * kg + (lane >> 2)][odd * 4 + hi * 2]) = d[kg];
        }
    };

    float4_t acc[4][2][MF];
#pragma unroll
    for (int q = 0; q < 4; q++)
#pragma unroll
        for (int v = 0; v < 2; v++)
#pragma unroll
            for (int f = 0; f < MF; f++) acc[q][v][f] = float4_t{0.f, 0.f, 0.f, 0.f};

    PairRows ring[kDepth][4];
#pragma unroll
    for (int d = 0; d < kDepth; d++) load_pairs(blk_begin + d, ring[d]);
    fetch_x(blk_begin);
    stage_x(0);
    if (blk_begin + 1 < blk_end) fetch_x(blk_begin + 1);
    // a wave stages exactly the operands it reads itself (row pair w), so the
    // waves of the workgroup never wait for each other inside the loop
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();

    static_assert(kDepth % 2 == 0, "the staging buffer of a block is its ring slot & 1");
    for (int blk4 = blk_begin; blk4 < blk_end; blk4 += kDepth) {
#pragma unroll
        for (int h = 0; h < kDepth; h++) {
            const int blk = blk4 + h;
            if (blk >= blk_end) break;
            // blk - blk_begin == h (mod kDepth): the staging buffer of this block is h & 1
            if (blk + 1 < blk_end) {
                stage_x((h + 1) & 1);
                if (blk + 2 < blk_end) fetch_x(blk + 2);
            }
            uint4_t a[MF];
#pragma unroll
            for (int f = 0; f < MF; f++)
                a[f] = *reinterpret_cast<const uint4_t*>(&xs[h & 1][f][wave][lane][0]);
#pragma unroll
            for (int q = 0; q < 4; q++) {
                uint32_t c0[4], c1[4];  // columns c and c + 8: k-slots of row 2w, then of row 2w + 1
                decode_row(ring[h][q].raw[0], c0[0], c0[1], c1[0], c1[1]);
                decode_row(ring[h][q].raw[1], c0[2], c0[3], c1[2], c1[3]);
                const uint4_t b0 = {c0[0], c0[1], c0[2], c0[3]};
                const uint4_t b1 = {c1[0], c1[1], c1[2], c1[3]};
#pragma unroll
                for (int f = 0; f < MF; f++) {
                    acc[q][0][f] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                        __builtin_bit_cast(half8_t, a[f]), __builtin_bit_cast(half8_t, b0),
                        acc[q][0][f], 0, 0, 0);
                    acc[q][1][f] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                        __builtin_bit_cast(half8_t, a[f]), __builtin_bit_cast(half8_t, b1),
                        acc[q][1][f], 0, 0, 0);
                }
            }
            load_pairs(blk + kDepth, ring[h]);
            // this block's operands are consumed, the next block's are staged
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
        }
    }

    // ---- the four waves' sums are added through LDS, (wave 0 + wave 1) +
    // (wave 2 + wave 3), in the staging memory once every wave has left the loop
    __syncthreads();
    float(*red)[M][kRedLd] = reinterpret_cast<float(*)[M][kRedLd]>(lds_raw);
#pragma unroll
    for (int phase = 0; phase < 2; phase++) {
        if ((wave & 1) == phase) {
            float(*dstbuf)[kRedLd] = red[wave >> 1];
#pragma unroll
            for (int q = 0; q < 4; q++)
#pragma unroll
                for (int v = 0; v < 2; v++)
#pragma unroll
                    for (int f = 0; f < MF; f++)
#pragma unroll
                        for (int r = 0; r < 4; r++) {
                            float* dst = &dstbuf[16 * f + 4 * kgroup + r]
                                                [(2 * q + (col16 >> 3)) * 16 + (col16 & 7) + 8 * v];
                            *dst = phase == 0 ? acc[q][v][f][r] : __fadd_rn(*dst, acc[q][v][f][r]);
                        }
        }
        __syncthreads();
    }

    // ---- publish this split's partial rows with device-scope stores (the XCDs' L2
    // caches are not coherent with each other), then count the workgroup in.
    const size_t out_total = (size_t)n_groups * 128;
    for (int idx = threadIdx.x; idx < rows * 64; idx += 256) {
        const int m = idx >> 6, c2 = idx & 63;
        const float2_t v = {__fadd_rn(red[0][m][2 * c2], red[1][m][2 * c2]),
                            __fadd_rn(red[0][m][2 * c2 + 1], red[1][m][2 * c2 + 1])};
        __hip_atomic_store(reinterpret_cast<uint64_t*>(partial + ((size_t)split * rows + m) * out_total +
                                                       (size_t)g * 128 + 2 * c2),
                           __builtin_bit_cast(uint64_t, v), __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0) {
        const int seen =
            __hip_atomic_fetch_add(&counters[g], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        last_flag = seen == n_splits - 1;
    }
    __syncthreads();
    if (!last_flag) return;
    asm volatile("" ::: "memory");

    // ---- the last workgroup of the group finishes its 128 columns: four batch
    // rows per wave at a time, eight splits of each in flight
    const size_t col = (size_t)g * 128 + 2 * lane;
    half2_t sv, bv;
    if (svh) sv = *reinterpret_cast<const half2_t*>(svh + col);
    if (bias) bv = *reinterpret_cast<const half2_t*>(bias + col);
    const size_t stride = (size_t)rows * out_total;
    constexpr int RB = 4, SB = 8;
    for (int m0 = wave * RB; m0 < rows; m0 += 4 * RB) {
        float sa[RB], sb[RB];
#pragma unroll
        for (int i = 0; i < RB; i++) sa[i] = sb[i] = 0.f;
        for (int s0 = 0; s0 < n_splits; s0 += SB) {
            uint64_t v[SB][RB];
#pragma unroll
            for (int j = 0; j < SB; j++)
#pragma unroll
                for (int i = 0; i < RB; i++) {
                    const int m = min(m0 + i, rows - 1);
                    const int s = min(s0 + j, n_splits - 1);
                    v[j][i] = __hip_atomic_load(
                        reinterpret_cast<const uint64_t*>(partial + (size_t)s * stride +
                                                          (size_t)m * out_total + col),
                        __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
#pragma unroll
            for (int j = 0; j < SB; j++)
                if (s0 + j < n_splits) {
#pragma unroll
                    for (int i = 0; i < RB; i++) {
                        const float2_t f = __builtin_bit_cast(float2_t, v[j][i]);
                        sa[i] = __fadd_rn(sa[i], f.x);
                        sb[i] = __fadd_rn(sb[i], f.y);
                    }
                }
        }
#pragma unroll
        for (int i = 0; i < RB; i++) {
            const int m = m0 + i;
            if (m >= rows) break;
            float a = (float)(half_t)sa[i], b = (float)(half_t)sb[i];
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
    if (threadIdx.x == 0)
        __hip_atomic_store(&counters[g], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

int linear_mid_max_rows() {
    static const int v = env_int("EXL3_LINEAR_MID_MAX_ROWS", kLinearMidMaxRows, 0, kLinearMidMaxRows);
    return v;
}

// Splits of the reduction: enough workgroups for kWgPerCu per CU, but never more
// than kMaxSplits partial rows per output (each costs a write and a read of
// rows x out floats, and the finishing workgroup fetches eight of them per round
// trip) - or twice that where a split then still has eight blocks to stream
// (17408 -> 5120 at 16 rows: 8 splits = 320 workgroups 34.0 us, 16 splits 29.8 us;
// with four or five blocks per split the extra splits cost more than they gain).
MidPlan plan_linear_mid(int rows, int in_tiles, int n_groups) {
    (void)rows;
    static const int kWgPerCu = env_int("EXL3_LINEAR_MID_WG_PER_CU", 4, 1, 16);
    static const int kMaxSplits = env_int("EXL3_LINEAR_MID_MAX_SPLITS", 8, 1, 256);
    const int n_blocks = in_tiles / 8;
    int want = (256 * kWgPerCu + n_groups - 1) / (n_groups > 0 ? n_groups : 1);
    if (want >= 2 * kMaxSplits && n_blocks >= 2 * kMaxSplits * 8) want = 2 * kMaxSplits;
    else if (want > kMaxSplits) want = kMaxSplits;
    if (want > n_blocks) want = n_blocks;
    if (want < 1) want = 1;
    const int blocks_per_split = (n_blocks + want - 1) / want;
    const int n_splits = (n_blocks + blocks_per_split - 1) / blocks_per_split;
    return MidPlan{n_splits, blocks_per_split};
}

int launch_linear_mid(const uint16_t* xh, int rows, const uint16_t* trellis, int in_tiles,
                      int out_tiles, int K, int cb, int n_sub, const int32_t* group_sub,
                      const uint16_t* svh, const uint16_t* bias, uint16_t* y, float* partial,
                      int* counters, MidPlan plan, hipStream_t stream) {
    if (int rc = check_k_cb(K, cb)) return rc;
    if (!xh || !trellis || !y || !partial || !counters) return EXL3_E_NULL_POINTER;
    if (rows < 1 || rows > kLinearMidMaxRows || n_sub < 1 || in_tiles < 8 || out_tiles < 8 ||
        in_tiles % 8 || out_tiles % 8)
        return EXL3_E_BAD_SHAPE;
    if (n_sub > 1 && !group_sub) return EXL3_E_BAD_INDEX;
    if (plan.n_splits < 1 || plan.n_splits > 65535 || plan.blocks_per_split < 1 ||
        (long long)plan.n_splits * plan.blocks_per_split < in_tiles / 8 ||
        (long long)(plan.n_splits - 1) * plan.blocks_per_split >= in_tiles / 8)
        return EXL3_E_BAD_SHAPE;
    const int n_groups = out_tiles / 8;
    const dim3 grid((unsigned)n_groups, (unsigned)plan.n_splits);
    const int mf = rows <= 16 ? 1 : 2;
    return dispatch_k_cb(K, cb, [&](auto k, auto c) {
        auto go = [&](auto mfc) {
            linear_mid_kernel<k.value, c.value, mfc.value><<<grid, dim3(256), 0, stream>>>(
                reinterpret_cast<const uint32_t*>(trellis), reinterpret_cast<const half_t*>(xh),
                reinterpret_cast<const half_t*>(svh), reinterpret_cast<const half_t*>(bias),
                reinterpret_cast<half_t*>(y), partial, counters, group_sub, in_tiles, out_tiles,
                rows, n_groups, plan.blocks_per_split, plan.n_splits, n_sub);
        };
        switch (mf) {
            case 1: go(std::integral_constant<int, 1>{}); break;
            default: go(std::integral_constant<int, 2>{}); break;
        }
        return launch_status();
    });
}

}  // namespace exl3
