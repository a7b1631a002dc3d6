// Device-side building blocks shared by every EXL3 kernel: fp16 helpers, the
// procedural codebooks and the per-lane view of a packed trellis tile.
//
// Written for gfx950 (CDNA4) only: 64-wide wavefronts, v_bitop3_b32,
// v_dot2_f32_f16 and the fp16 MFMA family are assumed to exist.
//
// Bitstream facts used throughout (reference: ponyexl3/ref/trellis.py:105-141):
//   * a tile is a circular stream of 256*K bits stored as 8*K little-endian
//     uint32 words; stream bit b is bit 31-(b%32) of word b/32;
//   * codeword c (0..255) is the 16 stream bits that end (exclusive) at bit
//     (c+1)*K, most significant bit first.
// Tile order facts (reference: ponyexl3/ref/perm.py:8-25): codewords 4l..4l+3
// (l = 0..63) all belong to output column (l>>3) + 8*(l&1) and to input rows
// {2q, 2q+1, 2q+8, 2q+9} with q = (l>>1)&3.
//
// Lane view: one tile is handled by 8 consecutive lanes. Lane u (0..7) owns
// codewords 32u..32u+31, whose fresh bits are the K dwords [u*K, (u+1)*K) of the
// tile, plus the last 16-K bits of the dword before them (the last dword of the
// tile for u = 0: the stream is circular). Those 32 codewords are the two output
// columns u and u+8 across all 16 input rows, so a lane can accumulate two
// output columns without ever exchanging data with another lane.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace exl3 {

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float2_t __attribute__((ext_vector_type(2)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef uint32_t uint2_t __attribute__((ext_vector_type(2)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));

constexpr int kWave = 64;
constexpr int kLanesPerTile = 8;    // lanes that share one 16x16 tile
constexpr int kTilesPerWave = 8;    // tiles covered by one wave-wide load
constexpr int kColsPerGroup = 128;  // output columns of one wave-wide load

template <int Begin, int End, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (Begin < End) {
        f(std::integral_constant<int, Begin>{});
        static_for<Begin + 1, End>(f);
    }
}

__device__ __forceinline__ half_t bits_to_half(uint16_t b) { return __builtin_bit_cast(half_t, b); }
__device__ __forceinline__ uint16_t half_to_bits(half_t h) { return __builtin_bit_cast(uint16_t, h); }
__device__ __forceinline__ half2_t bits_to_half2(uint32_t b) { return __builtin_bit_cast(half2_t, b); }
__device__ __forceinline__ uint32_t half2_to_bits(half2_t h) { return __builtin_bit_cast(uint32_t, h); }

// Codebook ids as in ponyexl3/ref/codebook.py:9-12.
enum : int { CB_3INST = 0, CB_MCG = 1, CB_MUL1 = 2 };

// One codeword (value < 65536) -> one fp16 weight, bit-exact with
// ponyexl3/ref/codebook.py:66-91.
//
// 3INST / MCG: x = cw*M + A (mod 2^32); x = (x & 0x8FFF8FFF) ^ 0x3B603B60; the
// result is the fp16 sum of the two halves of x (one rounding).
//
// MUL1: x = cw*0x83DCD12D; h = 1024 + (sum of the four bytes of x);
// result = fp16(h * K_INV + K_BIAS). h*K_INV + K_BIAS is an integer multiple of
// 2^-18 below 2^4, hence exact in fp32, so the single fp32->fp16 conversion is
// the only rounding (the reference rounds once from double).
//
// Instruction choice follows measured gfx950 issue rates: v_mul_lo_u32 and
// v_mad_u64_u32 run at the full 16 lanes/clk/SIMD, v_bitop3_b32 at the faster
// rate of the simple ALU ops, and a v_add_f16 with SDWA operands adds the two
// halves of one register and writes either half of the destination, so a pair
// of weights is produced already packed for v_dot2_f32_f16 / MFMA.

// x after the mask/xor step for 3INST and MCG.
template <int CB>
__device__ __forceinline__ uint32_t scramble(uint32_t cw) {
    static_assert(CB == CB_3INST || CB == CB_MCG, "MUL1 has its own path");
    uint32_t x;
    if constexpr (CB == CB_3INST) {
        // one v_mad_u64_u32: the low dword of cw*M + A
        uint64_t wide, carry;
        const uint64_t addend = 64248484ull;
        asm("v_mad_u64_u32 %0, %1, %2, %3, %4"
            : "=v"(wide), "=s"(carry)
            : "v"(cw), "s"(89226354u), "v"(addend));
        x = (uint32_t)wide;
    } else {
        x = cw * 0xCBAC1FEDu;
    }
    return __builtin_amdgcn_bitop3_b32(x, 0x8FFF8FFFu, 0x3B603B60u, 0x6A);  // c ^ (a & b)
}

// Two packed pairs at once:
//   ra = (half(x0.lo) + half(x0.hi), half(x1.lo) + half(x1.hi)), rb likewise from x2, x3.
// A VALU instruction that writes only half of a VGPR (SDWA dst_sel, here also the
// UNUSED_PRESERVE read-modify-write of the second add) must be separated by one
// wait state from any VALU or MFMA instruction that reads that VGPR on gfx950;
// the compiler inserts those for its own instructions but cannot see inside
// inline assembly. The block therefore interleaves the two pairs (each register
// is touched every other instruction) and ends with one s_nop, so whatever the
// scheduler places behind it is far enough away. Measured without it: an MFMA
// issued right after the add read a stale upper half.
__device__ __forceinline__ void add_halves_pack2(uint32_t x0, uint32_t x1, uint32_t x2,
                                                 uint32_t x3, half2_t& ra, half2_t& rb) {
    uint32_t a, b;
    asm("v_add_f16_sdwa %0, %2, %2 dst_sel:WORD_0 dst_unused:UNUSED_PAD src0_sel:WORD_0 "
        "src1_sel:WORD_1\n\t"
        "v_add_f16_sdwa %1, %4, %4 dst_sel:WORD_0 dst_unused:UNUSED_PAD src0_sel:WORD_0 "
        "src1_sel:WORD_1\n\t"
        "v_add_f16_sdwa %0, %3, %3 dst_sel:WORD_1 dst_unused:UNUSED_PRESERVE src0_sel:WORD_0 "
        "src1_sel:WORD_1\n\t"
        "v_add_f16_sdwa %1, %5, %5 dst_sel:WORD_1 dst_unused:UNUSED_PRESERVE src0_sel:WORD_0 "
        "src1_sel:WORD_1\n\t"
        "s_nop 0"
        : "=&v"(a), "=&v"(b)
        : "v"(x0), "v"(x1), "v"(x2), "v"(x3));
    ra = bits_to_half2(a);
    rb = bits_to_half2(b);
}

__device__ __forceinline__ half_t decode_mul1(uint32_t cw) {
    const uint32_t x = cw * 0x83DCD12Du;
    const uint32_t s = __builtin_amdgcn_sad_u8(x, 0u, 1024u);
    const float v = __builtin_fmaf((float)s, 0.00676727294921875f, -10.3828125f);
    return (half_t)v;
}

// Four codewords -> two packed pairs of fp16 weights (cw0, cw1) and (cw2, cw3).
template <int CB>
__device__ __forceinline__ void decode_pair2(uint32_t cw0, uint32_t cw1, uint32_t cw2,
                                             uint32_t cw3, half2_t& ra, half2_t& rb) {
    if constexpr (CB == CB_MUL1) {
        ra.x = decode_mul1(cw0);
        ra.y = decode_mul1(cw1);
        rb.x = decode_mul1(cw2);
        rb.y = decode_mul1(cw3);
    } else {
        add_halves_pack2(scramble<CB>(cw0), scramble<CB>(cw1), scramble<CB>(cw2),
                         scramble<CB>(cw3), ra, rb);
    }
}

// One codeword -> the dword whose two fp16 halves add up to the weight (3INST / MCG:
// the scrambled word itself; MUL1: the weight and a zero). A dot product is linear, so
// a kernel that feeds both halves to the matrix pipe as two k-slots against the same
// activation gets a * lo + a * hi in fp32 - the product with the exact sum of the two
// halves, which the fp16 weight is the rounding of - and saves the half add.
template <int CB>
__device__ __forceinline__ uint32_t weight_halves(uint32_t cw) {
    if constexpr (CB == CB_MUL1) return (uint32_t)half_to_bits(decode_mul1(cw));
    else return scramble<CB>(cw);
}

// The K+1 dwords a lane needs for its 32 codewords: w[0] is the dword that
// precedes the lane's own K dwords (already wrapped), w[1..K] are its own.
template <int K>
struct LaneWords {
    uint32_t w[K + 1];
};

// Codeword N (0..31) of a lane. Bits are numbered MSB-first from the start of
// w[0]; codeword N ends (exclusive) at bit 32 + (N+1)*K.
template <int K, int N>
__device__ __forceinline__ uint32_t lane_codeword(const LaneWords<K>& lw) {
    constexpr int end = 32 + (N + 1) * K;
    constexpr int wi = (end - 1) / 32;
    constexpr int sh = 32 * (wi + 1) - end;
    if constexpr (sh + 16 <= 32) {
        return (lw.w[wi] >> sh) & 0xFFFFu;  // one v_bfe_u32 (v_and / v_lshrrev at the ends)
    } else {
        // The window straddles two dwords. All straddling windows of one dword pair
        // share the same 16-bit funnel shift (one v_alignbit_b32, merged by common
        // subexpression elimination), after which each is one v_bfe_u32.
        const uint32_t mid = __builtin_amdgcn_alignbit(lw.w[wi - 1], lw.w[wi], 16);
        return (mid >> (sh - 16)) & 0xFFFFu;
    }
}

// Where codeword N of a lane sits inside the 16x16 tile:
//   column = u + 8*col_sel(N), row = tile_row(N).
__host__ __device__ constexpr int cw_col_sel(int n) { return (n >> 2) & 1; }
__host__ __device__ constexpr int cw_row(int n) {
    return 2 * ((n >> 3) & 3) + (n & 1) + 8 * ((n >> 1) & 1);
}

// Loads the K dwords of lane `lane` for the 8 tiles that start at dword
// `base` (tile tn0 of row tk) and fetches the preceding dword from the
// neighbouring lane (lane u-1 of the same tile, u = 0 wraps to u = 7).
template <int K>
__device__ __forceinline__ void load_lane_words(const uint32_t* __restrict__ base, int lane,
                                                uint32_t (&own)[K]) {
    const uint32_t* p = base + lane * K;
#pragma unroll
    for (int i = 0; i < K; i++) own[i] = p[i];
}

// The dword that precedes a lane's own K dwords: the last dword of lane u-1 of
// the same tile (u = 0 wraps to u = 7, the stream is circular). One ds_bpermute.
__device__ __forceinline__ uint32_t neighbour_word(uint32_t last_own, int lane) {
    const int src = (lane & ~7) | ((lane + 7) & 7);
    return (uint32_t)__shfl((int)last_own, src, kWave);
}

template <int K>
__device__ __forceinline__ LaneWords<K> make_lane_words(uint32_t prev, const uint32_t (&own)[K]) {
    LaneWords<K> lw;
    lw.w[0] = prev;
#pragma unroll
    for (int i = 0; i < K; i++) lw.w[i + 1] = own[i];
    return lw;
}

template <int K>
__device__ __forceinline__ LaneWords<K> finish_lane_words(const uint32_t (&own)[K], int lane) {
    return make_lane_words<K>(neighbour_word(own[K - 1], lane), own);
}

// Decodes the lane's 32 codewords into 16 half2 pairs.
// pair index p = 8*col_sel + q + 4*hi where the pair holds input rows
// (2q + 8*hi, 2q + 8*hi + 1) of column u + 8*col_sel, i.e. pair j of a column
// multiplies x[2j], x[2j+1] with j = q + 4*hi.
template <int K, int CB>
__device__ __forceinline__ void decode_lane(const LaneWords<K>& lw, half2_t (&wp)[16]) {
    static_for<0, 8>([&](auto pj) {
        constexpr int na = 4 * pj.value, nb = na + 2;  // even codewords of two consecutive pairs
        constexpr int ia = 8 * cw_col_sel(na) + (cw_row(na) >> 1);
        constexpr int ib = 8 * cw_col_sel(nb) + (cw_row(nb) >> 1);
        decode_pair2<CB>(lane_codeword<K, na>(lw), lane_codeword<K, na + 1>(lw),
                         lane_codeword<K, nb>(lw), lane_codeword<K, nb + 1>(lw), wp[ia], wp[ib]);
    });
}

// Cross-lane butterflies of the Walsh-Hadamard transforms, without a trip through LDS.
// Stage "lane ^ 2^BIT" of a value held one per lane: the lane whose BIT is clear gets
// v + partner, the other one partner - v. For BIT 0..3 the partner comes through a DPP
// operand (quad permutations for 1 and 2, a quad reversal followed by a half-row mirror
// for 4, a row rotation by 8 for 8) and the subtraction is the addition of v with its
// sign flipped in the upper lanes (`sign` = lane_sign_mask(lane, BIT)): partner + (-v)
// and v + partner round exactly like partner - v and v + partner.
__device__ __forceinline__ uint32_t lane_sign_mask(int lane, int bit) {
    return ((uint32_t)lane << (31 - bit)) & 0x80000000u;
}

template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
    return __builtin_bit_cast(
        float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, false));
}

template <int BIT>
__device__ __forceinline__ float butterfly_dpp(float v, uint32_t sign) {
    static_assert(BIT >= 0 && BIT <= 3, "lanes 16 and 32 apart are reached by swapping registers");
    const float own = __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, v) ^ sign);
    float partner;
    if constexpr (BIT == 0) partner = dpp_move<0xB1>(v);                         // quad_perm [1,0,3,2]
    else if constexpr (BIT == 1) partner = dpp_move<0x4E>(v);                    // quad_perm [2,3,0,1]
    else if constexpr (BIT == 2) partner = dpp_move<0x141>(dpp_move<0x1B>(v));   // [3,2,1,0], row_half_mirror
    else partner = dpp_move<0x128>(v);                                           // row_ror:8
    return __fadd_rn(partner, own);
}

// Stages "lane ^ 16" and "lane ^ 32" for two values a, b that both need them: the swap
// instructions of gfx950 exchange the odd 16-lane rows (upper 32 lanes) of a with the
// even rows (lower 32 lanes) of b, after which every lane holds a value and its partner
// side by side (even rows / lower half: those of a; the others: those of b), and the
// stage is an add and a subtract inside the lane. swap_back restores the layout (both
// swaps are involutions; undo them in reverse order).
__device__ __forceinline__ void swap_rows16(float& a, float& b) {
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ void swap_halves32(float& a, float& b) {
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ void butterfly_in_lane(float& a, float& b) {
    const float s = __fadd_rn(a, b), d = __fsub_rn(a, b);
    a = s;
    b = d;
}

// Unnormalised WHT over 128 values held as (a, b) = elements (2*lane, 2*lane+1);
// same butterfly order as ponyexl3/ref/hadamard.py:16-30 (stage h pairs i, i+h): inside
// the lane, then lanes 1, 2, 4, 8 apart through DPP operands, then 16 and 32 apart by
// swapping registers. No LDS traffic and no waits: a wave that has its activations
// starts decoding a few dozen instructions later.
__device__ __forceinline__ void wht128_lanes(float& a, float& b, int lane) {
    butterfly_in_lane(a, b);
    const uint32_t s0 = lane_sign_mask(lane, 0), s1 = lane_sign_mask(lane, 1),
                   s2 = lane_sign_mask(lane, 2), s3 = lane_sign_mask(lane, 3);
    a = butterfly_dpp<0>(a, s0);
    b = butterfly_dpp<0>(b, s0);
    a = butterfly_dpp<1>(a, s1);
    b = butterfly_dpp<1>(b, s1);
    a = butterfly_dpp<2>(a, s2);
    b = butterfly_dpp<2>(b, s2);
    a = butterfly_dpp<3>(a, s3);
    b = butterfly_dpp<3>(b, s3);
    swap_rows16(a, b);
    butterfly_in_lane(a, b);
    swap_halves32(a, b);
    butterfly_in_lane(a, b);
    swap_halves32(a, b);
    swap_rows16(a, b);
}

__device__ __forceinline__ float dot2(half2_t a, half2_t b, float c) {
    return __builtin_amdgcn_fdot2(a, b, c, false);
}

}  // namespace exl3
