// Shared pieces of the small-batch kernels (rows 1..8): the per-wave streaming
// loop that rotates or stages a 128-wide block of activations in LDS and runs
// the decode + dot pipeline over the block's 8 tile rows, and the 128-point
// Walsh-Hadamard butterfly on two values per lane.
#pragma once

#include "exl3_device.hpp"
#include "exl3_fixpoint.hpp"

namespace exl3 {

constexpr float kHadScaleF = 0.088388347648318440550f;  // 1/sqrt(128)

// Row stride (halfs) of a wave's staged activation block [MT][kXwLd]: the 128 values of
// a block, each stored twice in a row (x0, x0, x1, x1, ...: the matrix-pipe operand
// that meets the unsummed halves of the weights), plus 16 bytes, so that the four batch
// rows a quad of lanes reads with one ds_read_b128 start four LDS banks apart instead
// of in the same bank.
constexpr int kXwLd = 264;

// Activations of a tile row as the matrix pipe takes them, a quarter at a time: for each
// group of four batch rows, lane i of every quad reads batch row 4q+i; chunk c = input
// rows 4c..4c+3 of the tile row, each value twice (one ds_read_b128).
template <int MT>
struct XChunk {
    uint4_t v[(MT + 3) / 4];
};

// EXACT (weights rounded to fp16 before the product, see dot_tile_row_exact): the block is
// staged once per value and chunk c = input rows 8c..8c+7 of the tile row.
template <int MT, bool EXACT = false>
__device__ __forceinline__ XChunk<MT> load_x_chunk(half_t (*xw)[kXwLd], int row_in_block, int xlane,
                                                   int c) {
    constexpr int NQ = (MT + 3) / 4;
    XChunk<MT> t;
#pragma unroll
    for (int q = 0; q < NQ; q++) {
        int m = 4 * q + xlane;
        if (m > MT - 1) m = MT - 1;  // rows past the batch repeat a staged row; never used
        t.v[q] = *reinterpret_cast<const uint4_t*>(
            &xw[m][EXACT ? row_in_block * 16 + 8 * c : row_in_block * 32 + 8 * c]);
    }
    return t;
}

// The dot products of one tile row on the matrix pipe: v_mfma_f32_4x4x4_16b_f16
// multiplies, in each of its 16 independent blocks of 4 lanes, a 4x4 A (lane i of the
// block supplies row i) with a 4x4 B (lane j supplies column j) and leaves D[0..3][j] in
// lane j. A row i = activations of batch row 4q+i, B column j = two consecutive weights
// of lane j's own output column as their unsummed halves (lo, hi, lo', hi') against
// (a, a, a', a'): every lane gets the dot products of its weights with four batch rows,
// no data crosses lanes, and the VALU only extracts, multiplies and masks.
//
// Order of work: the sixteen codeword pairs of a lane are taken chunk by chunk of the
// activations (input rows 0-3, 8-11, 4-7, 12-15 of the tile row, both columns each), so
// that only two chunks are live at a time: the third and fourth are requested from LDS
// when the first and second have been used up. The matrix instruction of a pair is
// issued after the next pair has been decoded, so it never waits for the VALU result
// it reads.
template <int K, int CB, int MT, class LoadChunk>
__device__ __forceinline__ void dot_tile_row(const LaneWords<K>& lw, LoadChunk&& load_chunk,
                                             float4_t (&accv)[2][(MT + 3) / 4]) {
    constexpr int NQ = (MT + 3) / 4;
    // pair t: column select cs = (t >> 1) & 1 ... see pair_n below
    // t = 4*phase + 2*jj + cs with chunk(phase) = {0, 2, 1, 3}[phase], j = 2*chunk + jj
    auto pair_j = [](int t) constexpr { return 2 * ((t >> 2) == 0 ? 0 : (t >> 2) == 1 ? 2 : (t >> 2) == 2 ? 1 : 3) + ((t >> 1) & 1); };
    auto pair_cs = [](int t) constexpr { return t & 1; };
    // codewords n, n+1 hold input rows 2j, 2j+1 of column u + 8*cs (cw_row, cw_col_sel)
    auto pair_n = [](int j, int cs) constexpr { return 8 * (j & 3) + 4 * cs + 2 * (j >> 2); };
    XChunk<MT> xc[4];
    xc[0] = load_chunk(0);
    xc[2] = load_chunk(2);
    uint2_t wb[16];
    auto issue = [&](auto tc) {
        constexpr int t = tc.value;
        constexpr int j = pair_j(t), cs = pair_cs(t);
#pragma unroll
        for (int q = 0; q < NQ; q++) {
            const uint4_t xv = xc[j >> 1].v[q];
            const uint2_t xa = (j & 1) ? uint2_t{xv.z, xv.w} : uint2_t{xv.x, xv.y};
            accv[cs][q] = __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(half4_t, xa),
                                                           __builtin_bit_cast(half4_t, wb[t]),
                                                           accv[cs][q], 0, 0, 0);
        }
    };
    static_for<0, 16>([&](auto tc) {
        constexpr int t = tc.value;
        constexpr int n = pair_n(pair_j(t), pair_cs(t));
        static_assert(cw_col_sel(n) == pair_cs(t) && (cw_row(n) >> 1) == pair_j(t), "pair order");
        wb[t] = uint2_t{weight_halves<CB>(lane_codeword<K, n>(lw)),
                        weight_halves<CB>(lane_codeword<K, n + 1>(lw))};
        if constexpr (t >= 1) issue(std::integral_constant<int, t - 1>{});
        if constexpr (t == 4) xc[1] = load_chunk(1);   // chunk 0 has just been used up
        if constexpr (t == 8) xc[3] = load_chunk(3);   // chunk 2 likewise
    });
    issue(std::integral_constant<int, 15>{});
}

// The same with the weights as the reference defines them, rounded to fp16 (the half add
// of ponyexl3/ref/codebook.py:45-51) before they are multiplied: four weights per matrix
// instruction against four activations. 32 more VALU instructions per tile row than the
// unsummed form, whose products carry the exact sum of the two halves instead - a relative
// difference of up to 2^-11 per weight, 4-5e-4 rel-L2 on a layer's output. Chains of
// layers with a nonlinearity in between (the MoE experts) take this form for the
// projections in front of it.
template <int K, int CB, int MT, class LoadChunk>
__device__ __forceinline__ void dot_tile_row_exact(const LaneWords<K>& lw, LoadChunk&& load_chunk,
                                                   float4_t (&accv)[2][(MT + 3) / 4]) {
    constexpr int NQ = (MT + 3) / 4;
    const XChunk<MT> xc[2] = {load_chunk(0), load_chunk(1)};
    half2_t wp[16];
    decode_lane<K, CB>(lw, wp);
    // fresh-row groups outermost: consecutive MFMAs then write different accumulators
#pragma unroll
    for (int j4 = 0; j4 < 4; j4++) {  // input rows 4*j4 .. 4*j4+3 of the tile
#pragma unroll
        for (int q = 0; q < NQ; q++) {
            const uint4_t xv = xc[j4 >> 1].v[q];
            const uint2_t xa = (j4 & 1) ? uint2_t{xv.z, xv.w} : uint2_t{xv.x, xv.y};
#pragma unroll
            for (int cs = 0; cs < 2; cs++) {
                const uint2_t wb = {half2_to_bits(wp[8 * cs + 2 * j4]),
                                    half2_to_bits(wp[8 * cs + 2 * j4 + 1])};
                accv[cs][q] = __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(half4_t, xa),
                                                               __builtin_bit_cast(half4_t, wb),
                                                               accv[cs][q], 0, 0, 0);
            }
        }
    }
}

template <int K>
__device__ __forceinline__ void load_lane_words_nt(const uint32_t* __restrict__ p,
                                                   uint32_t (&own)[K]) {
#pragma unroll
    for (int i = 0; i < K; i++) own[i] = __builtin_nontemporal_load(p + i);
}

// The same through a pointer that is declared to be in global memory (for addresses
// whose origin the compiler cannot see; it would otherwise emit flat loads).
using global_words_t = const uint32_t __attribute__((address_space(1)))*;

template <int K>
__device__ __forceinline__ void load_lane_words_nt(global_words_t p, uint32_t (&own)[K]) {
#pragma unroll
    for (int i = 0; i < K; i++) own[i] = __builtin_nontemporal_load(p + i);
}

// One wave streams tile rows [tk_begin, tk_end) (both multiples of 8, non-empty)
// of the 8 tile columns that start at `base` (already offset by lane*K dwords)
// and accumulates acc[m][0..1] += x[m][rows of the tile] . W[:, column u / u+8].
//
// Activations enter through the wave's own LDS slot xw[MT][kXwLd], one 128-wide
// block (8 tile rows) at a time:
//   ROTATE  xw = fp16(had128(x * suh) / sqrt(128))   (ponyexl3/ref/forward.py:32-34)
//   else    xw = x                                   (x is already rotated)
// The raw block after the current one is in flight while the current one is
// used; a tile row's 16 activations come back with two broadcast ds_read_b128.
// kSlots wave-wide trellis loads are kept in flight.
//
// HALF: the range is one half of a block, [tk_begin, tk_begin + 4) with tk_begin a
// multiple of 4. The wave still rotates (or stages) the whole 128-wide block, then
// uses four of its eight tile rows. Narrow layers get twice the waves this way.
//
// The batch rows are given by address (xrow[m], m < MT; entries past `rows` repeat a
// valid row), so that a caller can gather them. GUARD: rows past `rows` are neither
// loaded nor rotated (their LDS rows and sums are then meaningless and must not be
// used). PRELOADED: the caller has already issued the first trellis loads into `buf`
// with issue_first_rows (to overlap their latency with work of its own).
constexpr int kStreamSlots = 4;  // wave-wide loads in flight (divides the 8 steps of a block)

template <int K, bool HALF, class Words>
__device__ __forceinline__ void issue_first_rows(Words base, size_t row_words, int tk_begin,
                                                 int tk_end, uint32_t (&buf)[kStreamSlots][K]) {
#pragma unroll
    for (int s = 0; s < kStreamSlots; s++) {
        const int tk = HALF ? tk_begin + s : min(tk_begin + s, tk_end - 1);
        load_lane_words_nt<K>(base + (size_t)tk * row_words, buf[s]);
    }
}

template <int K, int CB, int MT, bool ROTATE, bool HALF, bool GUARD, bool PRELOADED,
          bool EXACT = false>
__device__ __forceinline__ void stream_block_rows_at(const uint32_t* __restrict__ base,
                                                     size_t row_words, int tk_begin, int tk_end,
                                                     const half_t* const (&xrow)[MT], int rows,
                                                     const half_t* __restrict__ suh_row,
                                                     half_t (*xw)[kXwLd], int lane,
                                                     float (&acc)[MT][2],
                                                     uint32_t (&buf)[kStreamSlots][K]) {
    half2_t xraw[MT], sraw;
    auto fetch_block = [&](int blk) {
        const int off = blk * 128 + 2 * lane;
#pragma unroll
        for (int m = 0; m < MT; m++) {
            if (GUARD && m >= rows) break;
            xraw[m] = *reinterpret_cast<const half2_t*>(xrow[m] + off);
        }
        if (ROTATE && suh_row) sraw = *reinterpret_cast<const half2_t*>(suh_row + off);
    };
    auto stage_block = [&]() {
#pragma unroll
        for (int m = 0; m < MT; m++) {
            if (GUARD && m >= rows) break;
            half2_t o = xraw[m];
            if constexpr (ROTATE) {
                float a = (float)xraw[m].x, b = (float)xraw[m].y;
                if (suh_row) {
                    a = __fmul_rn(a, (float)sraw.x);
                    b = __fmul_rn(b, (float)sraw.y);
                }
                wht128_lanes(a, b, lane);
                o.x = (half_t)__fmul_rn(a, kHadScaleF);
                o.y = (half_t)__fmul_rn(b, kHadScaleF);
            }
            if constexpr (EXACT) {
                *reinterpret_cast<half2_t*>(&xw[m][2 * lane]) = o;
            } else {
                const uint32_t lo = half_to_bits(o.x), hi = half_to_bits(o.y);
                *reinterpret_cast<uint2_t*>(&xw[m][4 * lane]) =
                    uint2_t{lo | (lo << 16), hi | (hi << 16)};
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    };
    constexpr int NQ = (MT + 3) / 4;  // groups of four batch rows
    float4_t accv[2][NQ];
#pragma unroll
    for (int cs = 0; cs < 2; cs++)
#pragma unroll
        for (int q = 0; q < NQ; q++) accv[cs][q] = float4_t{0.f, 0.f, 0.f, 0.f};
    const int xlane = lane & 3;
    auto consume = [&](const uint32_t (&words)[K], uint32_t prev, int row_in_block) {
        auto chunk = [&](int c) { return load_x_chunk<MT, EXACT>(xw, row_in_block, xlane, c); };
        if constexpr (EXACT)
            dot_tile_row_exact<K, CB, MT>(make_lane_words<K>(prev, words), chunk, accv);
        else
            dot_tile_row<K, CB, MT>(make_lane_words<K>(prev, words), chunk, accv);
    };
    auto add_up = [&]() {
#pragma unroll
        for (int m = 0; m < MT; m++) {
            acc[m][0] += accv[0][m >> 2][m & 3];
            acc[m][1] += accv[1][m >> 2][m & 3];
        }
    };
    constexpr int kSlots = kStreamSlots;
    // The activations are requested before the trellis rows: loads return in issue
    // order, so the rotation then only waits for the activations and the decode of the
    // first row only for that row, not for all kSlots rows.
    fetch_block(tk_begin >> 3);
    if constexpr (!PRELOADED) issue_first_rows<K, HALF>(base, row_words, tk_begin, tk_end, buf);
    __builtin_amdgcn_sched_barrier(0);  // all of them in flight before the rotation starts
    if constexpr (HALF) {
        // all four loads up front, no refills
        stage_block();
        const int row0 = tk_begin & 7;  // 0 or 4
        uint32_t prev = neighbour_word(buf[0][K - 1], lane);
#pragma unroll
        for (int s = 0; s < kSlots; s++) {
            const uint32_t prev_next =
                s + 1 < kSlots ? neighbour_word(buf[s + 1][K - 1], lane) : 0u;
            __builtin_amdgcn_sched_barrier(0);
            consume(buf[s], prev, row0 + s);
            __builtin_amdgcn_sched_barrier(0);
            prev = prev_next;
        }
        add_up();
        return;
    }
    // Ranges are whole blocks, so the staging sits outside the unrolled 8-step
    // pipeline and the LDS offsets of the activations are compile-time constants.
    // (the first block is staged before anything touches the trellis rows)
    stage_block();
    uint32_t prev = neighbour_word(buf[0][K - 1], lane);
    int tkb = tk_begin;
    do {  // the range is not empty (no loop guard for loads to sink behind)
        if (tkb != tk_begin) stage_block();
        if (tkb + 8 < tk_end) fetch_block((tkb >> 3) + 1);
#pragma unroll
        for (int s8 = 0; s8 < 8; s8++) {
            const int tk = tkb + s8;
            const int slot = s8 & (kSlots - 1);
            const uint32_t prev_next = neighbour_word(buf[(slot + 1) & (kSlots - 1)][K - 1], lane);
            __builtin_amdgcn_sched_barrier(0);
            consume(buf[slot], prev, s8);
            const int tn = min(tk + kSlots, tk_end - 1);
            load_lane_words_nt<K>(base + (size_t)tn * row_words, buf[slot]);
            __builtin_amdgcn_sched_barrier(0);
            prev = prev_next;
        }
        tkb += 8;
    } while (tkb < tk_end);
    add_up();
}

// The same over `rows` consecutive rows of a row-major activation matrix.
template <int K, int CB, int MT, bool ROTATE, bool HALF = false, bool EXACT = false>
__device__ __forceinline__ void stream_block_rows(const uint32_t* __restrict__ base,
                                                  size_t row_words, int tk_begin, int tk_end,
                                                  const half_t* __restrict__ x, size_t x_stride,
                                                  int rows, const half_t* __restrict__ suh_row,
                                                  half_t (*xw)[kXwLd], int lane,
                                                  float (&acc)[MT][2]) {
    const half_t* xrow[MT];
#pragma unroll
    for (int m = 0; m < MT; m++) xrow[m] = x + (size_t)(m < rows ? m : 0) * x_stride;
    uint32_t buf[kStreamSlots][K];
    stream_block_rows_at<K, CB, MT, ROTATE, HALF, false, false, EXACT>(
        base, row_words, tk_begin, tk_end, xrow, rows, suh_row, xw, lane, acc, buf);
}

}  // namespace exl3
