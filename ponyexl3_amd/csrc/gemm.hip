// Prefill GEMM: y = xh @ W_inner with the trellis decoded into LDS and
// contracted on fp16 MFMA (v_mfma_f32_16x16x32_f16), fp32 accumulation.
//
// One workgroup = 8 wavefronts (2 per SIMD), one workgroup per CU.
//   block tile   BM x 256 columns, BK = 64 (four tile rows); BM = 256 (MI = 8),
//                128 (MI = 4) or 64 (MI = 2) for small batches: less padding
//                work per decoded tile
//   wave tile    (BM/2) x 64 -> MI x 4 accumulator tiles of 16x16
//   LDS          two stages of A [BM][64] and B [256][64] fp16 (128 KiB at MI = 8):
//                stage s^1 is filled while stage s is contracted, one barrier per
//                64-deep step
//   B fill       wave w decodes tile row (w & 3) of the 8 tile columns of half
//                (w >> 2): one 256*K-byte wave-wide load, 32 codewords per lane
//   A fill       global -> LDS direct loads (global_load_lds_dwordx4): lane l of a
//                wave-wide load lands at byte 16*l of a 1 KiB block = 8 rows of 64
//                halfs, so no VGPRs and no ds_write are spent on activations
// LDS rows are 64 halfs (128 B) unpadded; the 16-byte chunk c of row r is stored
// at chunk c ^ (((r >> 1) & 3) << 1). Measured on gfx950 this makes the b128
// fragment reads (16 rows x 4 chunks per wave) run at the same ~190 B/clk/CU as a
// padded layout while keeping each 8-row block contiguous for the direct loads.
//
// Decode work is spread over the MFMA stream: after each group of 8 MFMAs a wave
// decodes 32/MI codewords, which the hardware issues in the shadow of the matrix
// pipe (about two VALU instructions per MFMA are free).
//
// The MFMA is issued as D^T = B^T A^T (weights as the first operand), so a lane
// ends up with 4 consecutive output columns of one row.
//
// Tail handling: tiles are dealt to CUs in rounds. The tiles of a last, partly
// filled round are not given a CU each but cut along the reduction into runs of
// 64-deep steps, one workgroup per run; the planner takes the cheaper of two
// shapes: s runs per tile (in as many rounds as rem*s runs need), or the tiles'
// steps laid end to end and cut into equal runs, one per CU, so that the round
// costs rem/CUs of a tile time - a run that crosses a tile border then works on
// two tiles one after the other (kernel instantiation TWO). Every piece writes an
// fp32 partial tile to a workspace and a small second kernel adds the pieces of
// each tile in run order and rounds once to fp16.
//
// Replaces the rows > 16 ladder of EXL3Linear.__call__
// (ponyexl3/mlx/exl3_linear.py:137-161) and the decode-into-threadgroup-memory
// GEMM of ponyexl3/mlx/gemv_metal.py:1518-1741.
#include "exl3_device.hpp"
#include "exl3_host.hpp"

namespace exl3 {

constexpr int kGemmBN = 256;       // columns per block tile
constexpr int kGemmThreads = 512;  // 8 waves
constexpr int kGemmStageB = kGemmBN * 64;

__device__ __forceinline__ int lds_chunk_swizzle(int row) { return ((row >> 1) & 3) << 1; }

// One piece of work: a whole tile (partial_slot < 0, direct fp16 output) or a range
// of a split tile's steps whose fp32 partial tile goes to slot `partial_slot`.
struct GemmWork {
    int tile, k_begin, k_end, partial_slot;
};

// The split region: every tile's `ksteps` steps sit at the start of a stretch of
// `pitch` >= ksteps positions, the stretches end to end, cut into runs of `per`
// positions (per <= pitch, so a run touches at most two tiles; the planner never
// makes a run that starts in the unused end of a stretch). Two shapes are used:
// pitch = ksteps, runs of any length that cross tile borders (as many runs as CUs,
// all equally long), and pitch = s * per, s runs per tile that never cross.
// Piece `si` (0 or 1) of run v covers tile j = first tile of the run + si; its
// partial tile is slot v + j, which numbers the pieces in run order (slots < runs +
// tiles). The pieces of tile j are those of runs first_run(j) .. last_run(j).
// (tiles * pitch < 2^31: the planner does not split otherwise)
__host__ __device__ __forceinline__ int split_first_run(int j, int pitch, int per) {
    return (j * pitch) / per;
}
__host__ __device__ __forceinline__ int split_last_run(int j, int pitch, int ksteps, int per) {
    return (j * pitch + ksteps - 1) / per;
}

// Workgroups are handed to the eight XCDs round-robin by index, and each XCD has
// its own L2. Whole tiles are numbered column block first (tile = g * n_row_blocks
// + row block), so consecutive indices would spread the row blocks of one column
// block -- which all decode the same trellis columns -- over all eight L2s. For the
// part of the schedule that holds complete sets of eight column blocks, workgroup b
// therefore takes column block 8*(q / n_row_blocks) + b % 8, row block q %
// n_row_blocks with q = b / 8: a column block stays on one XCD.
__device__ __forceinline__ int xcd_tile_order(int b, int full_tiles, int n_row_blocks) {
    const int set = 8 * n_row_blocks;
    const int whole = full_tiles / set * set;
    if (b >= whole) return b;
    const int q = b >> 3;
    const int g = (q / n_row_blocks) * 8 + (b & 7);
    return g * n_row_blocks + q % n_row_blocks;
}

// Split geometry as the kernel gets it.
struct GemmSplit {
    int per, pitch, runs_per_tile;  // runs_per_tile > 0: runs never cross tiles
    int positions;                  // tiles * pitch
};

// Number of pieces of workgroup `unit` and piece `si` of it.
__device__ __forceinline__ int gemm_pieces(int unit, int full_tiles, const GemmSplit& sp) {
    if (unit < full_tiles) return 1;
    const int p0 = (unit - full_tiles) * sp.per;
    const int p1 = min(p0 + sp.per, sp.positions);
    return p1 - 1 >= (p0 / sp.pitch + 1) * sp.pitch ? 2 : 1;
}

__device__ __forceinline__ GemmWork gemm_work(int unit, int si, int full_tiles, int ksteps,
                                              const GemmSplit& sp, int n_row_blocks,
                                              int split_units) {
    GemmWork w;
    if (unit < full_tiles) {
        w.tile = xcd_tile_order(unit, full_tiles, n_row_blocks);
        w.k_begin = 0;
        w.k_end = ksteps;
        w.partial_slot = -1;
    } else {
        int v = unit - full_tiles;
        if (sp.runs_per_tile > 0 && full_tiles % n_row_blocks == 0) {
            // The runs that share trellis data are the row blocks of one (column block,
            // range) pair. Those pairs are numbered gv = column block * runs_per_tile +
            // range, workgroups u = gv * n_row_blocks + row block, and u is dealt to the
            // XCDs like the whole tiles above.
            const int s = sp.runs_per_tile;
            const int u = xcd_tile_order(v, split_units, n_row_blocks);
            const int gv = u / n_row_blocks, rb = u % n_row_blocks;
            v = ((gv / s) * n_row_blocks + rb) * s + gv % s;
        }
        const int p0 = v * sp.per;
        const int p1 = min(p0 + sp.per, sp.positions);
        const int j = p0 / sp.pitch + si;
        const int t0 = j * sp.pitch;
        w.tile = full_tiles + j;
        w.k_begin = si ? 0 : p0 - t0;
        w.k_end = min(p1 - t0, ksteps);
        w.partial_slot = v + j;
    }
    return w;
}

// The kernel's arguments, as one block at the start of its argument segment.
struct GemmArgs {
    const uint32_t* trellis;
    const half_t* xh;
    half_t* y;
    float* partial;
    int rows;
    size_t ldx, ldy;
    int in_tiles, out_tiles, tn_offset, tn_count, n_row_blocks, full_tiles;
    GemmSplit split;
    const int4* group_tab;
    int group_tiles, n_groups;
    const int* block_sub;
    size_t sub_stride;
    const half_t* post_svh;
    const half_t* post_bias;
    half_t* post_out;
    size_t ldo;
};

// TWO: the launch has runs that cross tile borders, i.e. workgroups with two pieces.
template <int K, int CB, int MI, bool TWO>
__global__ __launch_bounds__(kGemmThreads, 1) void gemm_kernel(GemmArgs by_value) {
    extern __shared__ __attribute__((aligned(16))) half_t smem[];
    constexpr int BM = 32 * MI;
    constexpr int STAGE_A = BM * 64, STAGE_B = kGemmStageB;
    half_t* a_s = smem;
    half_t* b_s = smem + 2 * STAGE_A;

    // Plain mode: workgroup -> (column block g, row block) of one matrix, whole, or
    // one or two pieces of split tiles. Grouped mode (group_tab != NULL): the rows are
    // sorted into groups (experts) that each multiply their own `group_tiles` tile
    // columns; group_tab[b] = {group, first row, end row} of row block b (first ==
    // end marks an unused entry), blockIdx.x = b * n_col_blocks + g, whole reduction.
    //
    // A workgroup with two pieces reads its arguments again for the second one, from
    // the argument segment through a pointer the compiler cannot see through: kept in
    // registers across the first piece's main loop they would cost more scalar
    // registers than there are, and the spills would land in the loop.
    const GemmArgs __attribute__((address_space(4)))* args =
        (const GemmArgs __attribute__((address_space(4)))*)__builtin_amdgcn_kernarg_segment_ptr();
    (void)by_value;
    int n_pieces = 1;
    if constexpr (TWO) {
        const GemmArgs __attribute__((address_space(4)))* a0 = args;
        asm volatile("" : "+s"(a0));
        const GemmSplit split = {a0->split.per, a0->split.pitch, a0->split.runs_per_tile,
                                 a0->split.positions};
        n_pieces = a0->group_tab ? 1 : gemm_pieces(blockIdx.x, a0->full_tiles, split);
    }
    for (int piece = 0; piece < n_pieces; piece++) {
    const GemmArgs __attribute__((address_space(4)))* ap = args;
    if constexpr (TWO) asm volatile("" : "+s"(ap));
    const uint32_t* __restrict__ trellis = ap->trellis;
    const half_t* __restrict__ xh = ap->xh;
    half_t* __restrict__ y = ap->y;
    float* __restrict__ partial = ap->partial;
    const int rows_arg = ap->rows;
    const size_t ldx = ap->ldx, ldy = ap->ldy;
    const int in_tiles = ap->in_tiles, out_tiles = ap->out_tiles;
    const int tn_offset_arg = ap->tn_offset, tn_count_arg = ap->tn_count;
    const int n_row_blocks = ap->n_row_blocks, full_tiles = ap->full_tiles;
    const int4* __restrict__ group_tab = ap->group_tab;
    const int group_tiles = ap->group_tiles, n_groups = ap->n_groups;
    const int* __restrict__ block_sub = ap->block_sub;
    const size_t sub_stride = ap->sub_stride;
    const half_t* __restrict__ post_svh = ap->post_svh;
    const half_t* __restrict__ post_bias = ap->post_bias;
    half_t* __restrict__ post_out = ap->post_out;
    const size_t ldo = ap->ldo;
    // (the lane's indices, too, are derived anew for every piece)
    int tid = threadIdx.x;
    if constexpr (TWO) asm volatile("" : "+v"(tid));
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 2, wn = wave & 3;  // wave tile origin: rows wm*16*MI, columns wn*64
    GemmWork work;
    int g, m0, rows, tn_offset, tn_count;
    const half_t* xh_t = xh;
    if (group_tab) {
        const int n_col_blocks = (group_tiles + 15) >> 4;
        int4 t = group_tab[blockIdx.x / n_col_blocks];
        // the table is caller memory: a group outside the trellis slice or a row range
        // outside xh / y would fault, so such entries are dropped / clamped
        if (t.z > rows_arg) t.z = rows_arg;
        if (t.x < 0 || t.x >= n_groups || t.y < 0 || t.y >= t.z) return;  // whole workgroup, before any barrier
        work.tile = 0;
        work.k_begin = 0;
        work.k_end = in_tiles / 4;
        work.partial_slot = -1;
        g = blockIdx.x % n_col_blocks;
        m0 = t.y;
        rows = t.z;
        tn_offset = tn_offset_arg + t.x * group_tiles;
        tn_count = group_tiles;
    } else {
        const GemmSplit split = {ap->split.per, ap->split.pitch, ap->split.runs_per_tile,
                                 ap->split.positions};
        work = gemm_work(blockIdx.x, piece, full_tiles, in_tiles / 4, split, n_row_blocks,
                         (int)gridDim.x - full_tiles);
        g = work.tile / n_row_blocks;  // 256-column block inside the slice
        m0 = (work.tile % n_row_blocks) * BM;
        rows = rows_arg;
        tn_offset = tn_offset_arg;
        tn_count = tn_count_arg;
        // sibling-fused layers: every 256-column block multiplies the activations that
        // were rotated with its own member's suh, xh[row][block_sub[g]][:]
        if (block_sub) xh_t += (size_t)block_sub[g] * sub_stride;
    }
    const int k_begin = work.k_begin, k_last = work.k_end - 1;
    const int nsteps = work.k_end - work.k_begin;

    // ---- fill side: what this wave brings into LDS every step ----
    const int tr = wave & 3;
    // the last column block of a slice may hold only 8 tile columns: its upper half
    // re-decodes the lower half's tiles (results never stored)
    const int ch = (g * 16 + 8 < tn_count) ? (wave >> 2) : 0;
    const size_t row_words = (size_t)out_tiles * (8 * K);
    const uint32_t* tbase = trellis + (size_t)(tn_offset + g * 16 + ch * 8) * (8 * K) +
                            (size_t)tr * row_words + lane * K;
    const size_t t_step = 4 * row_words;
    int b_w[2];  // half offsets of the lane's two columns inside a B stage (chunk 2*tr)
#pragma unroll
    for (int cs = 0; cs < 2; cs++) {
        const int n = (wave >> 2) * 128 + (lane >> 3) * 16 + (lane & 7) + 8 * cs;
        b_w[cs] = n * 64 + ((2 * tr) ^ lds_chunk_swizzle(n)) * 8;
    }
    // A tile: wave w copies rows w*4*MI .. +4*MI-1 with MI/2 direct loads of 8 rows each
    const char* abase = reinterpret_cast<const char*>(xh_t + (size_t)m0 * ldx);
    uint32_t a_off[MI / 2];
    {
        const int rl = lane >> 3;
        const int c = (lane & 7) ^ lds_chunk_swizzle(rl);
#pragma unroll
        for (int i = 0; i < MI / 2; i++) {
            int r = wave * (4 * MI) + i * 8 + rl;
            if (m0 + r >= rows) r = rows - 1 - m0;  // rows past the end are never stored
            a_off[i] = (uint32_t)((size_t)r * ldx * 2 + c * 16);
        }
    }
    uint32_t w_reg[2][K];

    auto load_w = [&](int kstep, auto slot) {
        constexpr int s = decltype(slot)::value;
        const uint32_t* p = tbase + (size_t)kstep * t_step;
#pragma unroll
        for (int i = 0; i < K; i++) w_reg[s][i] = __builtin_nontemporal_load(p + i);
    };
    auto load_a = [&](int kstep, int stage) {
        const char* ab = abase + (size_t)kstep * 128;
        half_t* as = a_s + stage * STAGE_A + wave * (4 * MI) * 64;
#pragma unroll
        for (int i = 0; i < MI / 2; i++)
            __builtin_amdgcn_global_load_lds(
                (const void __attribute__((address_space(1)))*)(ab + a_off[i]),
                (void __attribute__((address_space(3)))*)(as + i * 8 * 64), 16, 0, 0);
    };
    // Pair pi (0..15) of a lane = codewords 2pi, 2pi+1 = input rows (2j, 2j+1) of
    // column u + 8*cs with cs = (pi>>1)&1, j = (pi>>2) + 4*(pi&1). The four pairs
    // {2cs + hh + 4t, t = 0..3} are the 8 consecutive rows 8hh..8hh+7 of column cs:
    // one 16-byte store. Element e = 4*quad + t of the decode order; two elements
    // are decoded per call (see add_halves_pack2 for why).
    auto decode_element2 = [&](const LaneWords<K>& lw, auto e_c, uint4_t& quad, half_t* bdst) {
        constexpr int e = decltype(e_c)::value;  // even: elements e and e + 1
        constexpr int q = e >> 2, t = e & 3;
        constexpr int cs = q >> 1, hh = q & 1;
        constexpr int pa = 2 * cs + hh + 4 * t, pb = pa + 4;
        half2_t da, db;
        decode_pair2<CB>(lane_codeword<K, 2 * pa>(lw), lane_codeword<K, 2 * pa + 1>(lw),
                         lane_codeword<K, 2 * pb>(lw), lane_codeword<K, 2 * pb + 1>(lw), da, db);
        if constexpr (t == 0) {
            quad.x = half2_to_bits(da);
            quad.y = half2_to_bits(db);
        } else {
            quad.z = half2_to_bits(da);
            quad.w = half2_to_bits(db);
            *reinterpret_cast<uint4_t*>(bdst + b_w[cs] + 8 * hh) = quad;
        }
    };

    // ---- MFMA side ----
    float4_t acc[MI][4];
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = float4_t{0.f, 0.f, 0.f, 0.f};
    const int fr = lane & 15;
    // half offset of the lane's 16-byte chunk for the first 32 k; the second 32 k flip chunk bit 2
    const int pk0 = ((lane >> 4) ^ lds_chunk_swizzle(fr)) * 8;
    const half_t* a_frag = a_s + (wm * (16 * MI) + fr) * 64;
    const half_t* b_frag = b_s + (wn * 64 + fr) * 64;

    using S0 = std::integral_constant<int, 0>;
    using S1 = std::integral_constant<int, 1>;
    auto clamp_k = [&](int k) { return k < k_last ? k : k_last; };

    // prologue: stage 0 <- step 0; slot 1 <- step 1, slot 0 <- step 2
    {
        load_w(k_begin, S0{});
        load_a(k_begin, 0);
        load_w(clamp_k(k_begin + 1), S1{});
        const LaneWords<K> lw = finish_lane_words<K>(w_reg[0], lane);
        uint4_t quad;
        static_for<0, 8>([&](auto e2) {
            decode_element2(lw, std::integral_constant<int, 2 * decltype(e2)::value>{}, quad, b_s);
        });
        load_w(clamp_k(k_begin + 2), S0{});
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();

    // Step i contracts stage i&1 and fills stage (i+1)&1 with step i+1, whose
    // trellis words sit in slot (i+1)&1; that slot is then refilled with step i+3.
    auto step = [&](int i, auto slot) {
        constexpr int s = decltype(slot)::value;
        const int stage = i & 1;
        const int k = k_begin + i;
        const half_t* as = a_frag + stage * STAGE_A;
        const half_t* bs = b_frag + stage * STAGE_B;
        half_t* bdst = b_s + (stage ^ 1) * STAGE_B;
        uint4_t quad;
        half8_t bf[4];
        half8_t af[3][2];
        auto lda = [&](int kk, int ii) {
            return *reinterpret_cast<const half8_t*>(as + ii * 16 * 64 + (pk0 ^ (kk * 32)));
        };
        auto ldb = [&](int kk, int j) {
            return *reinterpret_cast<const half8_t*>(bs + j * 16 * 64 + (pk0 ^ (kk * 32)));
        };
        // MFMA group gi = 8 MFMAs = two 16-row tiles x four 16-column tiles x 32 k;
        // MI groups per step, A fragments are requested two groups ahead.
        constexpr int G = MI;
        constexpr int GH = MI / 2;  // groups per 32-deep half
        constexpr int EPG = 16 / G;  // decode elements per group
        auto lda_group = [&](auto gi_c) {
            constexpr int gi = decltype(gi_c)::value;
            af[gi % 3][0] = lda(gi / GH, 2 * (gi % GH));
            af[gi % 3][1] = lda(gi / GH, 2 * (gi % GH) + 1);
        };
        // The first fragments are requested right after the barrier; the fills of the
        // other stage and the first slice of decode work are issued while they fly.
#pragma unroll
        for (int j = 0; j < 4; j++) bf[j] = ldb(0, j);
        lda_group(std::integral_constant<int, 0>{});
        lda_group(std::integral_constant<int, 1>{});
        __builtin_amdgcn_sched_barrier(0);
        load_a(clamp_k(k + 1), stage ^ 1);
        const LaneWords<K> lw = finish_lane_words<K>(w_reg[s], lane);
        __builtin_amdgcn_sched_barrier(0);  // keeps the trellis load behind the direct loads
        load_w(clamp_k(k + 3), slot);
        static_for<0, EPG / 2>([&](auto e2) {
            decode_element2(lw, std::integral_constant<int, 2 * decltype(e2)::value>{}, quad, bdst);
        });
        __builtin_amdgcn_sched_barrier(0);
        static_for<0, G>([&](auto gi_c) {
            constexpr int gi = decltype(gi_c)::value;
            constexpr int ip = gi % GH;
            if constexpr (gi + 2 < G) lda_group(std::integral_constant<int, gi + 2>{});
#pragma unroll
            for (int h = 0; h < 2; h++)
#pragma unroll
                for (int j = 0; j < 4; j++)
                    acc[2 * ip + h][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                        bf[j], af[gi % 3][h], acc[2 * ip + h][j], 0, 0, 0);
            if constexpr (gi == GH - 1) {  // weights of the second half, once the first half is issued
#pragma unroll
                for (int j = 0; j < 4; j++) bf[j] = ldb(1, j);
            }
            if constexpr (gi + 1 < G)
                static_for<(gi + 1) * EPG / 2, (gi + 2) * EPG / 2>([&](auto e2) {
                    decode_element2(lw, std::integral_constant<int, 2 * decltype(e2)::value>{},
                                    quad, bdst);
                });
            __builtin_amdgcn_sched_barrier(0);
        });
        // Memory operations retire in order and at least one trellis load was issued
        // after the direct loads of stage^1: with at most one load outstanding those
        // have landed, and the trellis prefetch may stay in flight across the barrier.
        asm volatile("s_waitcnt vmcnt(1)" ::: "memory");
        __syncthreads();
    };

    int i = 0;
    for (; i + 1 < nsteps; i += 2) {
        step(i, S1{});
        step(i + 1, S0{});
    }
    if (i < nsteps) step(i, S1{});

    // acc[i][j] is D^T: lane holds columns 4*(lane/16)+0..3 of row lane%16
    const int col0 = g * kGemmBN + wn * 64 + (lane >> 4) * 4;
    if (post_out && work.partial_slot < 0) {
        // Output transform of a whole tile inside the kernel (ponyexl3/ref/forward.py:41-45):
        // y16 = fp16(acc) goes to LDS, then Z = Y16 x H128 per 128-column block runs on the
        // matrix pipe as well - 128 more MFMAs per wave next to the 64 of every k-step, instead
        // of a pass that reads and writes all of y again. H is symmetric with entries +-1,
        // exact in fp16, so the products are exact and the sums are fp32 as in the butterfly
        // form (another order of additions: the fp16 result can differ from the separate pass
        // in its last bit). The fragments of H come from four register sets per lane: entry
        // (k, n) has sign parity(k & n); with n = 16 nt + fr and k = 32 ks + 8 q + t the parity
        // splits into a part the lane knows (fr, q, t), a part that needs nt & 1 and a part
        // that is the same for every lane of the instruction (nt >> 1 and ks, compile time).
        constexpr int kYLd = kGemmBN + 8;  // row stride in halfs: 16-byte reads of 16 rows hit 64 banks
        half_t* ys = smem;
        const int q = lane >> 4;
#pragma unroll
        for (int ii = 0; ii < MI; ii++) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                half4_t o;
                o.x = (half_t)acc[ii][j].x;
                o.y = (half_t)acc[ii][j].y;
                o.z = (half_t)acc[ii][j].z;
                o.w = (half_t)acc[ii][j].w;
                *reinterpret_cast<half4_t*>(ys + (wm * (16 * MI) + ii * 16 + fr) * kYLd + wn * 64 +
                                            j * 16 + q * 4) = o;
            }
        }
        uint32_t hsign[2][2][4];  // [nt & 1][uniform flip][pair of k-slots]
        {
            const uint32_t lane_flip0 = ((fr >> 3) & q & 1) ? 0x80008000u : 0u;
            const uint32_t lane_flip1 = lane_flip0 ^ ((q >> 1) ? 0x80008000u : 0u);
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t lo = __builtin_popcount(fr & 7 & (2 * i)) & 1;
                const uint32_t hi = __builtin_popcount(fr & 7 & (2 * i + 1)) & 1;
                const uint32_t base = 0x3C003C00u | (lo << 15) | (hi << 31);
                hsign[0][0][i] = base ^ lane_flip0;
                hsign[0][1][i] = base ^ lane_flip0 ^ 0x80008000u;
                hsign[1][0][i] = base ^ lane_flip1;
                hsign[1][1][i] = base ^ lane_flip1 ^ 0x80008000u;
            }
        }
        __syncthreads();
        constexpr int U = MI / 2;  // (16-row tile, 128-column block) units per wave
        static_for<0, U>([&](auto ui) {
            const int u = wave * U + ui.value;
            const int rt = u >> 1, blk = u & 1;
            float4_t z[8];
#pragma unroll
            for (int nt = 0; nt < 8; nt++) z[nt] = float4_t{0.f, 0.f, 0.f, 0.f};
            const half_t* yrow = ys + (rt * 16 + fr) * kYLd + blk * 128 + q * 8;
            static_for<0, 4>([&](auto ks) {
                const half8_t yf = *reinterpret_cast<const half8_t*>(yrow + ks.value * 32);
                static_for<0, 8>([&](auto nt) {
                    constexpr int uni = ((nt.value >> 1) & ks.value & 1) ^
                                        ((nt.value >> 2) & (ks.value >> 1) & 1);
                    const uint4_t hv = {hsign[nt.value & 1][uni][0], hsign[nt.value & 1][uni][1],
                                        hsign[nt.value & 1][uni][2], hsign[nt.value & 1][uni][3]};
                    z[nt.value] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                        __builtin_bit_cast(half8_t, hv), yf, z[nt.value], 0, 0, 0);
                });
            });
            const int r = m0 + rt * 16 + fr;
            const int cb0 = g * kGemmBN + blk * 128 + q * 4;
            if (r < rows && cb0 < tn_count * 16) {  // (a half-width last block has no second block)
#pragma unroll
                for (int nt = 0; nt < 8; nt++) {
                    const int col = cb0 + nt * 16;
                    float v[4] = {z[nt].x, z[nt].y, z[nt].z, z[nt].w};
                    half4_t sv, bv;
                    if (post_svh) sv = *reinterpret_cast<const half4_t*>(post_svh + col);
                    if (post_bias) bv = *reinterpret_cast<const half4_t*>(post_bias + col);
                    half4_t o;
#pragma unroll
                    for (int c = 0; c < 4; c++) {
                        float a = __fmul_rn(v[c], 0.088388347648318440550f);  // 1/sqrt(128)
                        if (post_svh) a = __fmul_rn(a, (float)sv[c]);
                        half_t h = (half_t)a;
                        if (post_bias) h = h + bv[c];
                        o[c] = h;
                    }
                    *reinterpret_cast<half4_t*>(post_out + (size_t)r * ldo + col) = o;
                }
            }
        });
        return;  // a whole tile is a workgroup's only piece
    }
    if (g * kGemmBN + wn * 64 >= tn_count * 16) continue;  // upper half of a half-width last block
    if (work.partial_slot < 0) {
#pragma unroll
        for (int ii = 0; ii < MI; ii++) {
            const int r = m0 + wm * (16 * MI) + ii * 16 + fr;
            if (r < rows) {
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    half4_t o;
                    o.x = (half_t)acc[ii][j].x;
                    o.y = (half_t)acc[ii][j].y;
                    o.z = (half_t)acc[ii][j].z;
                    o.w = (half_t)acc[ii][j].w;
                    *reinterpret_cast<half4_t*>(y + (size_t)r * ldy + col0 + j * 16) = o;
                }
            }
        }
    } else {
        float* pt = partial + (size_t)work.partial_slot * (BM * kGemmBN);
#pragma unroll
        for (int ii = 0; ii < MI; ii++) {
            const int rl = wm * (16 * MI) + ii * 16 + fr;
            if (m0 + rl < rows) {
#pragma unroll
                for (int j = 0; j < 4; j++)
                    *reinterpret_cast<float4_t*>(pt + rl * kGemmBN + wn * 64 + (lane >> 4) * 4 +
                                                 j * 16) = acc[ii][j];
            }
        }
    }
    }  // pieces: every wave has passed the closing barrier of the last step, so the
       // next piece's prologue may refill the LDS stages
}

// Sums the fp32 partial tiles of every split tile in run order and rounds once to
// fp16. grid = (split tiles, BM/8): a workgroup of 256 threads finishes 8 rows x
// 256 columns, one float4 per thread and piece.
template <int MI>
__global__ __launch_bounds__(256) void gemm_fixup_kernel(const float* __restrict__ partial,
                                                         half_t* __restrict__ y, int rows,
                                                         size_t ldy, int tn_count,
                                                         int n_row_blocks, int full_tiles,
                                                         int ksteps, int pitch, int per) {
    constexpr int BM = 32 * MI;
    const int j = blockIdx.x;
    const int tile = full_tiles + j;
    const int g = tile / n_row_blocks;
    const int m0 = (tile % n_row_blocks) * BM;
    const int c4 = (threadIdx.x & 63) * 4;
    if (g * kGemmBN + c4 >= tn_count * 16) return;
    const int v0 = split_first_run(j, pitch, per), v1 = split_last_run(j, pitch, ksteps, per);
    const float* p0 = partial + (size_t)(v0 + j) * (BM * kGemmBN);
#pragma unroll
    for (int it = 0; it < 2; it++) {
        const int rl = blockIdx.y * 8 + it * 4 + (threadIdx.x >> 6);
        if (m0 + rl >= rows) return;
        const float* p = p0 + rl * kGemmBN + c4;
        float4_t s = *reinterpret_cast<const float4_t*>(p);
#pragma unroll 4
        for (int v = 1; v <= v1 - v0; v++)
            s = s + *reinterpret_cast<const float4_t*>(p + (size_t)v * (BM * kGemmBN));
        half4_t o;
        o.x = (half_t)s.x;
        o.y = (half_t)s.y;
        o.z = (half_t)s.z;
        o.w = (half_t)s.w;
        *reinterpret_cast<half4_t*>(y + (size_t)(m0 + rl) * ldy + g * kGemmBN + c4) = o;
    }
}

// The fix-up with the output transform folded in (every tile of the launch split):
// a wave finishes one row of the tile's 256 columns, i.e. two Hadamard blocks, one
// per half-wave, four values per lane. Same steps as the separate kernels: sum in
// range order, one cast to fp16, fp32 butterflies in ascending stride, scale, svh,
// cast, bias.
template <int MI>
__global__ __launch_bounds__(256) void gemm_fixup_post_kernel(
    const float* __restrict__ partial, int rows, int tn_count, int n_row_blocks, int full_tiles,
    int ksteps, int pitch, int per, const half_t* __restrict__ svh,
    const half_t* __restrict__ bias,
    half_t* __restrict__ out, size_t ldo) {
    constexpr int BM = 32 * MI;
    constexpr float kScale = 0.088388347648318440550f;  // 1/sqrt(128)
    const int tj = blockIdx.x;
    const int tile = full_tiles + tj;
    const int g = tile / n_row_blocks;
    const int m0 = (tile % n_row_blocks) * BM;
    const int lane = threadIdx.x & 63;
    const int c4 = lane * 4;
    const int col = g * kGemmBN + c4;
    const bool col_ok = col < tn_count * 16;  // false in the upper half of a half-width last block
    const int v0 = split_first_run(tj, pitch, per), v1 = split_last_run(tj, pitch, ksteps, per);
    const float* p0 = partial + (size_t)(v0 + tj) * (BM * kGemmBN);
#pragma unroll
    for (int it = 0; it < 2; it++) {
        const int rl = blockIdx.y * 8 + it * 4 + (threadIdx.x >> 6);
        if (m0 + rl >= rows) return;  // whole wave
        float4_t s = {0.f, 0.f, 0.f, 0.f};
        if (col_ok) {
            const float* p = p0 + rl * kGemmBN + c4;
            s = *reinterpret_cast<const float4_t*>(p);
            for (int v = 1; v <= v1 - v0; v++)
                s = s + *reinterpret_cast<const float4_t*>(p + (size_t)v * (BM * kGemmBN));
        }
        float v[4] = {(float)(half_t)s.x, (float)(half_t)s.y, (float)(half_t)s.z,
                      (float)(half_t)s.w};
#pragma unroll
        for (int h = 1; h < 4; h <<= 1) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                if ((j & h) == 0) {
                    const float lo = v[j], hi = v[j + h];
                    v[j] = __fadd_rn(lo, hi);
                    v[j + h] = __fsub_rn(lo, hi);
                }
            }
        }
        // lanes 1, 2, 4, 8 apart through DPP operands, 16 apart by swapping registers
        static_for<0, 4>([&](auto bit) {
            const uint32_t sign = lane_sign_mask(lane, bit.value);
#pragma unroll
            for (int j = 0; j < 4; j++) v[j] = butterfly_dpp<bit.value>(v[j], sign);
        });
#pragma unroll
        for (int j = 0; j < 4; j += 2) {
            swap_rows16(v[j], v[j + 1]);
            butterfly_in_lane(v[j], v[j + 1]);
            swap_rows16(v[j], v[j + 1]);
        }
        if (col_ok) {
            half_t o[4];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                float a = __fmul_rn(v[j], kScale);
                if (svh) a = __fmul_rn(a, (float)svh[col + j]);
                o[j] = (half_t)a;
                if (bias) o[j] = o[j] + bias[col + j];
            }
            half4_t ov;
            ov.x = o[0];
            ov.y = o[1];
            ov.z = o[2];
            ov.w = o[3];
            *reinterpret_cast<half4_t*>(out + (size_t)(m0 + rl) * ldo + col) = ov;
        }
    }
}

static int gemm_slots() {
    // one workgroup per CU; the count only shapes the schedule, never the result of a tile
    static const int cus = [] {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
            n < 1)
            n = 256;
        return n;
    }();
    return env_int("EXL3_GEMM_SLOTS", cus, 1, 4096);
}

GemmPlan plan_gemm(int rows, int in_tiles, int tn_count, bool allow_split) {
    GemmPlan p{};
    p.mi = rows <= 64 ? 2 : rows <= 128 ? 4 : 8;
    const int bm = 32 * p.mi;
    p.n_row_blocks = (rows + bm - 1) / bm;
    p.n_col_blocks = (tn_count + 15) / 16;
    const long long tiles = (long long)p.n_row_blocks * p.n_col_blocks;
    const int ksteps = in_tiles / 4;
    const int slots = gemm_slots();
    p.full_tiles = (int)tiles;
    p.split_tiles = p.split_runs = 0;
    p.split_per = ksteps;
    p.split_pitch = ksteps;
    p.split_runs_per_tile = 0;
    const int rem = (int)(tiles % slots);
    if (allow_split && rem > 0 && (long long)rem * ksteps * 2 < 0x7fffffffLL) {
        // Cost of the last round in tile times; 1 if its tiles stay whole. Every piece
        // also writes (and the fix-up reads) one fp32 tile and has a pipeline of its own
        // to fill: about the time of 8 steps.
        const int max_split = env_int("EXL3_GEMM_MAX_SPLIT", 16, 1, 64);
        const double piece_cost = 8.0;
        double best = 0.95;
        // (a) s runs per tile, none crossing a border: ceil(rem*s/slots) rounds of them
        for (int s = 2; s <= max_split && ksteps / s >= 4; s++) {
            const int kps = (ksteps + s - 1) / s;
            if ((ksteps + kps - 1) / kps != s) continue;  // some range would be empty
            const double cost =
                (double)(((long long)rem * s + slots - 1) / slots) * (kps + piece_cost) / ksteps;
            if (cost < best - 1e-9) {
                best = cost;
                p.split_per = kps;
                p.split_pitch = s * kps;
                p.split_runs_per_tile = s;
                p.split_runs = rem * s;
            }
        }
        // (b) one run per CU over the steps end to end: the runs that cross a border
        // work on two pieces
        if (max_split > 1) {
            const long long steps = (long long)rem * ksteps;
            long long per = (steps + slots - 1) / slots;
            const long long floor_per = (ksteps + max_split - 1) / max_split;
            if (per < floor_per) per = floor_per;
            if (per < 4) per = 4;
            if (per < ksteps) {
                const double cost = ((double)per + piece_cost * (ksteps % per ? 2 : 1)) / ksteps;
                if (cost < best - 1e-9) {
                    best = cost;
                    p.split_per = (int)per;
                    p.split_pitch = ksteps;
                    p.split_runs_per_tile = 0;
                    p.split_runs = (int)((steps + per - 1) / per);
                }
            }
        }
        if (best < 0.95) {
            p.full_tiles = (int)(tiles - rem);
            p.split_tiles = rem;
        } else {
            p.split_runs = 0;
        }
    }
    return p;
}

// fp32 partial tiles of the split region: slot = run + tile < runs + tiles
static size_t gemm_partial_slots(const GemmPlan& p) {
    return p.split_tiles ? (size_t)p.split_runs + p.split_tiles : 0;
}

size_t gemm_workspace_bytes(int rows, int in_tiles, int tn_count) {
    const GemmPlan p = plan_gemm(rows, in_tiles, tn_count, true);
    return gemm_partial_slots(p) * (32 * p.mi) * kGemmBN * sizeof(float);
}

template <int K, int CB, int MI>
static int launch_gemm_mi(const GemmPlan& p, const uint16_t* xh, int rows, size_t ldx,
                          const uint16_t* trellis, int in_tiles, int out_tiles, int tn_offset,
                          int tn_count, uint16_t* y_out, size_t ldy, float* partial,
                          hipStream_t stream, const GemmPost* post, const int32_t* block_sub,
                          size_t sub_stride) {
    // two stages of A and B, or (output transform inside the kernel) the fp16 tile with padded rows
    constexpr size_t lds_stages = (2 * (size_t)(32 * MI) * 64 + 2 * (size_t)kGemmStageB) * sizeof(half_t);
    constexpr size_t lds_tile = (size_t)(32 * MI) * (kGemmBN + 8) * sizeof(half_t);
    constexpr size_t lds = lds_stages > lds_tile ? lds_stages : lds_tile;
    const bool two = p.split_tiles > 0 && p.split_runs_per_tile == 0;
    auto kernel = two ? gemm_kernel<K, CB, MI, true> : gemm_kernel<K, CB, MI, false>;
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
        return EXL3_E_LAUNCH;
    const unsigned units = (unsigned)(p.full_tiles + p.split_runs);
    GemmArgs a{};
    a.trellis = reinterpret_cast<const uint32_t*>(trellis);
    a.xh = reinterpret_cast<const half_t*>(xh);
    a.y = reinterpret_cast<half_t*>(y_out);
    a.partial = partial;
    a.rows = rows;
    a.ldx = ldx;
    a.ldy = ldy;
    a.in_tiles = in_tiles;
    a.out_tiles = out_tiles;
    a.tn_offset = tn_offset;
    a.tn_count = tn_count;
    a.n_row_blocks = p.n_row_blocks;
    a.full_tiles = p.full_tiles;
    a.split = GemmSplit{p.split_per, p.split_pitch, p.split_runs_per_tile,
                        p.split_tiles * p.split_pitch};
    a.block_sub = block_sub;
    a.sub_stride = sub_stride;
    if (post) {
        a.post_svh = reinterpret_cast<const half_t*>(post->svh);
        a.post_bias = reinterpret_cast<const half_t*>(post->bias);
        a.post_out = reinterpret_cast<half_t*>(post->out);
        a.ldo = post->ldo;
    }
    kernel<<<dim3(units), dim3(kGemmThreads), lds, stream>>>(a);
    if (int rc = launch_status()) return rc;
    if (post) {
        // whole tiles were transformed by the kernel itself; split tiles by the pass that
        // adds their partial tiles
        if (p.split_tiles > 0) {
            gemm_fixup_post_kernel<MI>
                <<<dim3((unsigned)p.split_tiles, 4 * MI), dim3(256), 0, stream>>>(
                    partial, rows, tn_count, p.n_row_blocks, p.full_tiles, in_tiles / 4,
                    p.split_pitch, p.split_per, reinterpret_cast<const half_t*>(post->svh),
                    reinterpret_cast<const half_t*>(post->bias),
                    reinterpret_cast<half_t*>(post->out), post->ldo);
            return launch_status();
        }
        return EXL3_OK;
    }
    if (p.split_tiles > 0) {
        gemm_fixup_kernel<MI><<<dim3((unsigned)p.split_tiles, 4 * MI), dim3(256), 0, stream>>>(
            partial, reinterpret_cast<half_t*>(y_out), rows, ldy, tn_count, p.n_row_blocks,
            p.full_tiles, in_tiles / 4, p.split_pitch, p.split_per);
        return launch_status();
    }
    return EXL3_OK;
}

int launch_gemm(const uint16_t* xh, int rows, size_t ldx, const uint16_t* trellis, int in_tiles,
                int out_tiles, int K, int cb, int tn_offset, int tn_count, uint16_t* y_out,
                size_t ldy, void* workspace, size_t workspace_bytes, hipStream_t stream,
                const GemmPost* post, bool* post_done, const int32_t* block_sub,
                size_t sub_stride) {
    if (post_done) *post_done = false;
    if (int rc = check_k_cb(K, cb)) return rc;
    if (!xh || !trellis || !y_out) return EXL3_E_NULL_POINTER;
    if (rows < 1 || in_tiles < 4 || in_tiles % 4 || tn_offset < 0 || tn_count < 8 ||
        tn_count % 8 || tn_offset + tn_count > out_tiles || ldx < (size_t)in_tiles * 16 ||
        ldy < (size_t)tn_count * 16 || ldx % 8 || ldy % 4)
        return EXL3_E_BAD_SHAPE;
    if ((reinterpret_cast<uintptr_t>(xh) & 15) || (reinterpret_cast<uintptr_t>(y_out) & 7))
        return EXL3_E_BAD_SHAPE;
    if (ldx * 2 * 256 >= (1ull << 31)) return EXL3_E_BAD_SHAPE;  // 32-bit row offsets inside a block
    GemmPlan p = plan_gemm(rows, in_tiles, tn_count, workspace != nullptr);
    const size_t need = gemm_partial_slots(p) * (32 * p.mi) * kGemmBN * sizeof(float);
    if (need > workspace_bytes || (reinterpret_cast<uintptr_t>(workspace) & 15))
        p = plan_gemm(rows, in_tiles, tn_count, false);
    if ((long long)p.full_tiles + (long long)p.split_runs > 0x7fffffffLL) return EXL3_E_BAD_SHAPE;
    float* partial = reinterpret_cast<float*>(workspace);
    // the output transform rides on the kernel's epilogue (whole tiles) and on the fix-up
    // (split tiles); it needs whole Hadamard blocks of the whole width
    const bool fold = post && post->out && post_done && tn_offset == 0 && tn_count % 8 == 0 &&
                      post->ldo >= (size_t)tn_count * 16 && post->ldo % 4 == 0 &&
                      !(reinterpret_cast<uintptr_t>(post->out) & 7) &&
                      !(reinterpret_cast<uintptr_t>(post->svh) & 7) &&
                      !(reinterpret_cast<uintptr_t>(post->bias) & 7);
    const GemmPost* fp = fold ? post : nullptr;
    const int rc = dispatch_k_cb(K, cb, [&](auto k, auto c) {
        if (p.mi == 2)
            return launch_gemm_mi<k.value, c.value, 2>(p, xh, rows, ldx, trellis, in_tiles,
                                                       out_tiles, tn_offset, tn_count, y_out, ldy,
                                                       partial, stream, fp, block_sub, sub_stride);
        if (p.mi == 4)
            return launch_gemm_mi<k.value, c.value, 4>(p, xh, rows, ldx, trellis, in_tiles,
                                                       out_tiles, tn_offset, tn_count, y_out, ldy,
                                                       partial, stream, fp, block_sub, sub_stride);
        return launch_gemm_mi<k.value, c.value, 8>(p, xh, rows, ldx, trellis, in_tiles, out_tiles,
                                                   tn_offset, tn_count, y_out, ldy, partial,
                                                   stream, fp, block_sub, sub_stride);
    });
    if (rc == EXL3_OK && fold) *post_done = true;
    return rc;
}

template <int K, int CB, int MI>
static int launch_gemm_grouped_mi(const uint16_t* xh, int n_rows, size_t ldx,
                                  const uint16_t* trellis, int in_tiles, int out_tiles,
                                  int tn_base, int group_tiles, int n_groups,
                                  const int32_t* group_tab, int n_row_blocks, uint16_t* y_out,
                                  size_t ldy, hipStream_t stream) {
    constexpr size_t lds = (2 * (size_t)(32 * MI) * 64 + 2 * (size_t)kGemmStageB) * sizeof(half_t);
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_kernel<K, CB, MI, false>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
        return EXL3_E_LAUNCH;
    const long long units = (long long)n_row_blocks * ((group_tiles + 15) / 16);
    if (units > 0x7fffffffLL) return EXL3_E_BAD_SHAPE;
    GemmArgs a{};
    a.trellis = reinterpret_cast<const uint32_t*>(trellis);
    a.xh = reinterpret_cast<const half_t*>(xh);
    a.y = reinterpret_cast<half_t*>(y_out);
    a.rows = n_rows;
    a.ldx = ldx;
    a.ldy = ldy;
    a.in_tiles = in_tiles;
    a.out_tiles = out_tiles;
    a.tn_offset = tn_base;
    a.tn_count = group_tiles;
    a.n_row_blocks = 1;
    a.split = GemmSplit{in_tiles / 4, in_tiles / 4, 0, 0};
    a.group_tab = reinterpret_cast<const int4*>(group_tab);
    a.group_tiles = group_tiles;
    a.n_groups = n_groups;
    gemm_kernel<K, CB, MI, false><<<dim3((unsigned)units), dim3(kGemmThreads), lds, stream>>>(a);
    return launch_status();
}

int launch_gemm_grouped(const uint16_t* xh, int n_rows, size_t ldx, const uint16_t* trellis,
                        int in_tiles, int out_tiles, int K, int cb, int tn_base, int group_tiles,
                        int n_groups, const int32_t* group_tab, int n_row_blocks, int block_rows,
                        uint16_t* y_out, size_t ldy, hipStream_t stream) {
    if (int rc = check_k_cb(K, cb)) return rc;
    if (!xh || !trellis || !y_out || !group_tab) return EXL3_E_NULL_POINTER;
    if (n_rows < 1 || in_tiles < 4 || in_tiles % 4 || tn_base < 0 || group_tiles < 8 ||
        group_tiles % 8 || n_groups < 1 ||
        (long long)tn_base + (long long)n_groups * group_tiles > out_tiles || n_row_blocks < 1 ||
        ldx < (size_t)in_tiles * 16 || ldy < (size_t)group_tiles * 16 || ldx % 8 || ldy % 4)
        return EXL3_E_BAD_SHAPE;
    if (block_rows != 64 && block_rows != 128 && block_rows != 256) return EXL3_E_BAD_SHAPE;
    if ((reinterpret_cast<uintptr_t>(xh) & 15) || (reinterpret_cast<uintptr_t>(y_out) & 7) ||
        (reinterpret_cast<uintptr_t>(group_tab) & 15))
        return EXL3_E_BAD_SHAPE;
    if (ldx * 2 * 256 >= (1ull << 31)) return EXL3_E_BAD_SHAPE;
    return dispatch_k_cb(K, cb, [&](auto k, auto c) {
        if (block_rows == 64)
            return launch_gemm_grouped_mi<k.value, c.value, 2>(xh, n_rows, ldx, trellis, in_tiles,
                                                               out_tiles, tn_base, group_tiles,
                                                               n_groups, group_tab, n_row_blocks,
                                                               y_out, ldy, stream);
        if (block_rows == 128)
            return launch_gemm_grouped_mi<k.value, c.value, 4>(xh, n_rows, ldx, trellis, in_tiles,
                                                               out_tiles, tn_base, group_tiles,
                                                               n_groups, group_tab, n_row_blocks,
                                                               y_out, ldy, stream);
        return launch_gemm_grouped_mi<k.value, c.value, 8>(xh, n_rows, ldx, trellis, in_tiles,
                                                           out_tiles, tn_base, group_tiles,
                                                           n_groups, group_tab, n_row_blocks, y_out,
                                                           ldy, stream);
    });
}

}  // namespace exl3

EXL3_EXPORT int exl3_gemm_grouped(const uint16_t* xh, int n_rows, size_t ldx,
                                  const uint16_t* trellis, int in_tiles, int out_tiles, int K,
                                  int cb, int tn_base, int group_tiles, int n_groups,
                                  const int32_t* group_tab, int n_row_blocks, int block_rows,
                                  uint16_t* y_out, size_t ldy, void* stream) {
    return exl3::launch_gemm_grouped(xh, n_rows, ldx, trellis, in_tiles, out_tiles, K, cb, tn_base,
                                     group_tiles, n_groups, group_tab, n_row_blocks, block_rows,
                                     y_out, ldy, exl3::as_stream(stream));
}

EXL3_EXPORT size_t exl3_gemm_workspace_bytes(int rows, int in_tiles, int tn_count) {
    if (rows < 1 || in_tiles < 4 || tn_count < 8) return 0;
    return exl3::gemm_workspace_bytes(rows, in_tiles, tn_count);
}

EXL3_EXPORT int exl3_gemm(const uint16_t* xh, int rows, size_t ldx, const uint16_t* trellis,
                          int in_tiles, int out_tiles, int K, int cb, int tn_offset, int tn_count,
                          uint16_t* y_out, size_t ldy, void* workspace, size_t workspace_bytes,
                          void* stream) {
    return exl3::launch_gemm(xh, rows, ldx, trellis, in_tiles, out_tiles, K, cb, tn_offset,
                             tn_count, y_out, ldy, workspace, workspace_bytes,
                             exl3::as_stream(stream));
}
