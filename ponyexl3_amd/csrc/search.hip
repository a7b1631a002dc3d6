// Encoder side of the trellis: exl3_quantize_tiles (tail-biting Viterbi search
// over the bitshift trellis) and exl3_pack_trellis (K-bit symbols -> packed tile).
//
// The search follows the arithmetic of the reference's production kernel
// (ponyexl3/convert/metal_search.py:63-196) step for step so that both choose the
// same path: compressed state e = the newest 16-K bits of the codeword; the
// candidate for (fresh, e) is cw = (fresh << (16-K)) | e with predecessor
// cw >> K; path costs are kept as fp16 between steps, the update is one fp32 fma
// clamped to 65504, ties keep the lowest fresh. Pass 0 starts at position 128,
// runs once around the tile and backtracks to the state in front of position 0;
// pass 1 starts at position 0 pinned to that state and has to end in it.
//
// One workgroup of 256 lanes owns a tile; both cost rows live in LDS
// (2 * 2^(16-K) halfs: 64 KiB at K=2, 512 B at K=8), the backpointers (256 steps x
// 2^(16-K) uint16) in the caller's workspace, one slot per resident workgroup; a
// workgroup walks over tiles blockIdx.x, blockIdx.x + gridDim.x, .. reusing its
// slot. Every step evaluates all 65536 codewords, five VALU instructions each, so
// a tile costs about 2 * 256 * 65536 * 5 lane-operations whatever K is; the serial
// backtrack (256 dependent loads by one lane) overlaps with the other workgroup
// of the CU.
#include "exl3_device.hpp"
#include "exl3_host.hpp"

namespace exl3 {

constexpr float kCostInf = 65504.0f;

// fp32 values of four codewords.
template <int CB>
__device__ __forceinline__ void decode4_f32(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3,
                                            float (&v)[4]) {
    half2_t a, b;
    decode_pair2<CB>(c0, c1, c2, c3, a, b);
    v[0] = (float)a.x;
    v[1] = (float)a.y;
    v[2] = (float)b.x;
    v[3] = (float)b.y;
}

template <int CB>
__device__ __forceinline__ float decode1_f32(uint32_t cw) {
    float v[4];
    decode4_f32<CB>(cw, cw, cw, cw, v);
    return v[0];
}

// if (err < best) { best = err; best_f = F; } with F an inline constant (0..64):
// compare into VCC and two selects, nothing held in scalar registers.
template <int F>
__device__ __forceinline__ void take_if_less(float err, float& best, uint32_t& best_f) {
    static_assert(F >= 0 && F <= 64, "inline integer constants end at 64");
    asm("v_cmp_lt_f32_e32 vcc, %2, %0\n\t"
        "v_cndmask_b32_e32 %0, %0, %2, vcc\n\t"
        "v_cndmask_b32_e64 %1, %1, %3, vcc"
        : "+v"(best), "+v"(best_f)
        : "v"(err), "n"(F)
        : "vcc");
}

// Lane <-> state assignment. With L = tid & (2^K - 1) and hi = tid >> K a lane owns
// the PER_LANE = 2^(8-K) compressed states e(j) = L | ((hi*PER_LANE + j) << K).
// Their predecessors for one fresh value f, (f << (16-2K)) | (hi*PER_LANE + j), are
// consecutive in j, so a lane fetches the previous costs of up to eight of its
// states with one LDS read. The 256 codewords (f, j) a lane ever evaluates do
// not depend on the step: their decoded fp16 values stay in 128 registers for the
// whole launch, and a candidate costs five VALU instructions: two mixed-precision
// fmas (value - target; dh*dh + previous cost, both reading their fp16 operand
// directly), one compare and two selects.
template <int K, int CB>
__global__ __launch_bounds__(256, 2) void quantize_tiles_kernel(const float* __restrict__ tiles,
                                                             float* __restrict__ q_tiles,
                                                             uint16_t* __restrict__ indices,
                                                             uint16_t* back_ws, int n_tiles,
                                                             float one) {
    constexpr int KR = 16 - K, EDGES = 1 << KR, KK = 1 << K;
    constexpr int PER_LANE = EDGES / 256;             // states per lane
    constexpr int CH = PER_LANE < 8 ? PER_LANE : 8;   // states per LDS read
    // A cost row is stored in blocks of 256 states with PAD halfs between blocks:
    // the lanes of a wave write the states of 64 / 2^K different blocks at the same
    // offset, and unpadded those would all fall into the same LDS banks.
    constexpr int PAD = KK > 8 ? KK : 8;
    constexpr int ROW = EDGES + (EDGES / 256) * PAD;
    auto row_index = [](uint32_t e) { return e + (e >> 8) * PAD; };
    // Backpointers of one step are stored as [j][lane] (lane = owner of the state,
    // j = its index among the lane's states): wave-wide contiguous stores.
    auto back_index = [](uint32_t e) {
        const uint32_t pj = e >> K;
        const uint32_t owner = ((pj / PER_LANE) << K) | (e & (KK - 1));
        return (pj % PER_LANE) * 256 + owner;
    };
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    half_t* costs = reinterpret_cast<half_t*>(lds_raw);  // [2][EDGES]
    __shared__ float target_s[256];
    __shared__ uint32_t red_key[4];
    __shared__ uint32_t sh_pin;
    const int tid = threadIdx.x;
    const uint32_t low = (uint32_t)tid & (KK - 1);
    const uint32_t base = ((uint32_t)tid >> K) * PER_LANE;  // e(j) >> K = base + j
    uint16_t* back = back_ws + (size_t)blockIdx.x * 256 * EDGES;
    // lane parts of the cost-row addresses (see unit_addr and the store below)
    const uint32_t lane_rd0 = KR - K >= 8 ? base + (base >> 8) * PAD : base;
    const uint32_t lane_wr0 = row_index((base << K) | low);

    // decoded values of the lane's codewords, index c = f*PER_LANE + j, two per register
    half2_t lut[128];
#pragma unroll
    for (int c = 0; c < 256; c += 4) {
        uint32_t cw[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t f = (uint32_t)(c + i) / PER_LANE, j = (uint32_t)(c + i) % PER_LANE;
            cw[i] = (f << KR) | ((base + j) << K) | low;
        }
        decode_pair2<CB>(cw[0], cw[1], cw[2], cw[3], lut[c / 2], lut[c / 2 + 1]);
    }

    for (int tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        __syncthreads();  // the previous tile's backtrack has finished with target_s / back
        target_s[tid] = tiles[(size_t)tile * 256 + tid];
        uint32_t pin = 0;
        for (int pass = 0; pass < 2; pass++) {
            const int roll = pass == 0 ? 128 : 0;
            // Step 0 has no predecessor costs: a row of zeros stands in for them
            // (fma(dh, dh, 0) is the rounded square), and in the pinned pass +inf
            // everywhere but at the pin keeps every other predecessor from winning.
            {
                const half_t open = pass == 0 ? (half_t)0.0f : bits_to_half(0x7C00);
                for (int i = 0; i < PER_LANE; i++) {
                    const uint32_t e = (uint32_t)(tid + 256 * i);
                    costs[ROW + row_index(e)] = (pass == 1 && e == pin) ? (half_t)0.0f : open;
                }
            }
            __syncthreads();
#pragma unroll 1
            for (int step = 0; step < 256; step++) {
                const int ri = (step + roll) & 255;
                const half_t* cprev = costs + ((step & 1) ^ 1) * ROW;
                half_t* ccurr = costs + (step & 1) * ROW;
                const float negt = -target_s[ri];
                // The table is the same in every step; without this the compiler hoists
                // its 256 fp16 -> fp32 conversions out of the loop and runs out of registers.
#pragma unroll
                for (int i = 0; i < 128; i++) asm volatile("" : "+v"(lut[i]));

                // Read units: UNIT previous costs from consecutive LDS addresses. For
                // K <= 7 a unit is one fresh value f and CH consecutive states of the
                // lane; at K = 8 a lane has one state whose predecessors are the fresh
                // values themselves, eight to a unit. One unit is fetched ahead.
                constexpr bool ALONG_F = PER_LANE == 1;
                constexpr int UNIT = ALONG_F ? 8 : CH;
                constexpr int N_UNITS = 256 / UNIT;
                // Address = lane part (computed once) + a compile-time part that fits the
                // immediate offset of the LDS instruction. The split is exact: the fresh
                // value contributes whole 256-state blocks (K <= 4) or decides the block
                // on its own (K > 4), and a lane's states never cross a block.
                auto unit_addr = [&](int u) -> const half_t* {
                    if constexpr (ALONG_F) {
                        return cprev + u * 8;  // base = 0: predecessor = fresh
                    } else {
                        const int ch = u / KK, f = u % KK;
                        const int fpart = f << (KR - K);
                        const int blocks = KR - K >= 8 ? fpart >> 8 : f >> (8 - (KR - K));
                        return cprev + lane_rd0 + (fpart + ch * CH + blocks * PAD);
                    }
                };
                auto fetch = [&](int u) {
                    uint4_t v = {0u, 0u, 0u, 0u};
                    const half_t* src = unit_addr(u);
                    if constexpr (UNIT == 8) {
                        v = *reinterpret_cast<const uint4_t*>(src);
                    } else if constexpr (UNIT == 4) {
                        const uint2_t t = *reinterpret_cast<const uint2_t*>(src);
                        v.x = t.x;
                        v.y = t.y;
                    } else {
                        v.x = *reinterpret_cast<const uint32_t*>(src);
                    }
                    return v;
                };
                // Fresh values are walked in blocks of 64 so that the index a select
                // writes is an inline constant; blocks after the first are merged into
                // the running minimum with a strict <, which keeps the first minimum.
                constexpr int NB = ALONG_F ? 1 : CH;  // running minima held at a time
                constexpr uint32_t kNone = 64;        // block-local "nothing beat the bound"
                constexpr uint32_t kNoneAll = KK > 64 ? KK : 64;  // the same for the whole walk
                float best[NB], blk_best[NB];
                uint32_t best_f[NB], blk_f[NB];
                uint4_t cur = fetch(0);
                static_for<0, N_UNITS>([&](auto uc) {
                    constexpr int u = uc.value;
                    const uint4_t nxt = fetch(u + 1 < N_UNITS ? u + 1 : u);
                    constexpr int ch = ALONG_F ? 0 : u / KK;
                    constexpr int f0 = ALONG_F ? u * 8 : u % KK;
                    if constexpr ((f0 & 63) == 0) {
#pragma unroll
                        for (int b = 0; b < NB; b++) {
                            if (f0 == 0) {
                                best[b] = kCostInf;
                                best_f[b] = kNoneAll;
                            }
                            blk_best[b] = kCostInf;
                            blk_f[b] = kNone;
                        }
                    }
                    const uint32_t words[4] = {cur.x, cur.y, cur.z, cur.w};
                    static_for<0, UNIT>([&](auto ic) {
                        constexpr int i = ic.value;
                        constexpr int f = ALONG_F ? f0 + i : f0;
                        constexpr int b = ALONG_F ? 0 : i;
                        constexpr int c = ALONG_F ? f : f * PER_LANE + ch * CH + i;
                        const half_t val = (c & 1) ? lut[c >> 1].y : lut[c >> 1].x;
                        const half2_t pp = bits_to_half2(words[i >> 1]);
                        const half_t pc = (i & 1) ? pp.y : pp.x;
                        // `one` is 1.0f passed as a kernel argument, so both fmas keep an
                        // fp16 operand and are converted inside the instruction
                        const float dh = __builtin_fmaf((float)val, one, negt);
                        const float err = __builtin_fmaf(dh, dh, (float)pc);
                        // an error at or above the bound never wins, which is all the
                        // reference's clamp to 65504 achieves
                        if constexpr (KK <= 64)
                            take_if_less<f>(err, best[b], best_f[b]);
                        else
                            take_if_less<(f & 63)>(err, blk_best[b], blk_f[b]);
                    });
                    constexpr int f_last = ALONG_F ? f0 + 7 : f0;
                    if constexpr (KK > 64 && (f_last & 63) == 63) {
#pragma unroll
                        for (int b = 0; b < NB; b++) {
                            if (blk_best[b] < best[b]) {
                                best[b] = blk_best[b];
                                best_f[b] = blk_f[b] + (uint32_t)(f_last & ~63);
                            }
                        }
                    }
                    if constexpr (f_last == KK - 1) {
                        // one scalar base per chunk; the stores below differ only in their
                        // immediate offsets and share the lane offset (otherwise the compiler
                        // keeps a separate offset register per store, 64 of them at K = 2)
                        size_t row_off = (size_t)ri * EDGES + (ch * CH) * 256;
                        asm volatile("" : "+s"(row_off));
                        uint16_t* rowbase = back + row_off;
#pragma unroll
                        for (int b = 0; b < NB; b++) {
                            const uint32_t pj = base + ch * CH + b;
                            // state (pj << K) | low: all states of a lane lie in one block
                            ccurr[lane_wr0 + ((ch * CH + b) << K)] = (half_t)best[b];
                            // The reference leaves the backpointer at 0 when nothing beat the
                            // bound. It skips the store for positions 128..255 of the warm-up
                            // pass, which nobody reads; storing them anyway (the pinned pass
                            // rewrites every row before it is walked) keeps the loop free of
                            // branches.
                            const uint32_t bp =
                                best_f[b] == kNoneAll ? 0u : (best_f[b] << (KR - K)) | pj;
                            rowbase[b * 256 + tid] = (uint16_t)bp;
                        }
                    }
                    cur = nxt;
                    __builtin_amdgcn_sched_barrier(0);
                });
                __syncthreads();
            }

            // first minimum of the final costs (pass 0): key = cost bits : state
            if (pass == 0) {
                uint32_t key = 0xFFFFFFFFu;
                const half_t* cfin = costs + ROW;  // step 255 wrote row 1
                for (int i = 0; i < PER_LANE; i++) {
                    const uint32_t e = (uint32_t)(tid + 256 * i);
                    const uint32_t kbits = (uint32_t)half_to_bits(cfin[row_index(e)]);
                    const uint32_t cand = (kbits << 16) | e;
                    key = cand < key ? cand : key;
                }
#pragma unroll
                for (int off = 32; off > 0; off >>= 1) {
                    const uint32_t o = (uint32_t)__shfl_xor((int)key, off, kWave);
                    key = o < key ? o : key;
                }
                if ((tid & 63) == 0) red_key[tid >> 6] = key;
            }
            __syncthreads();
            if (tid == 0) {
                uint32_t edge = pin;
                if (pass == 0) {
                    uint32_t key = red_key[0];
                    for (int w = 1; w < 4; w++) key = red_key[w] < key ? red_key[w] : key;
                    // a cost that never dropped below the bound selects state 0
                    edge = (key >> 16) >= 0x7BFFu ? 0u : (key & 0xFFFFu);
                }
                for (int step_i = 255; step_i >= 0; step_i--) {
                    const int ri = (step_i + roll) & 255;
                    const uint32_t prev = back[(size_t)ri * EDGES + back_index(edge)];
                    const uint32_t state = ((prev << K) | edge) & 0xFFFFu;
                    edge = prev;
                    if (pass == 1) {
                        indices[(size_t)tile * 256 + ri] = (uint16_t)state;
                        q_tiles[(size_t)tile * 256 + ri] = decode1_f32<CB>(state);
                    } else if (ri == 0) {
                        break;
                    }
                }
                sh_pin = edge;
            }
            __syncthreads();
            pin = sh_pin;
        }
    }
}

// K-bit symbols -> packed tile (ponyexl3/ref/trellis.py:13-49, mlx_trellis.py:66-84).
// Symbol c occupies stream bits [c*K, (c+1)*K), MSB first inside each 32-bit
// word; one lane assembles one word.
__global__ __launch_bounds__(256) void pack_trellis_kernel(const uint16_t* __restrict__ encoded,
                                                           uint32_t* __restrict__ packed,
                                                           long long n_words, int K) {
    const long long gid = (long long)blockIdx.x * 256 + threadIdx.x;
    if (gid >= n_words) return;
    const int words_per_tile = 8 * K;
    const long long tile = gid / words_per_tile;
    const int d = (int)(gid % words_per_tile);
    const uint16_t* src = encoded + tile * 256;
    const uint32_t mask = (1u << K) - 1u;
    const int first = (32 * d) / K, last = (32 * d + 31) / K;
    uint32_t word = 0;
    for (int c = first; c <= last; c++) {
        const int off = c * K - 32 * d;  // may be negative: the symbol began in the previous word
        const uint64_t v = (uint64_t)(src[c] & mask) << 32;
        word |= (uint32_t)(v >> (off + K));
    }
    packed[gid] = word;
}

// Workgroups the search keeps resident: the kernel holds its decode table in
// registers; its register count leaves room for two waves per SIMD, i.e. two
// workgroups per CU (three from K = 6 on, where fewer address registers are live).
static int quantize_slots_wanted(int K) {
    hipDeviceProp_t prop;
    int dev = 0;
    int cus = 256;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess)
        cus = prop.multiProcessorCount;
    return cus * (K >= 6 ? 3 : 2);
}

}  // namespace exl3

EXL3_EXPORT size_t exl3_quantize_slot_bytes(int K) {
    if (K < 2 || K > 8) return 0;
    return (size_t)256 * sizeof(uint16_t) << (16 - K);
}

EXL3_EXPORT size_t exl3_quantize_workspace_bytes(int n_tiles, int K) {
    if (K < 2 || K > 8 || n_tiles < 1) return 0;
    const int want = exl3::quantize_slots_wanted(K);
    return exl3_quantize_slot_bytes(K) * (size_t)(n_tiles < want ? n_tiles : want);
}

EXL3_EXPORT int exl3_quantize_tiles(const float* tiles, int n_tiles, int K, int cb, float* q_tiles,
                                    uint16_t* indices, void* workspace, size_t workspace_bytes,
                                    void* stream) {
    using namespace exl3;
    if (K < 2 || K > 8) return EXL3_E_BAD_K;  // K = 1 is not supported by the reference either
    if (int rc = check_k_cb(K, cb)) return rc;
    if (n_tiles < 0) return EXL3_E_BAD_SHAPE;
    if (n_tiles == 0) return EXL3_OK;
    if (!tiles || !q_tiles || !indices || !workspace) return EXL3_E_NULL_POINTER;
    const size_t slot = exl3_quantize_slot_bytes(K);
    size_t slots = workspace_bytes / slot;
    if (slots < 1) return EXL3_E_WORKSPACE;
    const size_t want = (size_t)quantize_slots_wanted(K);
    if (slots > want) slots = want;
    if (slots > (size_t)n_tiles) slots = (size_t)n_tiles;
    const size_t edges = (size_t)1 << (16 - K);
    const size_t pad = (size_t)((1 << K) > 8 ? (1 << K) : 8);
    const size_t lds = 2 * sizeof(uint16_t) * (edges + edges / 256 * pad);  // two padded cost rows
    return dispatch_k_cb(K, cb, [&](auto k, auto c) {
        if constexpr (k.value < 2) {
            return (int)EXL3_E_BAD_K;
        } else {
            if (hipFuncSetAttribute(
                    reinterpret_cast<const void*>(quantize_tiles_kernel<k.value, c.value>),
                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
                return (int)EXL3_E_LAUNCH;
            quantize_tiles_kernel<k.value, c.value>
                <<<dim3((unsigned)slots), dim3(256), lds, as_stream(stream)>>>(
                    tiles, q_tiles, indices, reinterpret_cast<uint16_t*>(workspace), n_tiles, 1.0f);
            return launch_status();
        }
    });
}

EXL3_EXPORT int exl3_pack_trellis(const uint16_t* encoded, long long n_tiles, int K,
                                  uint16_t* packed, void* stream) {
    using namespace exl3;
    if (K < 1 || K > 8) return EXL3_E_BAD_K;
    if (n_tiles < 0) return EXL3_E_BAD_SHAPE;
    if (n_tiles == 0) return EXL3_OK;
    if (!encoded || !packed) return EXL3_E_NULL_POINTER;
    if (reinterpret_cast<uintptr_t>(packed) & 3) return EXL3_E_BAD_SHAPE;
    const long long n_words = n_tiles * 8 * K;
    const long long grid = (n_words + 255) / 256;
    if (grid > 0x7FFFFFFFLL) return EXL3_E_BAD_SHAPE;
    pack_trellis_kernel<<<dim3((unsigned)grid), dim3(256), 0, as_stream(stream)>>>(
        encoded, reinterpret_cast<uint32_t*>(packed), n_words, K);
    return launch_status();
}
