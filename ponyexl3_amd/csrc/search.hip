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
// One workgroup of 256 lanes owns a tile: lane <-> compressed states e = lane,
// lane + 256, ..; both cost rows live in LDS (2 * 2^(16-K) halfs: 64 KiB at K=2,
// 512 B at K=8), the backpointers (256 steps x 2^(16-K) uint16) in the caller's
// workspace, one slot per resident workgroup; a workgroup walks over tiles
// blockIdx.x, blockIdx.x + gridDim.x, .. reusing its slot. Every step evaluates
// all 65536 codewords (decode + fma + compare), so a tile costs about
// 2 * 256 * 65536 * 12 lane-operations whatever K is; the serial backtrack
// (256 dependent loads by one lane) overlaps with the other workgroups of the CU.
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

template <int K, int CB>
__global__ __launch_bounds__(256) void quantize_tiles_kernel(const float* __restrict__ tiles,
                                                             float* __restrict__ q_tiles,
                                                             uint16_t* __restrict__ indices,
                                                             uint16_t* back_ws, int n_tiles) {
    constexpr int KR = 16 - K, EDGES = 1 << KR, KK = 1 << K;
    constexpr int PER_LANE = EDGES / 256;  // compressed states per lane (K <= 8)
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    half_t* costs = reinterpret_cast<half_t*>(lds_raw);  // [2][EDGES]
    __shared__ float target_s[256];
    __shared__ uint32_t red_key[4];
    __shared__ uint32_t sh_pin;
    const int tid = threadIdx.x;
    uint16_t* back = back_ws + (size_t)blockIdx.x * 256 * EDGES;

    for (int tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        __syncthreads();  // the previous tile's backtrack has finished with target_s / back
        target_s[tid] = tiles[(size_t)tile * 256 + tid];
        __syncthreads();
        uint32_t pin = 0;
        bool pinned = false;
        for (int pass = 0; pass < 2; pass++) {
            const int roll = pass == 0 ? 128 : 0;
            int curr = 0;
            for (int step = 0; step < 256; step++) {
                const int ri = (step + roll) & 255;
                const int prev_buf = curr;
                if (step > 0) curr ^= 1;
                const float target = target_s[ri];
                const half_t* cprev = costs + prev_buf * EDGES;
                half_t* ccurr = costs + curr * EDGES;
                const bool keep = pass == 1 || ri < 128;
#pragma unroll 1
                for (int i = 0; i < PER_LANE; i++) {
                    const uint32_t e = (uint32_t)(tid + 256 * i);
                    const uint32_t pred_lo = e >> K;  // low 16-2K bits of every predecessor
                    float best = kCostInf;
                    uint32_t best_fresh = KK;  // KK: no candidate beat the initial bound
#pragma unroll 4
                    for (int f4 = 0; f4 < KK; f4 += 4) {
                        float v[4];
                        decode4_f32<CB>(((uint32_t)(f4 + 0) << KR) | e, ((uint32_t)(f4 + 1) << KR) | e,
                                        ((uint32_t)(f4 + 2) << KR) | e, ((uint32_t)(f4 + 3) << KR) | e,
                                        v);
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            const uint32_t fresh = (uint32_t)(f4 + j);
                            const uint32_t pred = (fresh << (KR - K)) | pred_lo;
                            const float dh = __fsub_rn(v[j], target);
                            float err;
                            if (step == 0) {
                                err = __fmul_rn(dh, dh);
                                if (pinned && pred != pin) err = kCostInf;
                            } else {
                                err = __builtin_fmaf(dh, dh, (float)cprev[pred]);
                            }
                            err = err > kCostInf ? kCostInf : err;
                            if (err < best) {
                                best = err;
                                best_fresh = fresh;
                            }
                        }
                    }
                    ccurr[e] = (half_t)best;
                    if (keep) {
                        // the reference leaves the backpointer at 0 when nothing beat the bound
                        const uint32_t bp = best_fresh == KK ? 0u : (best_fresh << (KR - K)) | pred_lo;
                        back[(size_t)ri * EDGES + e] = (uint16_t)bp;
                    }
                }
                __syncthreads();
            }

            // first minimum of the final costs (pass 0) : key = cost bits : state
            if (pass == 0) {
                uint32_t key = 0xFFFFFFFFu;
                const half_t* cfin = costs + curr * EDGES;
                for (int i = 0; i < PER_LANE; i++) {
                    const uint32_t e = (uint32_t)(tid + 256 * i);
                    const uint32_t kbits = (uint32_t)__builtin_bit_cast(uint16_t, cfin[e]);
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
                    const uint32_t prev = back[(size_t)ri * EDGES + edge];
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
            pinned = true;
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

// Resident workgroups the search can keep per CU (waves and LDS), times the CUs.
static int quantize_slots_wanted(int K) {
    hipDeviceProp_t prop;
    int dev = 0;
    int cus = 256;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess)
        cus = prop.multiProcessorCount;
    const size_t lds = (size_t)4 << (16 - K);  // two rows of halfs
    size_t per_cu = (size_t)(160 * 1024 - 4096) / (lds + 2048);
    if (per_cu > 8) per_cu = 8;  // 8 workgroups x 4 waves fill the 32 wave slots
    if (per_cu < 1) per_cu = 1;
    return cus * (int)per_cu;
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
    const size_t lds = (size_t)4 << (16 - K);
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
                    tiles, q_tiles, indices, reinterpret_cast<uint16_t*>(workspace), n_tiles);
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
