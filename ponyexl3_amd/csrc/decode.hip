// exl3_decode_full and its two layout variants: packed trellis -> fp16 W_inner,
// bit-exact with ponyexl3/ref/decode.py:32-81.
//
// Row-major (in, out) and expert-grouped (E, in, out_e): one wavefront decodes
// the 8 tiles (tk, tn0..tn0+7): its 64 lanes read 256*K contiguous bytes, each
// lane decodes 32 codewords in registers, the 16x128 block is transposed through
// LDS and written as 16-byte chunks (half a tile row each, so a tile can be
// steered to its expert's slab).
//
// Transposed (out, in): one wavefront decodes the 8 tiles (tk0..tk0+7, tn), so
// that each of the tile column's 16 output rows receives 128 contiguous halfs.
#include "exl3_device.hpp"
#include "exl3_host.hpp"

namespace exl3 {

constexpr int kDecPad = 8;  // halfs of padding per staged row (keeps 16 B alignment)

template <int K, int CB>
__global__ __launch_bounds__(256) void decode_full_kernel(const uint32_t* __restrict__ trellis,
                                                          half_t* __restrict__ w_out, int in_tiles,
                                                          int out_tiles, int tn_offset,
                                                          int tn_count, int tiles_per_group) {
    __shared__ __attribute__((aligned(16))) half_t stage[4][16][128 + kDecPad];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int groups = (tn_count + 7) >> 3;
    const long long wid = (long long)blockIdx.x * 4 + wave;
    const bool active = wid < (long long)in_tiles * groups;
    const int g = active ? (int)(wid % groups) : 0;
    const int tk = active ? (int)(wid / groups) : 0;
    const int tile_local = g * 8 + (lane >> 3);
    const bool valid = active && tile_local < tn_count;
    // lanes of a tile past the slice re-read the last valid tile (never stored)
    const int tn = tn_offset + (valid ? tile_local : tn_count - 1);
    const uint32_t* p = trellis + ((size_t)tk * out_tiles + tn) * (8 * K) + (lane & 7) * K;
    uint32_t own[K];
#pragma unroll
    for (int i = 0; i < K; i++) own[i] = p[i];
    const LaneWords<K> lw = finish_lane_words<K>(own, lane);
    half2_t wp[16];
    decode_lane<K, CB>(lw, wp);
    const int c0 = (lane >> 3) * 16 + (lane & 7);
#pragma unroll
    for (int cs = 0; cs < 2; cs++)
#pragma unroll
        for (int j = 0; j < 8; j++) {
            stage[wave][2 * j][c0 + 8 * cs] = wp[8 * cs + j].x;
            stage[wave][2 * j + 1][c0 + 8 * cs] = wp[8 * cs + j].y;
        }
    __syncthreads();
    if (!active) return;
    // tiles_per_group == 0: one (in, 16*tn_count) matrix. Otherwise tile column t
    // goes to slab t / tiles_per_group, an (in, 16*tiles_per_group) matrix of its own.
    const int chunk = lane & 15;  // 8 halfs each; two chunks per tile
    const int t = g * 8 + (chunk >> 1);
    if (t >= tn_count) return;
    size_t ld = (size_t)tn_count * 16, col = (size_t)t * 16, slab = 0;
    if (tiles_per_group > 0) {
        ld = (size_t)tiles_per_group * 16;
        col = (size_t)(t % tiles_per_group) * 16;
        slab = (size_t)(t / tiles_per_group) * in_tiles * 16 * ld;
    }
#pragma unroll
    for (int pass = 0; pass < 4; pass++) {
        const int row = pass * 4 + (lane >> 4);
        const uint4_t v = *reinterpret_cast<const uint4_t*>(&stage[wave][row][chunk * 8]);
        *reinterpret_cast<uint4_t*>(w_out + slab + ((size_t)tk * 16 + row) * ld + col +
                                    (chunk & 1) * 8) = v;
    }
}

// W^T (16*tn_count, in): lanes 8t..8t+7 of a wave decode tile (tk0 + t, tn).
template <int K, int CB>
__global__ __launch_bounds__(256) void decode_full_t_kernel(const uint32_t* __restrict__ trellis,
                                                            half_t* __restrict__ w_out,
                                                            int in_tiles, int out_tiles,
                                                            int tn_offset, int tn_count) {
    __shared__ __attribute__((aligned(16))) half_t stage[4][16][128 + kDecPad];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int kgroups = (in_tiles + 7) >> 3;
    const long long wid = (long long)blockIdx.x * 4 + wave;
    const bool active = wid < (long long)tn_count * kgroups;
    const int kg = active ? (int)(wid % kgroups) : 0;
    const int tn_local = active ? (int)(wid / kgroups) : 0;
    const int tk_lane = kg * 8 + (lane >> 3);
    // lanes of a tile row past the matrix re-read the last tile row (never stored)
    const int tk = tk_lane < in_tiles ? tk_lane : in_tiles - 1;
    const uint32_t* p =
        trellis + ((size_t)tk * out_tiles + tn_offset + tn_local) * (8 * K) + (lane & 7) * K;
    uint32_t own[K];
#pragma unroll
    for (int i = 0; i < K; i++) own[i] = p[i];
    const LaneWords<K> lw = finish_lane_words<K>(own, lane);
    half2_t wp[16];
    decode_lane<K, CB>(lw, wp);
    // pair j of column u + 8*cs holds input rows 2j, 2j+1 of the tile: one 4-byte store
    const int u = lane & 7, r0 = (lane >> 3) * 16;
#pragma unroll
    for (int cs = 0; cs < 2; cs++)
#pragma unroll
        for (int j = 0; j < 8; j++)
            *reinterpret_cast<half2_t*>(&stage[wave][u + 8 * cs][r0 + 2 * j]) = wp[8 * cs + j];
    __syncthreads();
    if (!active) return;
    const size_t ld = (size_t)in_tiles * 16;
    const int chunk = lane & 15;
    if (kg * 8 + (chunk >> 1) >= in_tiles) return;
#pragma unroll
    for (int pass = 0; pass < 4; pass++) {
        const int c = pass * 4 + (lane >> 4);  // output row = column of the tile
        const uint4_t v = *reinterpret_cast<const uint4_t*>(&stage[wave][c][chunk * 8]);
        *reinterpret_cast<uint4_t*>(w_out + ((size_t)tn_local * 16 + c) * ld + (size_t)kg * 128 +
                                    chunk * 8) = v;
    }
}

// Packed tiles -> their 256 16-bit codewords in kernel (stream) order
// (unpack_trellis, ponyexl3/ref/trellis.py:153-214). Lanes 8t..8t+7 of a wave own
// tile t of eight consecutive tiles; lane u extracts codewords 32u..32u+31 and
// writes them as 64 contiguous bytes.
template <int K>
__global__ __launch_bounds__(256) void unpack_trellis_kernel(const uint32_t* __restrict__ trellis,
                                                             uint16_t* __restrict__ codewords,
                                                             long long n_tiles) {
    const int lane = threadIdx.x & 63;
    const long long wid = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
    const long long tile_lane = wid * 8 + (lane >> 3);
    // lanes past the last tile re-read it (never stored)
    const long long tile = tile_lane < n_tiles ? tile_lane : n_tiles - 1;
    const uint32_t* p = trellis + tile * (8 * K) + (lane & 7) * K;
    uint32_t own[K];
#pragma unroll
    for (int i = 0; i < K; i++) own[i] = p[i];
    const LaneWords<K> lw = finish_lane_words<K>(own, lane);
    uint32_t packed[16];
    static_for<0, 16>([&](auto i) {
        packed[i.value] = lane_codeword<K, 2 * i.value>(lw) | (lane_codeword<K, 2 * i.value + 1>(lw) << 16);
    });
    if (tile_lane >= n_tiles) return;
    uint4_t* dst = reinterpret_cast<uint4_t*>(codewords + tile * 256 + (lane & 7) * 32);
#pragma unroll
    for (int i = 0; i < 4; i++)
        dst[i] = uint4_t{packed[4 * i], packed[4 * i + 1], packed[4 * i + 2], packed[4 * i + 3]};
}

// Shared argument checks and launch of the row-major / expert-grouped kernel.
static int launch_decode_full(const uint16_t* trellis, int in_tiles, int out_tiles, int K, int cb,
                              int tn_offset, int tn_count, int tiles_per_group, uint16_t* w_out,
                              void* stream) {
    if (int rc = check_k_cb(K, cb)) return rc;
    if (!trellis || !w_out) return EXL3_E_NULL_POINTER;
    if (in_tiles < 0 || out_tiles < 0 || tn_offset < 0 || tn_count < 0 ||
        tn_offset + tn_count > out_tiles)
        return EXL3_E_BAD_SHAPE;
    if (in_tiles == 0 || tn_count == 0) return EXL3_OK;
    if ((reinterpret_cast<uintptr_t>(w_out) & 15) || (reinterpret_cast<uintptr_t>(trellis) & 3))
        return EXL3_E_BAD_SHAPE;
    const long long waves = (long long)in_tiles * ((tn_count + 7) / 8);
    const long long grid = (waves + 3) / 4;
    if (grid > 0x7FFFFFFFLL) return EXL3_E_BAD_SHAPE;
    return dispatch_k_cb(K, cb, [&](auto k, auto c) {
        decode_full_kernel<k.value, c.value><<<dim3((unsigned)grid), dim3(256), 0, as_stream(stream)>>>(
            reinterpret_cast<const uint32_t*>(trellis), reinterpret_cast<half_t*>(w_out), in_tiles,
            out_tiles, tn_offset, tn_count, tiles_per_group);
        return launch_status();
    });
}

}  // namespace exl3

EXL3_EXPORT int exl3_decode_full(const uint16_t* trellis, int in_tiles, int out_tiles, int K,
                                 int cb, int tn_offset, int tn_count, uint16_t* w_out,
                                 void* stream) {
    return exl3::launch_decode_full(trellis, in_tiles, out_tiles, K, cb, tn_offset, tn_count, 0,
                                    w_out, stream);
}

EXL3_EXPORT int exl3_decode_full_eg(const uint16_t* trellis, int in_tiles, int out_tiles, int K,
                                    int cb, int tiles_per_e, uint16_t* w_out, void* stream) {
    if (tiles_per_e < 1 || out_tiles < 0 || out_tiles % tiles_per_e) return EXL3_E_BAD_SHAPE;
    return exl3::launch_decode_full(trellis, in_tiles, out_tiles, K, cb, 0, out_tiles, tiles_per_e,
                                    w_out, stream);
}

EXL3_EXPORT int exl3_decode_full_t(const uint16_t* trellis, int in_tiles, int out_tiles, int K,
                                   int cb, int tn_offset, int tn_count, uint16_t* w_out_t,
                                   void* stream) {
    using namespace exl3;
    if (int rc = check_k_cb(K, cb)) return rc;
    if (!trellis || !w_out_t) return EXL3_E_NULL_POINTER;
    if (in_tiles < 0 || out_tiles < 0 || tn_offset < 0 || tn_count < 0 ||
        tn_offset + tn_count > out_tiles)
        return EXL3_E_BAD_SHAPE;
    if (in_tiles == 0 || tn_count == 0) return EXL3_OK;
    if ((reinterpret_cast<uintptr_t>(w_out_t) & 15) || (reinterpret_cast<uintptr_t>(trellis) & 3))
        return EXL3_E_BAD_SHAPE;
    const long long waves = (long long)tn_count * ((in_tiles + 7) / 8);
    const long long grid = (waves + 3) / 4;
    if (grid > 0x7FFFFFFFLL) return EXL3_E_BAD_SHAPE;
    return dispatch_k_cb(K, cb, [&](auto k, auto c) {
        decode_full_t_kernel<k.value, c.value>
            <<<dim3((unsigned)grid), dim3(256), 0, as_stream(stream)>>>(
                reinterpret_cast<const uint32_t*>(trellis), reinterpret_cast<half_t*>(w_out_t),
                in_tiles, out_tiles, tn_offset, tn_count);
        return launch_status();
    });
}

EXL3_EXPORT int exl3_unpack_trellis(const uint16_t* trellis, long long n_tiles, int K,
                                    uint16_t* codewords, void* stream) {
    using namespace exl3;
    if (K < 1 || K > 8) return EXL3_E_BAD_K;
    if (n_tiles < 0) return EXL3_E_BAD_SHAPE;
    if (n_tiles == 0) return EXL3_OK;
    if (!trellis || !codewords) return EXL3_E_NULL_POINTER;
    if ((reinterpret_cast<uintptr_t>(trellis) & 3) || (reinterpret_cast<uintptr_t>(codewords) & 15))
        return EXL3_E_BAD_SHAPE;
    const long long grid = (n_tiles + 31) / 32;
    if (grid > 0x7FFFFFFFLL) return EXL3_E_BAD_SHAPE;
    return dispatch_k_cb(K, 0, [&](auto k, auto) {
        unpack_trellis_kernel<k.value><<<dim3((unsigned)grid), dim3(256), 0, as_stream(stream)>>>(
            reinterpret_cast<const uint32_t*>(trellis), codewords, n_tiles);
        return launch_status();
    });
}
