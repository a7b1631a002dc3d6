// Composite C-ABI entry points: status text and the whole-layer forward that
// chains the Hadamard, GEMV/GEMM and finishing kernels on one stream.
#include "exl3_device.hpp"
#include "exl3_host.hpp"

#include <mutex>

namespace exl3 {

// Workspace layout of exl3_linear_forward:
//   [0, xh_bytes)            xh  fp16 [rows][n_sub][in]
//   [xh_bytes, ...)          rows <= kGemvMaxRows: fp32 split-K partials
//                            otherwise:            fp16 y [rows][out], or (rows <=
//                            kLinearMidMaxRows, medium-batch kernel) fp32 partials
//   then (rows > kGemvMaxRows) the fp32 partial tiles of the prefill GEMM
struct LinearWorkspace {
    size_t xh_bytes;
    size_t second_bytes;
    size_t gemm_bytes;
    size_t total() const { return xh_bytes + second_bytes + gemm_bytes; }
};

static LinearWorkspace linear_workspace(int rows, int in_features, int out_features, int n_sub) {
    LinearWorkspace w{};
    w.xh_bytes = align_up((size_t)rows * n_sub * in_features * 2, 256);
    if (rows <= kGemvMaxRows) {
        const GemvPlan a = plan_gemv(rows, in_features / 16, out_features / 128);
        const GemvPlan b = plan_linear_small(rows, in_features / 16, out_features / 128);
        const int n = a.n_partials() > b.n_partials() ? a.n_partials() : b.n_partials();
        w.second_bytes = (size_t)n * rows * out_features * sizeof(float);
    } else {
        w.second_bytes = (size_t)rows * out_features * 2;
        if (rows <= kLinearMidMaxRows) {
            const MidPlan m = plan_linear_mid(rows, in_features / 16, out_features / 128);
            const size_t mid = (size_t)m.n_splits * rows * out_features * sizeof(float);
            if (mid > w.second_bytes) w.second_bytes = mid;
        }
        w.gemm_bytes = align_up(gemm_workspace_bytes(rows, in_features / 16, out_features / 16), 256);
    }
    w.second_bytes = align_up(w.second_bytes, 256);
    return w;
}

}  // namespace exl3

EXL3_EXPORT int exl3_version(void) { return 100; }

EXL3_EXPORT const char* exl3_status_string(int status) {
    switch (status) {
        case EXL3_OK: return "ok";
        case EXL3_E_BAD_K: return "K must be in [1, 8]";
        case EXL3_E_BAD_CODEBOOK: return "codebook id must be 0 (3INST), 1 (MCG) or 2 (MUL1)";
        case EXL3_E_BAD_SHAPE: return "invalid shape, slice, row count or alignment";
        case EXL3_E_NULL_POINTER: return "a required pointer is NULL";
        case EXL3_E_WORKSPACE: return "workspace too small";
        case EXL3_E_LAUNCH: return "HIP kernel launch failed";
        case EXL3_E_BAD_INDEX: return "inconsistent group/expert index table";
        case EXL3_E_UNSUPPORTED: return "no kernel for this request";
        case EXL3_E_STATIC_LIMIT:
            return "request needs more scratch than the built-in array of exl3_linear_forward_static holds";
        case EXL3_E_INCOMPLETE:
            return "a split reduction gave up waiting (counters not zero on entry, or shared by "
                   "overlapping calls); the affected outputs are NaN and the counters must be zeroed";
        default: return "unknown status";
    }
}

EXL3_EXPORT size_t exl3_linear_workspace_bytes(int rows, int in_features, int out_features,
                                               int n_sub) {
    if (rows < 1 || in_features < 128 || out_features < 128 || n_sub < 1) return 0;
    return exl3::linear_workspace(rows, in_features, out_features, n_sub).total();
}

EXL3_EXPORT int exl3_linear_forward(const uint16_t* x, int rows, const uint16_t* trellis,
                                    int in_tiles, int out_tiles, int K, int cb,
                                    const uint16_t* suh, int n_sub, const int32_t* group_sub,
                                    const uint16_t* svh, const uint16_t* bias, uint16_t* y,
                                    void* workspace, size_t workspace_bytes, int32_t* counters,
                                    size_t counters_len, void* stream) {
    using namespace exl3;
    if (int rc = check_k_cb(K, cb)) return rc;
    if (!x || !trellis || !y || !workspace) return EXL3_E_NULL_POINTER;
    if (rows < 1 || in_tiles < 8 || out_tiles < 8 || in_tiles % 8 || out_tiles % 8 || n_sub < 1)
        return EXL3_E_BAD_SHAPE;  // Hadamard-128 needs multiples of 128 (ref/hadamard.py:67-68)
    if (n_sub > 1 && (!group_sub || !suh)) return EXL3_E_BAD_INDEX;
    const int in_features = in_tiles * 16, out_features = out_tiles * 16;
    const LinearWorkspace ws = linear_workspace(rows, in_features, out_features, n_sub);
    if (workspace_bytes < ws.total()) return EXL3_E_WORKSPACE;
    hipStream_t s = as_stream(stream);
    uint16_t* xh = reinterpret_cast<uint16_t*>(workspace);
    char* second = reinterpret_cast<char*>(workspace) + ws.xh_bytes;

    if (rows <= kGemvMaxRows) {
        const int n_groups = out_tiles / 8;
        const GemvPlan plan = plan_gemv(rows, in_tiles, n_groups);
        float* partial = reinterpret_cast<float*>(second);
        if (counters && !exact_weights()) {
            // one launch: rotation, GEMV, split reduction and output transform fused;
            // the counters array holds the 64-bit accumulators (two ints each)
            const size_t need = linear_small_counter_ints(rows, out_features);
            if (counters_len < need) return EXL3_E_WORKSPACE;
            return launch_linear_small(x, rows, trellis, in_tiles, out_tiles, K, cb, suh, n_sub,
                                       group_sub, svh, bias, y, partial, counters,
                                       plan_linear_small_launch(rows, in_tiles, n_groups, K), s,
                                       counters_status_word(counters, counters_len, need));
        }
        if (int rc = launch_had_pre(x, rows, in_features, suh, n_sub, xh, s)) return rc;
        if (int rc = launch_gemv_partials(xh, rows, n_sub, trellis, in_tiles, out_tiles, K, cb,
                                          group_sub, nullptr, n_groups, partial, plan, s))
            return rc;
        return launch_had_post(partial, 1, plan.n_partials(), (size_t)rows * out_features, rows,
                               out_features, svh, bias, y, s);
    }

    // Prefill: rotation kernel, MFMA GEMM, output transform.
    if (int rc = launch_had_pre(x, rows, in_features, suh, n_sub, xh, s)) return rc;
    if (counters && rows <= linear_mid_max_rows()) {
        // a few dozen rows: the decode still sets the pace; every weight is decoded
        // once and goes from registers into 16x16x32 MFMA; split reduction and output
        // transform in the same launch
        const int n_groups = out_tiles / 8;
        if (counters_len < (size_t)n_groups) return EXL3_E_WORKSPACE;
        return launch_linear_mid(xh, rows, trellis, in_tiles, out_tiles, K, cb, n_sub, group_sub,
                                 svh, bias, y, reinterpret_cast<float*>(second), counters,
                                 plan_linear_mid(rows, in_tiles, n_groups), s);
    }
    uint16_t* ytmp = reinterpret_cast<uint16_t*>(second);
    if (n_sub == 1) {
        const GemmPost post{svh, bias, y, (size_t)out_features};
        bool post_done = false;
        if (int rc = launch_gemm(xh, rows, (size_t)in_features, trellis, in_tiles, out_tiles, K, cb,
                                 0, out_tiles, ytmp, (size_t)out_features,
                                 second + ws.second_bytes, ws.gemm_bytes, s, &post, &post_done))
            return rc;
        if (post_done) return EXL3_OK;  // few rows: the fix-up pass applied the output transform
    } else {
        return EXL3_E_UNSUPPORTED;  // fused groups run their members one by one on the host side
    }
    return launch_had_post(ytmp, 0, 1, 0, rows, out_features, svh, bias, y, s);
}

// Prefill of a layer whose activations are already rotated: MFMA GEMM over
// xh [rows][n_sub][in] (block_sub picks the rotation of every 256-column block when
// n_sub > 1), then the output transform, folded into the GEMM's fix-up pass where
// every tile is split.
EXL3_EXPORT size_t exl3_linear_prefill_workspace_bytes(int rows, int in_features, int out_features) {
    if (rows < 1 || in_features < 64 || out_features < 128) return 0;
    using namespace exl3;
    return align_up((size_t)rows * out_features * 2, 256) +
           align_up(gemm_workspace_bytes(rows, in_features / 16, out_features / 16), 256);
}

EXL3_EXPORT int exl3_linear_prefill(const uint16_t* xh, int rows, int n_sub, const uint16_t* trellis,
                                    int in_tiles, int out_tiles, int K, int cb,
                                    const int32_t* block_sub, const uint16_t* svh,
                                    const uint16_t* bias, uint16_t* y, void* workspace,
                                    size_t workspace_bytes, void* stream) {
    using namespace exl3;
    if (int rc = check_k_cb(K, cb)) return rc;
    if (!xh || !trellis || !y || !workspace) return EXL3_E_NULL_POINTER;
    if (rows < 1 || in_tiles < 8 || out_tiles < 8 || in_tiles % 8 || out_tiles % 8 || n_sub < 1)
        return EXL3_E_BAD_SHAPE;
    if (n_sub > 1 && !block_sub) return EXL3_E_BAD_INDEX;
    const int in_features = in_tiles * 16, out_features = out_tiles * 16;
    const size_t y_bytes = align_up((size_t)rows * out_features * 2, 256);
    const size_t g_bytes = align_up(gemm_workspace_bytes(rows, in_tiles, out_tiles), 256);
    if (workspace_bytes < y_bytes + g_bytes) return EXL3_E_WORKSPACE;
    hipStream_t s = as_stream(stream);
    uint16_t* ytmp = reinterpret_cast<uint16_t*>(workspace);
    const GemmPost post{svh, bias, y, (size_t)out_features};
    bool post_done = false;
    if (int rc = launch_gemm(xh, rows, (size_t)n_sub * in_features, trellis, in_tiles, out_tiles, K,
                             cb, 0, out_tiles, ytmp, (size_t)out_features,
                             reinterpret_cast<char*>(workspace) + y_bytes, g_bytes, s, &post,
                             &post_done, n_sub > 1 ? block_sub : nullptr, (size_t)in_features))
        return rc;
    if (post_done) return EXL3_OK;
    return launch_had_post(ytmp, 0, 1, 0, rows, out_features, svh, bias, y, s);
}

// ---------------------------------------------------------------------------
// exl3_linear_forward_static: the one-launch small-batch layer for callers that
// cannot allocate device memory (code under HIP graph capture, serving loops,
// harnesses that forbid hipMalloc). The split-K accumulators, which
// exl3_linear_forward takes from the caller (its counters argument), live in a
// file-scope device array instead. Each GPU holds its own copy of the array at
// its own address for the life of the process; the address is looked up once
// per device and only that pointer is ever handed to a kernel (the array's name
// is a host-side stand-in, not a device address).
namespace exl3 {

constexpr size_t kStaticPartialBytes = (size_t)16 << 20;  // fp32 partial rows (large launches)
constexpr size_t kStaticCounterBytes = (size_t)16 << 20;  // 64-bit accumulators / group counters
constexpr size_t kStaticScratchBytes = kStaticPartialBytes + kStaticCounterBytes;
constexpr int kStaticMaxDevices = 64;

__global__ void static_zero_kernel(int32_t* p, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0;
}

}  // namespace exl3

static __device__ __align__(256) unsigned char scratch[exl3::kStaticScratchBytes];

namespace exl3 {

// Device address of this GPU's copy of `scratch`, resolved on first use with that
// device current. The counter half is cleared once by a fill kernel on `stream`, and the
// address is published only after that fill has completed (a stream synchronisation:
// it allocates nothing), so a later first call on another stream cannot overtake it.
// The first use on a device must not happen under stream capture (the fill and the
// synchronisation cannot be captured): such a call is refused with EXL3_E_UNSUPPORTED
// and nothing is launched; one eager call beforehand is enough.
static unsigned char* g_static_ptrs[kStaticMaxDevices];  // zero-initialised; one slot per device
static std::mutex g_static_lock;

static int static_scratch(hipStream_t stream, unsigned char** out) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kStaticMaxDevices)
        return EXL3_E_LAUNCH;
    std::lock_guard<std::mutex> guard(g_static_lock);
    if (!g_static_ptrs[dev]) {
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(stream, &capturing) != hipSuccess ||
            capturing != hipStreamCaptureStatusNone) {
            (void)hipGetLastError();
            return EXL3_E_UNSUPPORTED;
        }
        void* p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return EXL3_E_LAUNCH;
        const int n_ints = (int)(kStaticCounterBytes / sizeof(int32_t));
        static_zero_kernel<<<dim3((unsigned)((n_ints + 255) / 256)), dim3(256), 0, stream>>>(
            reinterpret_cast<int32_t*>(static_cast<unsigned char*>(p) + kStaticPartialBytes), n_ints);
        if (int rc = launch_status()) return rc;
        if (hipStreamSynchronize(stream) != hipSuccess) return EXL3_E_LAUNCH;
        g_static_ptrs[dev] = static_cast<unsigned char*>(p);
    }
    *out = g_static_ptrs[dev];
    return EXL3_OK;
}

// Status word of the static array: the last int of the counter half (static_need keeps
// the accumulators out of the last eight bytes).
static int* static_status_word(unsigned char* base) {
    return reinterpret_cast<int*>(base + kStaticScratchBytes) - 1;
}

}  // namespace exl3

EXL3_EXPORT size_t exl3_linear_static_scratch_bytes(void) { return exl3::kStaticPartialBytes; }

namespace exl3 {

// What a launch with this plan keeps in the two halves of the array: fp32 partial rows
// and group counters, or the accumulators (which live in the counter half).
struct StaticNeed {
    size_t partial_bytes, counter_bytes;
    size_t larger() const { return partial_bytes > counter_bytes ? partial_bytes : counter_bytes; }
};
static StaticNeed static_need(int rows, int out_features, GemvPlan plan) {
    const int n_groups = out_features / 128;
    if (linear_small_uses_atomics(rows, n_groups, plan))
        return {0, linear_small_counter_ints(rows, out_features) * sizeof(int32_t)};
    return {(size_t)plan.n_partials() * rows * out_features * sizeof(float),
            (size_t)n_groups * sizeof(int32_t)};
}

}  // namespace exl3

EXL3_EXPORT size_t exl3_linear_static_need_bytes(int rows, int in_features, int out_features) {
    using namespace exl3;
    if (rows < 1 || rows > kLinearSmallMaxRows || in_features < 128 || out_features < 128) return 0;
    // the launch plan depends on K (deeper splits from K = 5 on): the larger of the two
    size_t need = 0;
    for (int K : {4, 8}) {
        const GemvPlan plan = plan_linear_small_launch(rows, in_features / 16, out_features / 128, K);
        const size_t n = static_need(rows, out_features, plan).larger();
        if (n > need) need = n;
    }
    return need;
}

EXL3_EXPORT int exl3_linear_forward_static(const uint16_t* x, int rows, const uint16_t* trellis,
                                           int in_tiles, int out_tiles, int K, int cb,
                                           const uint16_t* suh, int n_sub, const int32_t* group_sub,
                                           const uint16_t* svh, const uint16_t* bias, uint16_t* y,
                                           void* stream) {
    using namespace exl3;
    if (int rc = check_k_cb(K, cb)) return rc;
    if (!x || !trellis || !y) return EXL3_E_NULL_POINTER;
    if (rows < 1 || in_tiles < 8 || out_tiles < 8 || in_tiles % 8 || out_tiles % 8 || n_sub < 1)
        return EXL3_E_BAD_SHAPE;
    if (rows > kLinearSmallMaxRows) return EXL3_E_UNSUPPORTED;  // only the one-launch kernel
    if (exact_weights()) return EXL3_E_UNSUPPORTED;  // the chain that rounds the weights needs a workspace
    if (n_sub > 1 && (!group_sub || !suh)) return EXL3_E_BAD_INDEX;
    const int n_groups = out_tiles / 8;
    const GemvPlan plan = plan_linear_small_launch(rows, in_tiles, n_groups, K);
    const StaticNeed need = static_need(rows, out_tiles * 16, plan);
    if (need.partial_bytes > kStaticPartialBytes || need.counter_bytes > kStaticCounterBytes - 8)
        return EXL3_E_STATIC_LIMIT;
    hipStream_t s = as_stream(stream);
    unsigned char* base = nullptr;
    if (int rc = static_scratch(s, &base)) return rc;
    return launch_linear_small(x, rows, trellis, in_tiles, out_tiles, K, cb, suh, n_sub, group_sub,
                               svh, bias, y, reinterpret_cast<float*>(base),
                               reinterpret_cast<int*>(base + kStaticPartialBytes), plan, s,
                               static_status_word(base));
}

// Whether a finishing workgroup of an accumulator reduction gave up on this counters
// array since it was last zeroed. Waits for `stream`, then reads the status word.
EXL3_EXPORT int exl3_counters_status(const int32_t* counters, size_t counters_len, void* stream) {
    using namespace exl3;
    hipStream_t s = as_stream(stream);
    const int* word = nullptr;
    if (counters) {
        if (counters_len < 2) return EXL3_E_BAD_SHAPE;
        word = counters + (counters_len - 1);
    } else {
        int dev = -1;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kStaticMaxDevices)
            return EXL3_E_LAUNCH;
        std::lock_guard<std::mutex> guard(g_static_lock);
        if (!g_static_ptrs[dev]) return EXL3_OK;  // never used on this device
        word = static_status_word(g_static_ptrs[dev]);
    }
    int host = 0;
    if (hipMemcpyAsync(&host, word, sizeof(int), hipMemcpyDeviceToHost, s) != hipSuccess ||
        hipStreamSynchronize(s) != hipSuccess)
        return EXL3_E_LAUNCH;
    return host ? EXL3_E_INCOMPLETE : EXL3_OK;
}
