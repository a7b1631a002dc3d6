/*
 * CPU oracle for the EXL3 quantized-linear path.
 *
 * TEST INFRASTRUCTURE ONLY. This file is a plain-C restatement of the
 * reference's numpy codec (the modules under ponyexl3/ref). It exists so the HIP kernels can
 * be checked against it and so a CPU baseline can be timed. Nothing in the
 * shipped package links, loads or calls it; only tests/, the smoke check and
 * the cpu_baseline leg of bench.py do.
 *
 * Each function cites the reference lines it follows. Parity status of every
 * function is listed at the end of this header.
 *
 * Conventions
 *   - fp16 values travel as uint16_t bit patterns; all fp16 roundings are
 *     round-to-nearest-even done in software (no _Float16 dependency).
 *   - trellis is uint16 [in_tiles][out_tiles][16*K], little-endian host.
 *   - W_inner is fp16 [in][out] row-major (in = 16*in_tiles).
 *
 * Parity pins (see tests/test_oracle_*.py):
 *   exl3o_decode_cw        pinned: full 65536-entry tables x 3 codebooks written
 *                          by the reference (tests/golden), closed form
 *                          c ^ (a & b), hand-derived known answers.
 *   exl3o_unpack_tile      pinned: reference-written unpacked tiles K=1..8
 *                          (tests/golden), independent two-lap sliding-window
 *                          model, shift consistency, all-zero / all-one tiles.
 *   exl3o_pack_tile        pinned: round trip through exl3o_unpack_tile and the
 *                          reference-written packed tiles.
 *   exl3o_perm             pinned: closed form, bijection, reference table.
 *   exl3o_decode_trellis   pinned: reference-decoded small layers per (K, cb).
 *   exl3o_hadamard128      pinned: scipy.linalg.hadamard dense product,
 *                          involution, Parseval.
 *   exl3o_linear_forward   pinned: reference forward outputs on small layers
 *                          (tolerance: the reference sums in BLAS order),
 *                          public-weight identity.
 *   MoE expert chain       (moe_experts_forward / glu in exl3_oracle.py) composition
 *                          of the pinned linear forward with the GLU. The reference
 *                          has no CPU twin of the chain (only Metal kernels) and so
 *                          no vectors; it is pinned by what the mathematics fixes:
 *                          SiLU and tanh-GELU against their closed forms in float64,
 *                          and the chain against dense public-weight products
 *                          y = (act(x Wg) * (x Wu)) Wd per expert, with wrong expert,
 *                          exchanged gate/up and missing activation as failing cases.
 *   exl3o_quantize_tile_exact
 *                          exact Viterbi over the bitshift trellis
 *                          (convert/reference_search.py). Pinned: states and
 *                          decoded values written by the reference's
 *                          quantize_tile_reference for six (K, codebook) cases
 *                          (tests/golden/search_exact.npz, bit-exact, closing
 *                          passes and tie-breaking included); brute force over
 *                          every path of a short trellis; recovery of exactly
 *                          representable tiles; chain validity of the states.
 *   exl3o_quantize_tiles_search
 *                          the production search kernel's arithmetic
 *                          (convert/metal_search.py:63-196: compressed states,
 *                          fp16 cost storage, warm-up pass + one pinned pass).
 *                          Pinned by the same assertions plus the reference's
 *                          quality bound against the exact search (mse <= 1.10 x).
 *                          Its bit-for-bit agreement with the Metal kernel itself
 *                          cannot be checked here (no Metal): "parity unpinned"
 *                          for the exact path chosen among near-ties.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define EXL3O_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------ fp16 */

static double h2d(uint16_t h) {
    uint32_t sign = (h >> 15) & 1u, exp = (h >> 10) & 0x1Fu, man = h & 0x3FFu;
    double v;
    if (exp == 0) {
        v = ldexp((double)man, -24);
    } else if (exp == 31) {
        v = man ? NAN : INFINITY;
    } else {
        v = ldexp((double)(man | 0x400u), (int)exp - 25);
    }
    return sign ? -v : v;
}

/* double -> fp16, one rounding, nearest-even. */
static uint16_t d2h(double d) {
    uint64_t b;
    memcpy(&b, &d, 8);
    uint16_t sign = (uint16_t)((b >> 48) & 0x8000u);
    int64_t bexp = (int64_t)((b >> 52) & 0x7FF);
    uint64_t man = b & ((1ULL << 52) - 1);
    if (bexp == 0x7FF) return (uint16_t)(sign | 0x7C00u | (man ? 0x200u : 0u));
    if (bexp == 0) return sign; /* zero or double-subnormal: far below half range */
    int e = (int)bexp - 1023;
    if (e > 15) return (uint16_t)(sign | 0x7C00u);
    man |= 1ULL << 52;
    int shift = (e >= -14) ? 42 : 42 + (-14 - e);
    if (shift > 63) return sign;
    uint64_t q = man >> shift;
    uint64_t rem = man & ((1ULL << shift) - 1);
    uint64_t halfway = 1ULL << (shift - 1);
    if (rem > halfway || (rem == halfway && (q & 1))) q++;
    if (e >= -14) {
        uint32_t r = ((uint32_t)(e + 15) << 10) + (uint32_t)(q - 1024);
        if (r >= 0x7C00u) return (uint16_t)(sign | 0x7C00u);
        return (uint16_t)(sign | r);
    }
    return (uint16_t)(sign | (uint16_t)q);
}

static float h2f(uint16_t h) { return (float)h2d(h); }
static uint16_t f2h(float f) { return d2h((double)f); }

EXL3O_API void exl3o_half_to_float(const uint16_t *h, float *f, size_t n) {
    for (size_t i = 0; i < n; i++) f[i] = h2f(h[i]);
}
EXL3O_API void exl3o_float_to_half(const float *f, uint16_t *h, size_t n) {
    for (size_t i = 0; i < n; i++) h[i] = f2h(f[i]);
}
EXL3O_API void exl3o_double_to_half(const double *f, uint16_t *h, size_t n) {
    for (size_t i = 0; i < n; i++) h[i] = d2h(f[i]);
}

/* -------------------------------------------------------------- codebook */

/* ref/codebook.py:66-91 decode_3inst; constants :16-20.
 * cb: 0 DEFAULT (3INST), 1 MCG, 2 MUL1 (ref/codebook.py:9-12). */
EXL3O_API uint16_t exl3o_decode_cw(uint32_t cw, int cb) {
    uint32_t x = cw & 0xFFFFu;
    if (cb == 0 || cb == 1) {
        if (cb == 0)
            x = x * 89226354u + 64248484u; /* :76 */
        else
            x = x * 0xCBAC1FEDu; /* :81 */
        /* lop3 imm 0x6A == c ^ (a & b): ref/codebook.py:23-42 */
        x = (x & 0x8FFF8FFFu) ^ 0x3B603B60u;
        /* one fp16 add of the two halves: ref/codebook.py:45-51. The exact
         * sum of two fp16 values fits a double, so d2h rounds once. */
        return d2h(h2d((uint16_t)(x & 0xFFFFu)) + h2d((uint16_t)(x >> 16)));
    }
    /* MUL1: ref/codebook.py:85-89, vabsdiff4 against 0 = byte sum (:54-63) */
    x = x * 0x83DCD12Du;
    uint32_t s = 0x6400u + (x & 0xFF) + ((x >> 8) & 0xFF) + ((x >> 16) & 0xFF) + (x >> 24);
    double h = h2d((uint16_t)(s & 0xFFFFu));
    /* float(h)*float(K_INV)+float(K_BIAS) in double, then one cast to fp16;
     * the product has <= 22 significant bits so the double expression is exact. */
    return d2h(h * h2d(0x1EEE) + h2d(0xC931));
}

EXL3O_API void exl3o_decode_table(int cb, uint16_t *out65536) {
    for (uint32_t c = 0; c < 65536u; c++) out65536[c] = exl3o_decode_cw(c, cb);
}

/* --------------------------------------------------------------- trellis */

/* ref/trellis.py:105-141 unpack_trellis_tile (funnel-shift formulation). */
EXL3O_API int exl3o_unpack_tile(const uint16_t *packed, int k, uint16_t *cw256) {
    if (k < 1 || k > 8) return -1;
    const int n_words = 8 * k; /* uint32 words per tile: (k*256)/32 */
    uint32_t words[64];
    memcpy(words, packed, (size_t)n_words * 4); /* .view(np.uint32), LE host */
    for (int t = 0; t < 128; t++) {
        int b0 = t * 2 * k + k - 16 + 256 * k;
        int b2 = b0 + k + 16;
        int i0 = b0 / 32;
        int i1 = (b2 - 1) / 32;
        int s1 = (i1 + 1) * 32 - b2;
        uint64_t a = words[i0 % n_words];
        uint64_t b = words[i1 % n_words];
        uint32_t w1 = (uint32_t)(((a << 32) | b) >> s1); /* _funnel_shift_r :8-10 */
        cw256[2 * t] = (uint16_t)((w1 >> k) & 0xFFFFu);
        cw256[2 * t + 1] = (uint16_t)(w1 & 0xFFFFu);
    }
    return 0;
}

/* ref/trellis.py:13-49 pack_trellis_tile (test helper: the encoder side). */
EXL3O_API int exl3o_pack_tile(const uint16_t *encoded256, int k, uint16_t *packed) {
    if (k < 1 || k > 8) return -1;
    const int packed_size = 16 * k;
    memset(packed, 0, (size_t)packed_size * 2);
    for (int t = 0; t < 16; t++) {
        int i = 16 * t, j = k * t;
        uint32_t buf = 0;
        int bit_pos = 32;
        for (int n = 0; n < 16; n++) {
            uint32_t v = encoded256[i] & ((1u << k) - 1u);
            bit_pos -= k;
            buf |= v << bit_pos;
            if (bit_pos <= 16) {
                packed[j] = (uint16_t)(buf >> 16);
                buf <<= 16;
                bit_pos += 16;
                j++;
            }
            i++;
        }
    }
    for (int w = 0; w < packed_size; w += 2) { /* SWAP16 per uint32 :47-48 */
        uint16_t t0 = packed[w];
        packed[w] = packed[w + 1];
        packed[w + 1] = t0;
    }
    return 0;
}

/* ------------------------------------------------------------------ perm */

/* ref/perm.py:8-25 tensor_core_perm: kernel-order index i lands at row-major
 * position perm[i] (ref/perm.py:36-40: out[p] = values[inv[p]]). */
EXL3O_API void exl3o_perm(int32_t *perm256) {
    for (int t = 0; t < 32; t++) {
        int r0 = (t % 4) * 2, c0 = t / 4;
        int rows[4] = {r0, r0 + 1, r0 + 8, r0 + 9};
        for (int j = 0; j < 8; j++) perm256[t * 8 + j] = rows[j % 4] * 16 + c0 + 8 * (j / 4);
    }
}

/* ---------------------------------------------------------------- decode */

/* ref/decode.py:20-29 decode_packed_tile -> row-major 16x16 fp16. */
EXL3O_API int exl3o_decode_tile(const uint16_t *packed, int k, int cb, uint16_t *tile256) {
    uint16_t cw[256];
    int32_t perm[256];
    if (exl3o_unpack_tile(packed, k, cw)) return -1;
    exl3o_perm(perm);
    for (int i = 0; i < 256; i++) tile256[perm[i]] = exl3o_decode_cw(cw[i], cb);
    return 0;
}

/* ref/decode.py:32-81 decode_packed_trellis with a tile-column slice
 * [tn_offset, tn_offset+tn_count). Output fp16 [16*in_tiles][16*tn_count].
 * Uses a 65536-entry table built from exl3o_decode_cw (same values). */
EXL3O_API int exl3o_decode_trellis(const uint16_t *trellis, int in_tiles, int out_tiles, int k,
                                   int cb, int tn_offset, int tn_count, uint16_t *w_out) {
    if (k < 1 || k > 8 || cb < 0 || cb > 2) return -1;
    if (tn_offset < 0 || tn_count < 0 || tn_offset + tn_count > out_tiles) return -2;
    uint16_t *table = (uint16_t *)malloc(65536 * 2);
    if (!table) return -3;
    exl3o_decode_table(cb, table);
    int32_t perm[256];
    exl3o_perm(perm);
    const size_t tile_u16 = (size_t)16 * k;
    const size_t ld = (size_t)16 * tn_count;
#pragma omp parallel for schedule(static)
    for (int tk = 0; tk < in_tiles; tk++) {
        uint16_t cw[256];
        for (int tn = 0; tn < tn_count; tn++) {
            const uint16_t *p = trellis + ((size_t)tk * out_tiles + tn_offset + tn) * tile_u16;
            exl3o_unpack_tile(p, k, cw);
            for (int i = 0; i < 256; i++) {
                int r = perm[i] >> 4, c = perm[i] & 15;
                w_out[((size_t)tk * 16 + r) * ld + (size_t)tn * 16 + c] = table[cw[i]];
            }
        }
    }
    free(table);
    return 0;
}

/* -------------------------------------------------------------- hadamard */

/* ref/hadamard.py:50-80 had_r_128 on fp32 rows: per 128-wide block
 * block = x * pre; block = block @ (H128 / sqrt(128)); block *= post.
 * The reference multiplies by a dense fp32 matrix whose entries are
 * +-float32(1/sqrt(128)); here the products are summed in double and rounded to
 * fp32 once per output, which is within 1 fp32 ulp of any BLAS summation order.
 * pre/post are fp16 bit patterns or NULL. */
EXL3O_API int exl3o_hadamard128(const float *x, int rows, int n, const uint16_t *pre,
                                const uint16_t *post, float *out) {
    if (n % 128) return -1;
    const float hs = (float)(1.0 / sqrt(128.0)); /* HAD_SCALE cast to fp32 (:26-27) */
#pragma omp parallel for schedule(static)
    for (int r = 0; r < rows; r++) {
        double buf[128], tmp[128];
        for (int j0 = 0; j0 < n; j0 += 128) {
            for (int i = 0; i < 128; i++) {
                float v = x[(size_t)r * n + j0 + i];
                if (pre) v = v * h2f(pre[j0 + i]); /* fp32 multiply (:74-75) */
                buf[i] = (double)v;
            }
            /* fast Walsh-Hadamard in natural (Sylvester) order, exact in double */
            for (int len = 1; len < 128; len <<= 1) {
                for (int i = 0; i < 128; i += len << 1)
                    for (int j = i; j < i + len; j++) {
                        double a = buf[j], b = buf[j + len];
                        tmp[j] = a + b;
                        tmp[j + len] = a - b;
                    }
                memcpy(buf, tmp, sizeof buf);
            }
            for (int i = 0; i < 128; i++) {
                float v = (float)(buf[i] * (double)hs);
                if (post) v = v * h2f(post[j0 + i]); /* (:77-78) */
                out[(size_t)r * n + j0 + i] = v;
            }
        }
    }
    return 0;
}

/* --------------------------------------------------------------- forward */

/* ref/forward.py:14-49 linear_forward_reconstruct.
 * x fp16 [rows][in]; suh fp16[in] or NULL; svh fp16[out] or NULL; bias fp16[out]
 * or NULL; w_inner fp16 [in][out] may be passed pre-decoded (else NULL and it is
 * decoded here). y fp16 [rows][out]. Optional taps: xh_out fp16 [rows][in],
 * yraw_out fp16 [rows][out] (the value cast at ref/forward.py:41). */
EXL3O_API int exl3o_linear_forward(const uint16_t *trellis, int in_tiles, int out_tiles, int k,
                                   int cb, const uint16_t *suh, const uint16_t *svh,
                                   const uint16_t *bias, const uint16_t *w_inner,
                                   const uint16_t *x, int rows, uint16_t *y, uint16_t *xh_out,
                                   uint16_t *yraw_out) {
    const int in = in_tiles * 16, out = out_tiles * 16;
    if (in % 128 || out % 128) return -1; /* ref/hadamard.py:67-68 */
    int rc = 0;
    uint16_t *w_own = NULL;
    float *xf = (float *)malloc((size_t)rows * in * 4);
    float *xh = (float *)malloc((size_t)rows * in * 4);
    float *yf = (float *)malloc((size_t)rows * out * 4);
    float *yh = (float *)malloc((size_t)rows * out * 4);
    if (!xf || !xh || !yf || !yh) { rc = -3; goto done; }
    if (!w_inner) {
        w_own = (uint16_t *)malloc((size_t)in * out * 2);
        if (!w_own) { rc = -3; goto done; }
        rc = exl3o_decode_trellis(trellis, in_tiles, out_tiles, k, cb, 0, out_tiles, w_own);
        if (rc) goto done;
        w_inner = w_own;
    }
    for (size_t i = 0; i < (size_t)rows * in; i++) xf[i] = h2f(x[i]);
    exl3o_hadamard128(xf, rows, in, suh, NULL, xh);
    /* .astype(fp16) :34 then back to fp32 :41 */
    for (size_t i = 0; i < (size_t)rows * in; i++) {
        uint16_t h = f2h(xh[i]);
        if (xh_out) xh_out[i] = h;
        xh[i] = h2f(h);
    }
    /* y = xh.f32 @ w.f32 (:41): summed in double, rounded to fp32, then fp16 */
#pragma omp parallel
    {
        double *acc = (double *)malloc((size_t)out * sizeof(double));
        float *wrow = (float *)malloc((size_t)out * sizeof(float));
#pragma omp for schedule(static)
        for (int r = 0; r < rows; r++) {
            for (int c = 0; c < out; c++) acc[c] = 0.0;
            for (int i = 0; i < in; i++) {
                const double xv = (double)xh[(size_t)r * in + i];
                const uint16_t *wr = w_inner + (size_t)i * out;
                for (int c = 0; c < out; c++) wrow[c] = h2f(wr[c]);
                for (int c = 0; c < out; c++) acc[c] += xv * (double)wrow[c];
            }
            for (int c = 0; c < out; c++) {
                uint16_t h = f2h((float)acc[c]);
                if (yraw_out) yraw_out[(size_t)r * out + c] = h;
                yf[(size_t)r * out + c] = h2f(h);
            }
        }
        free(acc);
        free(wrow);
    }
    exl3o_hadamard128(yf, rows, out, NULL, svh, yh);
    for (size_t i = 0; i < (size_t)rows * out; i++) {
        uint16_t h = f2h(yh[i]); /* :42 */
        if (bias) h = d2h(h2d(h) + h2d(bias[i % (size_t)out])); /* fp16 add :44-45 */
        y[i] = h;
    }
done:
    free(xf); free(xh); free(yf); free(yh); free(w_own);
    return rc;
}

/* Single-row matvec against a decoded table, streaming the trellis: the shape
 * of work a CPU would do at batch 1 (decode + Hadamard-128 + matvec) without
 * materialising W. Same arithmetic as exl3o_linear_forward with rows = 1 except
 * that partial sums are kept per thread over disjoint tile-row ranges and added
 * in thread order (double accumulation; fp32/fp16 casts at the same points).
 * Used by the cpu_baseline timing. */
EXL3O_API int exl3o_linear_forward_bs1(const uint16_t *trellis, int in_tiles, int out_tiles, int k,
                                       int cb, const uint16_t *suh, const uint16_t *svh,
                                       const uint16_t *x, uint16_t *y) {
    const int in = in_tiles * 16, out = out_tiles * 16;
    if (in % 128 || out % 128) return -1;
    if (k < 1 || k > 8 || cb < 0 || cb > 2) return -1;
    float *xf = (float *)malloc((size_t)in * 4);
    float *xh = (float *)malloc((size_t)in * 4);
    float *yf = (float *)malloc((size_t)out * 4);
    float *yh = (float *)malloc((size_t)out * 4);
    float *table = (float *)malloc(65536 * 4);
    int nthreads = 1;
#ifdef _OPENMP
    nthreads = omp_get_max_threads();
#endif
    double *part = (double *)calloc((size_t)nthreads * out, sizeof(double));
    if (!xf || !xh || !yf || !yh || !table || !part) return -3;
    for (uint32_t c = 0; c < 65536u; c++) table[c] = h2f(exl3o_decode_cw(c, cb));
    int32_t perm[256];
    exl3o_perm(perm);
    for (int i = 0; i < in; i++) xf[i] = h2f(x[i]);
    exl3o_hadamard128(xf, 1, in, suh, NULL, xh);
    for (int i = 0; i < in; i++) xh[i] = h2f(f2h(xh[i]));
    const size_t tile_u16 = (size_t)16 * k;
#pragma omp parallel
    {
        int tid = 0;
#ifdef _OPENMP
        tid = omp_get_thread_num();
#endif
        double *acc = part + (size_t)tid * out;
        uint16_t cw[256];
#pragma omp for schedule(static)
        for (int tk = 0; tk < in_tiles; tk++) {
            for (int tn = 0; tn < out_tiles; tn++) {
                exl3o_unpack_tile(trellis + ((size_t)tk * out_tiles + tn) * tile_u16, k, cw);
                for (int i = 0; i < 256; i++) {
                    int r = perm[i] >> 4, c = perm[i] & 15;
                    acc[tn * 16 + c] += (double)xh[tk * 16 + r] * (double)table[cw[i]];
                }
            }
        }
    }
    for (int c = 0; c < out; c++) {
        double s = 0.0;
        for (int t = 0; t < nthreads; t++) s += part[(size_t)t * out + c];
        yf[c] = h2f(f2h((float)s));
    }
    exl3o_hadamard128(yf, 1, out, NULL, svh, yh);
    for (int c = 0; c < out; c++) y[c] = f2h(yh[c]);
    free(xf); free(xh); free(yf); free(yh); free(table); free(part);
    return 0;
}

/* ---------------------------------------------------------------- search */

static float *decode_lut_f32(int cb) {
    float *lut = (float *)malloc(65536 * sizeof(float));
    if (lut)
        for (uint32_t c = 0; c < 65536u; c++) lut[c] = h2f(exl3o_decode_cw(c, cb));
    return lut;
}

/* convert/reference_search.py:32-56 _forward: one Viterbi pass over 2^16 states
 * with float64 path costs. s' = ((s << K) | fresh) & 0xFFFF, so the predecessors
 * of s' are (s' >> K) | (j << (16-K)), j = 0..2^K-1; ties keep the lowest j
 * (numpy argmin). init_state < 0: free start. n_steps = 256 in the reference; the
 * parameter only exists so a short trellis can be brute-forced in the tests. */
static int viterbi_forward(const float *w, int n_steps, int k, const float *lut, int init_state,
                           uint16_t *back, double *cost, double *next) {
    const int kk = 1 << k;
    for (int s = 0; s < 65536; s++) cost[s] = init_state < 0 ? 0.0 : 1e30;
    if (init_state >= 0) cost[init_state] = 0.0;
    for (int t = 0; t < n_steps; t++) {
        const double wt = (double)w[t];
#pragma omp parallel for schedule(static)
        for (int s = 0; s < 65536; s++) {
            uint32_t best_p = (uint32_t)s >> k;
            double best = cost[best_p];
            for (int j = 1; j < kk; j++) {
                const uint32_t p = ((uint32_t)s >> k) | ((uint32_t)j << (16 - k));
                if (cost[p] < best) {
                    best = cost[p];
                    best_p = p;
                }
            }
            back[(size_t)t * 65536 + s] = (uint16_t)best_p;
            const double d = (double)lut[s] - wt;
            next[s] = best + d * d;
        }
        memcpy(cost, next, 65536 * sizeof(double));
    }
    int fin = 0;
    for (int s = 1; s < 65536; s++)
        if (cost[s] < cost[fin]) fin = s;
    return fin;
}

/* convert/reference_search.py:59-87 quantize_tile_reference: free pass, then up
 * to max_pins passes pinned to the previous pass's last state until the path
 * closes (pre-state of step 0 == states[n-1] == pin). */
EXL3O_API int exl3o_quantize_tile_exact(const float *w, int n_steps, int k, int cb, int max_pins,
                                        uint16_t *states, float *decoded) {
    if (k < 1 || k > 8 || cb < 0 || cb > 2 || n_steps < 1) return -1;
    float *lut = decode_lut_f32(cb);
    uint16_t *back = (uint16_t *)malloc((size_t)n_steps * 65536 * sizeof(uint16_t));
    double *cost = (double *)malloc(2 * 65536 * sizeof(double));
    if (!lut || !back || !cost) {
        free(lut); free(back); free(cost);
        return -2;
    }
    int pin = -1;
    for (int pass = 0; pass <= max_pins; pass++) {
        int s = viterbi_forward(w, n_steps, k, lut, pin, back, cost, cost + 65536);
        for (int t = n_steps - 1; t >= 0; t--) {
            states[t] = (uint16_t)s;
            s = back[(size_t)t * 65536 + s];
        }
        const int last = states[n_steps - 1];
        if (pass > 0 && s == pin && last == pin) break;
        pin = last;
    }
    for (int t = 0; t < n_steps; t++) decoded[t] = lut[states[t]];
    free(lut); free(back); free(cost);
    return 0;
}

/* convert/metal_search.py:63-196, one tile per call of the inner body.
 * Compressed state e = the newest 16-K bits; the candidate codeword for
 * (fresh, e) is (fresh << (16-K)) | e with predecessor cw >> K. Costs are kept
 * as fp16 between steps (:128,153), arithmetic is fp32 with one fma (:147),
 * clamped to 65504; ties keep the lowest fresh (strict <, :123,149). Pass 0
 * starts at position 128, runs once around and backtracks to the state before
 * position 0 (:176-190); pass 1 starts at 0 pinned to it and must end in it. */
EXL3O_API int exl3o_quantize_tiles_search(const float *tiles, int n_tiles, int k, int cb,
                                          float *q_tiles, uint16_t *indices) {
    if (k < 2 || k > 8 || cb < 0 || cb > 2 || n_tiles < 0) return -1;
    const int kr = 16 - k, edges = 1 << kr, kk = 1 << k;
    const float H_INF = 65504.0f;
    float *lut = decode_lut_f32(cb);
    if (!lut) return -2;
    int rc = 0;
#pragma omp parallel for schedule(dynamic)
    for (int tile = 0; tile < n_tiles; tile++) {
        uint16_t *edge_ptr = (uint16_t *)malloc((size_t)256 * edges * sizeof(uint16_t));
        uint16_t *costs = (uint16_t *)malloc((size_t)2 * edges * sizeof(uint16_t));
        if (!edge_ptr || !costs) {
            rc = -2;
            free(edge_ptr); free(costs);
            continue;
        }
        const float *in_tile = tiles + (size_t)tile * 256;
        float *out_tile = q_tiles + (size_t)tile * 256;
        uint16_t *out_idx = indices + (size_t)tile * 256;
        uint32_t pin = 0;
        int pinned = 0;
        for (int pass = 0; pass < 2; pass++) {
            int curr = 0;
            const int roll = pass == 0 ? 128 : 0;
            for (int step = 0; step < 256; step++) {
                const int ri = (step + roll) & 255;
                const int prev_buf = curr;
                if (step > 0) curr = 1 - curr;
                const float target = in_tile[ri];
                for (int e = 0; e < edges; e++) {
                    float best = H_INF;
                    uint32_t best_pred = 0;
                    for (int fresh = 0; fresh < kk; fresh++) {
                        const uint32_t cw = ((uint32_t)fresh << kr) | (uint32_t)e;
                        const uint32_t pred = cw >> k;
                        float err;
                        if (step == 0) {
                            if (pinned && pred != pin) {
                                err = H_INF;
                            } else {
                                const float dh = lut[cw] - target;
                                err = dh * dh;
                                if (err > H_INF) err = H_INF;
                            }
                        } else {
                            const float dh = lut[cw] - target;
                            err = fmaf(dh, dh, h2f(costs[(size_t)prev_buf * edges + pred]));
                            if (err > H_INF) err = H_INF;
                        }
                        if (err < best) {
                            best = err;
                            best_pred = pred;
                        }
                    }
                    costs[(size_t)curr * edges + e] = f2h(best);
                    if (pass == 1 || ri < 128) edge_ptr[(size_t)ri * edges + e] = (uint16_t)best_pred;
                }
            }
            uint32_t edge = pin;
            if (pass == 0) {
                float best = H_INF;
                edge = 0;
                for (int e = 0; e < edges; e++) {
                    const float v = h2f(costs[(size_t)curr * edges + e]);
                    if (v < best) {
                        best = v;
                        edge = (uint32_t)e;
                    }
                }
            }
            for (int step_i = 255; step_i >= 0; step_i--) {
                const int ri = (step_i + roll) & 255;
                const uint32_t prev = edge_ptr[(size_t)ri * edges + edge];
                const uint32_t state = ((prev << k) | edge) & 0xFFFFu;
                edge = prev;
                if (pass == 1) {
                    out_idx[ri] = (uint16_t)state;
                    out_tile[ri] = lut[state];
                } else if (ri == 0) {
                    break;
                }
            }
            pin = edge;
            pinned = 1;
        }
        free(edge_ptr); free(costs);
    }
    free(lut);
    return rc;
}

EXL3O_API int exl3o_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

EXL3O_API void exl3o_set_num_threads(int n) {
#ifdef _OPENMP
    if (n > 0) omp_set_num_threads(n);
#else
    (void)n;
#endif
}
