/*
 * rllama_oracle.c -- CPU restatement of rllama's per-token transformer forward path.
 *
 * TEST INFRASTRUCTURE ONLY (see rllama_oracle.h).  Build: oracle/Makefile
 *   gcc -O2 -mavx2 -mfma -mf16c -ffp-contract=off -fopenmp -shared -fPIC
 *
 * The reference is Rust (nightly) with un-vendored crates and cannot be compiled where this
 * file is built, so this restatement is pinned by independent checks instead of by a run of
 * the reference.  Which check pins which function (all under tests/):
 *
 *   f16 <-> f32 conversion          exhaustive 65,536-value round trip against numpy's IEEE half and
 *                                   against the F16C instructions; the reference's own property
 *                                   (tensor.rs:2881-2920: vector convert == half crate convert).
 *   hsum8 / dot8 lane order         hand-computed cases where fp32 rounding makes every other
 *                                   association give a different answer; scalar fmaf() re-derivation.
 *   matmul_transposed f32 / f16     naive triple loop in float64 at the reference's own tolerances
 *                                   (tensor.rs:2554-2856: 1e-5 f32, 1e-1 f16) and tighter ones.
 *   matmul seq-k, vector_matrix_mul naive float64 (tensor.rs:2749-2824 properties).
 *   rmsnorm, softmax, silu, RoPE,   textbook closed forms in float64 numpy; special cases (RoPE at pos 0
 *   freqs_cis, causal mask          is the identity, softmax of equal scores is 1/T, norm of a constant row).
 *   whole forward                   an independent float64 numpy LLaMA forward written with library
 *                                   matmuls; invariants (prefill(n) == prefill(n-1)+decode(1), zeroed wo/w2
 *                                   closed form, true_clone determinism).
 *   greedy sampler                  brute-force restatement in Python on small vocabularies.
 *   full sampler (candidates, pick) float64 closed form derived by hand from token_sampler.rs:99-159 (token 0 ends at exactly 0,
 *                                   nothing else is shifted), token-0-only penalty, NaN-last ordering on overflow, agreement with
 *                                   the greedy entry at top_k 1, frequency check of the cumulative walk over 20000 draws.
 *
 * parity unpinned (only a run of the real binary could pin them; none changes a tolerance-based check):
 *   - tie-break among exactly equal probabilities, greedy and full sampler alike (token_sampler.rs:131-145 uses sort_unstable_by);
 *   - whether LLVM folded powf(x, 2.0) to x*x in Tensor::pow (tensor.rs:537-547): at most 1 ulp per term,
 *     this file uses x*x;
 *   - num-complex's Complex::from_polar(1.0, t) == (cos t, sin t) (transformer.rs:880), taken from its docs.
 */
#include "rllama_oracle.h"

#include <immintrin.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>
#include <omp.h>

/* ------------------------------------------------------------------------------------------ */
/* f16 conversion                                                                              */
/* ------------------------------------------------------------------------------------------ */

uint16_t orc_f32_to_f16_bits(float v) {
    /* IEEE-754 binary32 -> binary16, round to nearest even, written with integer ops only. */
    uint32_t x;
    memcpy(&x, &v, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t absx = x & 0x7fffffffu;
    if (absx >= 0x7f800000u) { /* inf / nan */
        if (absx > 0x7f800000u) {
            return (uint16_t)(sign | 0x7e00u | ((absx >> 13) & 0x3ffu)); /* quiet nan, keep payload top bits */
        }
        return (uint16_t)(sign | 0x7c00u);
    }
    if (absx >= 0x477ff000u) { /* >= 65520 rounds to inf */
        return (uint16_t)(sign | 0x7c00u);
    }
    if (absx < 0x33000001u) { /* <= 2^-25 rounds to zero (2^-25 itself ties to even = 0) */
        return (uint16_t)sign;
    }
    int32_t exp = (int32_t)(absx >> 23) - 127;
    uint32_t mant = (absx & 0x7fffffu) | 0x800000u; /* 24 bits */
    uint32_t shift;
    uint32_t half_exp;
    if (exp < -14) { /* subnormal half */
        shift = (uint32_t)(13 + (-14 - exp));
        half_exp = 0;
    } else {
        shift = 13;
        half_exp = (uint32_t)(exp + 15);
    }
    uint32_t q = mant >> shift;
    uint32_t rem = mant & ((1u << shift) - 1u);
    uint32_t halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (q & 1u))) {
        q += 1;
    }
    uint32_t h;
    if (half_exp == 0) {
        h = q; /* q may reach 0x400 -> becomes smallest normal, which is the right encoding */
    } else {
        h = ((half_exp - 1) << 10) + q; /* q has the implicit bit at 0x400; carries roll into the exponent */
    }
    return (uint16_t)(sign | h);
}

float orc_f16_bits_to_f32(uint16_t h) {
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t mant = h & 0x3ffu;
    uint32_t x;
    if (exp == 0) {
        if (mant == 0) {
            x = sign;
        } else {
            int e = -1;
            do {
                mant <<= 1;
                e++;
            } while ((mant & 0x400u) == 0);
            x = sign | ((uint32_t)(127 - 15 - e) << 23) | ((mant & 0x3ffu) << 13);
        }
    } else if (exp == 31) {
        x = sign | 0x7f800000u | (mant << 13);
    } else {
        x = sign | ((exp + 127 - 15) << 23) | (mant << 13);
    }
    float f;
    memcpy(&f, &x, 4);
    return f;
}

uint16_t orc_f32_to_f16_hw(float v) { return _cvtss_sh(v, 0); }
float orc_f16_to_f32_hw(uint16_t h) { return _cvtsh_ss(h); }

void orc_f32_to_f16_array(const float *src, uint16_t *dst, size_t n) {
    size_t i = 0;
    for (; i + 8 <= n; i += 8) {
        __m128i h = _mm256_cvtps_ph(_mm256_loadu_ps(src + i), 0);
        _mm_storeu_si128((__m128i *)(dst + i), h);
    }
    for (; i < n; i++) dst[i] = _cvtss_sh(src[i], 0);
}

void orc_f16_to_f32_array(const uint16_t *src, float *dst, size_t n) {
    size_t i = 0;
    for (; i + 8 <= n; i += 8) {
        _mm256_storeu_ps(dst + i, _mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)(src + i))));
    }
    for (; i < n; i++) dst[i] = _cvtsh_ss(src[i]);
}

/* ------------------------------------------------------------------------------------------ */
/* dot8 and friends                                                                            */
/* ------------------------------------------------------------------------------------------ */

/* Sensitivity probe, off by default (orc_set_alt_order): with it on, the f16 projections sum their products in another,
 * equally valid fp32 order -- two sets of 8 lanes taking alternate blocks of 8, joined at the end, and the horizontal sum
 * taken left to right.  The values this produces are NOT the reference's; the switch exists to measure how far the
 * reference's own arithmetic moves under a reordering of its additions (the distance any other implementation can be
 * expected to stay within). */
static int g_alt_order = 0;
void orc_set_alt_order(int on) { g_alt_order = on ? 1 : 0; }

static inline float hsum8_alt(__m256 ymm) {
    float l[8];
    _mm256_storeu_ps(l, ymm);
    float t = l[0];
    for (int i = 1; i < 8; i++) t += l[i];
    return t;
}

/* Second probe, off by default (orc_set_exact_sums): every sum of products or of terms -- the dot products of the
 * projections, of the scores, of P.V and of the output head, the sum of squares of RMSNorm, the softmax denominator -- is
 * accumulated in float64 (products of f16 or f32 operands are exact in float64; the additions then carry a relative error
 * of 1e-16, nothing beside fp32's 6e-8) and rounded to f32 once.  Everything else is as in the reference's arithmetic: the
 * same f16 rounding points, the same f32 element-wise steps, the same libm calls.  The values are NOT the reference's:
 * they are what its arithmetic would give if no fp32 addition inside a sum rounded, i.e. the point that the reference and
 * any reordering of its additions scatter around.  Pinned by tests/test_oracle.py against math.fsum. */
static int g_exact = 0;
void orc_set_exact_sums(int on) { g_exact = on ? 1 : 0; }

static inline double hsum4d(__m256d v) {
    double l[4];
    _mm256_storeu_pd(l, v);
    return (l[0] + l[1]) + (l[2] + l[3]);
}

static double dotd_f32(const float *a, const float *b, int k) {
    __m256d s0 = _mm256_setzero_pd(), s1 = s0;
    int p = 0;
    for (; p + 8 <= k; p += 8) {
        __m256 av = _mm256_loadu_ps(a + p), bv = _mm256_loadu_ps(b + p);
        s0 = _mm256_fmadd_pd(_mm256_cvtps_pd(_mm256_castps256_ps128(av)), _mm256_cvtps_pd(_mm256_castps256_ps128(bv)), s0);
        s1 = _mm256_fmadd_pd(_mm256_cvtps_pd(_mm256_extractf128_ps(av, 1)), _mm256_cvtps_pd(_mm256_extractf128_ps(bv, 1)), s1);
    }
    double t = hsum4d(_mm256_add_pd(s0, s1));
    for (; p < k; p++) t += (double)a[p] * (double)b[p];
    return t;
}

static double dotd_f16(const uint16_t *a, const uint16_t *b, int k) {
    __m256d s0 = _mm256_setzero_pd(), s1 = s0;
    int p = 0;
    for (; p + 8 <= k; p += 8) {
        __m256 av = _mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)(a + p)));
        __m256 bv = _mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)(b + p)));
        s0 = _mm256_fmadd_pd(_mm256_cvtps_pd(_mm256_castps256_ps128(av)), _mm256_cvtps_pd(_mm256_castps256_ps128(bv)), s0);
        s1 = _mm256_fmadd_pd(_mm256_cvtps_pd(_mm256_extractf128_ps(av, 1)), _mm256_cvtps_pd(_mm256_extractf128_ps(bv, 1)), s1);
    }
    double t = hsum4d(_mm256_add_pd(s0, s1));
    for (; p < k; p++) t += (double)_cvtsh_ss(a[p]) * (double)_cvtsh_ss(b[p]);
    return t;
}

static inline float hsum8_v(__m256 ymm) {
    /* simd_support.rs:97-105, instruction for instruction */
    __m256 ymm2 = _mm256_permute2f128_ps(ymm, ymm, 1);
    ymm = _mm256_add_ps(ymm, ymm2);
    ymm = _mm256_hadd_ps(ymm, ymm);
    ymm = _mm256_hadd_ps(ymm, ymm);
    return _mm256_cvtss_f32(ymm);
}

float orc_hsum8(const float a[8]) { return hsum8_v(_mm256_loadu_ps(a)); }

float orc_dot8_f32(const float *a, const float *b, int k) {
    if (g_exact) return (float)dotd_f32(a, b, k);
    __m256 acc = _mm256_setzero_ps();
    int p = 0;
    for (; p + 8 <= k; p += 8) {
        acc = _mm256_fmadd_ps(_mm256_loadu_ps(a + p), _mm256_loadu_ps(b + p), acc);
    }
    if (p < k) { /* the reference reads zero padding past the last column (tensor.rs:192-222, 417-466) */
        float ta[8] = {0}, tb[8] = {0};
        for (int i = 0; p + i < k; i++) {
            ta[i] = a[p + i];
            tb[i] = b[p + i];
        }
        acc = _mm256_fmadd_ps(_mm256_loadu_ps(ta), _mm256_loadu_ps(tb), acc);
    }
    return hsum8_v(acc);
}

float orc_dot8_f32_scalar(const float *a, const float *b, int k) {
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int p = 0; p < k; p += 8) {
        for (int l = 0; l < 8; l++) {
            float av = (p + l < k) ? a[p + l] : 0.0f;
            float bv = (p + l < k) ? b[p + l] : 0.0f;
            acc[l] = fmaf(av, bv, acc[l]);
        }
    }
    float s04 = acc[0] + acc[4];
    float s15 = acc[1] + acc[5];
    float s26 = acc[2] + acc[6];
    float s37 = acc[3] + acc[7];
    float l = s04 + s15;
    float r = s26 + s37;
    return l + r;
}

static inline __m256 load8_f16(const uint16_t *p) { return _mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)p)); }

float orc_dot8_f16(const uint16_t *a, const uint16_t *b, int k) {
    if (g_exact) return (float)dotd_f16(a, b, k);
    __m256 acc = _mm256_setzero_ps();
    int p = 0;
    for (; p + 8 <= k; p += 8) {
        acc = _mm256_fmadd_ps(load8_f16(a + p), load8_f16(b + p), acc);
    }
    if (p < k) {
        uint16_t ta[8] = {0}, tb[8] = {0};
        for (int i = 0; p + i < k; i++) {
            ta[i] = a[p + i];
            tb[i] = b[p + i];
        }
        acc = _mm256_fmadd_ps(load8_f16(ta), load8_f16(tb), acc);
    }
    return hsum8_v(acc);
}

/* Four weight rows against one x row, sharing the x loads: the value per output is dot8. */
static inline void dot8x4_f16(const uint16_t *x, const uint16_t *w0, const uint16_t *w1, const uint16_t *w2,
                              const uint16_t *w3, int k, float out[4]) {
    if (g_exact) { /* not the reference's values: see orc_set_exact_sums */
        out[0] = (float)dotd_f16(x, w0, k);
        out[1] = (float)dotd_f16(x, w1, k);
        out[2] = (float)dotd_f16(x, w2, k);
        out[3] = (float)dotd_f16(x, w3, k);
        return;
    }
    __m256 a0 = _mm256_setzero_ps(), a1 = a0, a2 = a0, a3 = a0;
    int p = 0;
    if (g_alt_order) { /* not the reference's order: see orc_set_alt_order */
        __m256 b0 = a0, b1 = a0, b2 = a0, b3 = a0;
        for (; p + 16 <= k; p += 16) {
            __m256 xv = load8_f16(x + p), xw = load8_f16(x + p + 8);
            a0 = _mm256_fmadd_ps(xv, load8_f16(w0 + p), a0);
            a1 = _mm256_fmadd_ps(xv, load8_f16(w1 + p), a1);
            a2 = _mm256_fmadd_ps(xv, load8_f16(w2 + p), a2);
            a3 = _mm256_fmadd_ps(xv, load8_f16(w3 + p), a3);
            b0 = _mm256_fmadd_ps(xw, load8_f16(w0 + p + 8), b0);
            b1 = _mm256_fmadd_ps(xw, load8_f16(w1 + p + 8), b1);
            b2 = _mm256_fmadd_ps(xw, load8_f16(w2 + p + 8), b2);
            b3 = _mm256_fmadd_ps(xw, load8_f16(w3 + p + 8), b3);
        }
        for (; p < k; p++) { /* leftovers one by one into lane 0 */
            float xs = orc_f16_bits_to_f32(x[p]);
            float t[8] = {0};
            t[0] = xs * orc_f16_bits_to_f32(w0[p]); a0 = _mm256_add_ps(a0, _mm256_loadu_ps(t));
            t[0] = xs * orc_f16_bits_to_f32(w1[p]); a1 = _mm256_add_ps(a1, _mm256_loadu_ps(t));
            t[0] = xs * orc_f16_bits_to_f32(w2[p]); a2 = _mm256_add_ps(a2, _mm256_loadu_ps(t));
            t[0] = xs * orc_f16_bits_to_f32(w3[p]); a3 = _mm256_add_ps(a3, _mm256_loadu_ps(t));
        }
        out[0] = hsum8_alt(_mm256_add_ps(a0, b0));
        out[1] = hsum8_alt(_mm256_add_ps(a1, b1));
        out[2] = hsum8_alt(_mm256_add_ps(a2, b2));
        out[3] = hsum8_alt(_mm256_add_ps(a3, b3));
        return;
    }
    for (; p + 8 <= k; p += 8) {
        __m256 xv = load8_f16(x + p);
        a0 = _mm256_fmadd_ps(xv, load8_f16(w0 + p), a0);
        a1 = _mm256_fmadd_ps(xv, load8_f16(w1 + p), a1);
        a2 = _mm256_fmadd_ps(xv, load8_f16(w2 + p), a2);
        a3 = _mm256_fmadd_ps(xv, load8_f16(w3 + p), a3);
    }
    if (p < k) {
        uint16_t tx[8] = {0}, t0[8] = {0}, t1[8] = {0}, t2[8] = {0}, t3[8] = {0};
        for (int i = 0; p + i < k; i++) {
            tx[i] = x[p + i];
            t0[i] = w0[p + i];
            t1[i] = w1[p + i];
            t2[i] = w2[p + i];
            t3[i] = w3[p + i];
        }
        __m256 xv = load8_f16(tx);
        a0 = _mm256_fmadd_ps(xv, load8_f16(t0), a0);
        a1 = _mm256_fmadd_ps(xv, load8_f16(t1), a1);
        a2 = _mm256_fmadd_ps(xv, load8_f16(t2), a2);
        a3 = _mm256_fmadd_ps(xv, load8_f16(t3), a3);
    }
    out[0] = hsum8_v(a0);
    out[1] = hsum8_v(a1);
    out[2] = hsum8_v(a2);
    out[3] = hsum8_v(a3);
}

static inline void dot8x4_f32(const float *x, const float *w0, const float *w1, const float *w2, const float *w3,
                              int k, float out[4]) {
    if (g_exact) {
        out[0] = (float)dotd_f32(x, w0, k);
        out[1] = (float)dotd_f32(x, w1, k);
        out[2] = (float)dotd_f32(x, w2, k);
        out[3] = (float)dotd_f32(x, w3, k);
        return;
    }
    __m256 a0 = _mm256_setzero_ps(), a1 = a0, a2 = a0, a3 = a0;
    int p = 0;
    for (; p + 8 <= k; p += 8) {
        __m256 xv = _mm256_loadu_ps(x + p);
        a0 = _mm256_fmadd_ps(xv, _mm256_loadu_ps(w0 + p), a0);
        a1 = _mm256_fmadd_ps(xv, _mm256_loadu_ps(w1 + p), a1);
        a2 = _mm256_fmadd_ps(xv, _mm256_loadu_ps(w2 + p), a2);
        a3 = _mm256_fmadd_ps(xv, _mm256_loadu_ps(w3 + p), a3);
    }
    if (p < k) {
        float tx[8] = {0}, t0[8] = {0}, t1[8] = {0}, t2[8] = {0}, t3[8] = {0};
        for (int i = 0; p + i < k; i++) {
            tx[i] = x[p + i];
            t0[i] = w0[p + i];
            t1[i] = w1[p + i];
            t2[i] = w2[p + i];
            t3[i] = w3[p + i];
        }
        __m256 xv = _mm256_loadu_ps(tx);
        a0 = _mm256_fmadd_ps(xv, _mm256_loadu_ps(t0), a0);
        a1 = _mm256_fmadd_ps(xv, _mm256_loadu_ps(t1), a1);
        a2 = _mm256_fmadd_ps(xv, _mm256_loadu_ps(t2), a2);
        a3 = _mm256_fmadd_ps(xv, _mm256_loadu_ps(t3), a3);
    }
    out[0] = hsum8_v(a0);
    out[1] = hsum8_v(a1);
    out[2] = hsum8_v(a2);
    out[3] = hsum8_v(a3);
}

static int g_threads = 0;

void orc_set_threads(int n) {
    g_threads = n > 0 ? n : 0;
    if (g_threads > 0) omp_set_num_threads(g_threads);
}

int orc_get_threads(void) { return g_threads > 0 ? g_threads : omp_get_max_threads(); }

/* The reference hands 4x4 output tiles to threads round-robin (tensor.rs:1327-1340, 1520-1533); every
 * output element is produced by exactly one thread from start to finish, so the values do not depend on
 * the thread count.  Here the unit is a tile of 4 weight rows (all x rows), scheduled statically. */
void orc_matmul_transposed_f16(const uint16_t *x, int n_x, const uint16_t *w, int n_w, int k, uint16_t *out) {
    int tiles = (n_w + 3) / 4;
#pragma omp parallel for schedule(static)
    for (int t = 0; t < tiles; t++) {
        int c0 = t * 4;
        int nc = n_w - c0 < 4 ? n_w - c0 : 4;
        const uint16_t *w0 = w + (size_t)c0 * k;
        const uint16_t *w1 = nc > 1 ? w0 + k : w0;
        const uint16_t *w2 = nc > 2 ? w0 + 2 * (size_t)k : w0;
        const uint16_t *w3 = nc > 3 ? w0 + 3 * (size_t)k : w0;
        for (int r = 0; r < n_x; r++) {
            float o[4];
            dot8x4_f16(x + (size_t)r * k, w0, w1, w2, w3, k, o);
            for (int i = 0; i < nc; i++) {
                /* horizontal_sum_and_f32_to_f16 (simd_support.rs:108-116) */
                out[(size_t)r * n_w + c0 + i] = _cvtss_sh(o[i], 0);
            }
        }
    }
}

static void matmul_transposed_f32_impl(const float *x, int n_x, const float *w, int n_w, int k, float *out, int parallel) {
    int tiles = (n_w + 3) / 4;
#pragma omp parallel for schedule(static) if (parallel)
    for (int t = 0; t < tiles; t++) {
        int c0 = t * 4;
        int nc = n_w - c0 < 4 ? n_w - c0 : 4;
        const float *w0 = w + (size_t)c0 * k;
        const float *w1 = nc > 1 ? w0 + k : w0;
        const float *w2 = nc > 2 ? w0 + 2 * (size_t)k : w0;
        const float *w3 = nc > 3 ? w0 + 3 * (size_t)k : w0;
        for (int r = 0; r < n_x; r++) {
            float o[4];
            dot8x4_f32(x + (size_t)r * k, w0, w1, w2, w3, k, o);
            for (int i = 0; i < nc; i++) out[(size_t)r * n_w + c0 + i] = o[i];
        }
    }
}

void orc_matmul_transposed_f32(const float *x, int n_x, const float *w, int n_w, int k, float *out) {
    matmul_transposed_f32_impl(x, n_x, w, n_w, k, out, 1);
}

/* When set, the one-row f32 products run on one thread, as Tensor::matrix_vector_mul_transposed_f32 does
 * (tensor.rs:1837-1918: the output head always, and w1/w2/w3 in f32 mode when n == 1).  Values are the same
 * either way; only the timing of the CPU baseline changes. */
static int g_ref_threading = 0;
void orc_set_reference_threading(int on) { g_ref_threading = on ? 1 : 0; }

void orc_matmul_f32_seqk(const float *a, int m, const float *b, int n, int k, float *out) {
    /* tensor.rs:1078-1113: tgt[i, c] = fma(src[i, k2], other[k2, c], tgt[i, c]) with k2 ascending. The
     * blocking over rows/cols/k only changes the order in which different elements are visited. */
    for (int i = 0; i < m; i++) {
        for (int c = 0; c < n; c++) {
            if (g_exact) {
                double accd = 0.0;
                for (int kk = 0; kk < k; kk++) accd += (double)a[(size_t)i * k + kk] * (double)b[(size_t)kk * n + c];
                out[(size_t)i * n + c] = (float)accd;
                continue;
            }
            float acc = 0.0f;
            for (int kk = 0; kk < k; kk++) {
                acc = fmaf(a[(size_t)i * k + kk], b[(size_t)kk * n + c], acc);
            }
            out[(size_t)i * n + c] = acc;
        }
    }
}

void orc_vector_matrix_mul_f32(const float *a, const float *b, int k, int n, float *out) {
    /* tensor.rs:1954-1980: lane i of sum8 accumulates rows (row8*8 + i); rows past k contribute zeros. */
    for (int c = 0; c < n; c++) {
        if (g_exact) {
            double accd = 0.0;
            for (int row = 0; row < k; row++) accd += (double)a[row] * (double)b[(size_t)row * n + c];
            out[c] = (float)accd;
            continue;
        }
        float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        for (int row = 0; row < k; row += 8) {
            for (int i = 0; i < 8; i++) {
                float l = (row + i < k) ? a[row + i] : 0.0f;
                float r = (row + i < k) ? b[(size_t)(row + i) * n + c] : 0.0f;
                acc[i] = fmaf(l, r, acc[i]);
            }
        }
        out[c] = orc_hsum8(acc);
    }
}

/* ------------------------------------------------------------------------------------------ */
/* element-wise pieces                                                                         */
/* ------------------------------------------------------------------------------------------ */

void orc_rmsnorm_row(const float *x, const float *w, int d, double eps, float *out) {
    /* x.pow(2.0).mean_cols().add_scalar(eps as f32) ; x.scalar_multiply_broadcast(inner.rsqrt()) ;
     * .hadamard_product_broadcast(weight)   (transformer.rs:476-480; tensor.rs:537-547, 511-522, 595-605,
     * 561-571, 619-636, 654-677).  Every intermediate is an f32 tensor. */
    float sum = 0.0f;
    if (g_exact) {
        double sd = 0.0;
        for (int i = 0; i < d; i++) sd += (double)x[i] * (double)x[i];
        sum = (float)sd;
    } else {
        for (int i = 0; i < d; i++) {
            float sq = x[i] * x[i];
            sum += sq;
        }
    }
    float mean = sum / (float)d;
    float inner = mean + (float)eps;
    float rs = 1.0f / sqrtf(inner);
    for (int i = 0; i < d; i++) {
        float v = x[i] * rs;
        out[i] = v * w[i];
    }
}

void orc_softmax_row(const float *s, int n, float *out) {
    float sum = 0.0f;
    if (g_exact) {
        double sd = 0.0;
        for (int i = 0; i < n; i++) sd += (double)expf(s[i]);
        sum = (float)sd;
    } else {
        for (int i = 0; i < n; i++) sum += expf(s[i]);
    }
    for (int i = 0; i < n; i++) out[i] = expf(s[i]) / sum;
}

float orc_silu(float v) { return v / (1.0f + expf(-v)); }

void orc_freqs_cis(int head_dim, int max_seq_len, double theta, double *out) {
    int half = head_dim / 2;
    for (int pos = 0; pos < max_seq_len; pos++) {
        for (int j = 0; j < half; j++) {
            double freq = 1.0 / pow(theta, (double)j * 2.0 / (double)head_dim);
            double ang = freq * (double)pos;
            out[((size_t)pos * half + j) * 2 + 0] = cos(ang);
            out[((size_t)pos * half + j) * 2 + 1] = sin(ang);
        }
    }
}

void orc_rope_row(float *x, int n_heads, int head_dim, const double *fc) {
    /* transformer.rs:834-853: table cast to f32 at use; products and sums in f32 without FMA. */
    for (int h = 0; h < n_heads; h++) {
        float *row = x + (size_t)h * head_dim;
        for (int c = 0; c < head_dim / 2; c++) {
            float f_real = (float)fc[c * 2 + 0];
            float f_imag = (float)fc[c * 2 + 1];
            float re = row[c * 2];
            float im = row[c * 2 + 1];
            float p0 = re * f_real;
            float p1 = im * f_imag;
            float p2 = re * f_imag;
            float p3 = im * f_real;
            row[c * 2] = p0 - p1;
            row[c * 2 + 1] = p2 + p3;
        }
    }
}

/* TokenSampler::sample up to the random draw (token_sampler.rs:83-158): the candidates left after the top-k and top-p
 * cuts, in the order the draw walks them, with their softmax probabilities.  Returns the number of candidates (at most
 * min(top_k, vocab); out_ids / out_probs must hold that many); *total_p is their probability mass (:159-162).
 * Ties between equal probabilities are ordered by ascending id (the reference's sort_unstable_by leaves them unspecified). */
typedef struct { int32_t id; float p; } orc_cand;
static int orc_cand_cmp(const void *a, const void *b) {
    const orc_cand *x = (const orc_cand *)a, *y = (const orc_cand *)b;
    /* token_sampler.rs:131-145: descending by probability, NaN last */
    int xn = isnan(x->p), yn = isnan(y->p);
    if (xn || yn) {
        if (xn && yn) return (x->id > y->id) - (x->id < y->id);
        return xn ? 1 : -1;
    }
    if (x->p > y->p) return -1;
    if (x->p < y->p) return 1;
    return (x->id > y->id) - (x->id < y->id);
}

int32_t orc_sample_candidates(const float *logits_in, int vocab, float temperature, float top_p, int32_t top_k, float repetition_penalty,
                              const int32_t *existing_tokens, int32_t n_existing, int32_t *out_ids, float *out_probs, float *total_p) {
    float *l = (float *)malloc(sizeof(float) * (size_t)vocab);
    orc_cand *c = (orc_cand *)malloc(sizeof(orc_cand) * (size_t)vocab);
    memcpy(l, logits_in, sizeof(float) * (size_t)vocab);
    if (temperature > 0.0f) { /* :99-102, scalar_multiply_f32(1.0 / temperature) */
        float inv = 1.0f / temperature;
        for (int i = 0; i < vocab; i++) l[i] = l[i] * inv;
    }
    /* :104-123.  After the transpose the tensor is 1 x vocab and the three loops run over 0..rows() == 0..1: only
     * token 0 is penalised (by penalty^count), "maxv" is token 0's value, and only token 0 has it subtracted. */
    if (repetition_penalty != 1.0f) {
        int count = 0;
        for (int i = 0; i < n_existing; i++) count += existing_tokens[i] == 0;
        if (count > 0) l[0] = l[0] * powf(repetition_penalty, (float)count);
    }
    {
        float maxv = -INFINITY;
        if (l[0] > maxv) maxv = l[0];
        l[0] = l[0] - maxv;
    }
    float sum = 0.0f; /* :124 softmax (tensor.rs:479-494): no maximum subtracted, sequential f32 sum */
    for (int i = 0; i < vocab; i++) sum += expf(l[i]);
    for (int i = 0; i < vocab; i++) {
        c[i].id = i;
        c[i].p = expf(l[i]) / sum;
    }
    qsort(c, (size_t)vocab, sizeof(orc_cand), orc_cand_cmp);
    int32_t n = top_k < vocab ? top_k : vocab; /* :147 truncate(top_k) */
    if (n < 0) n = 0;
    float acc = 0.0f;
    for (int32_t i = 0; i < n; i++) { /* :148-155 */
        acc += c[i].p;
        if (acc >= top_p) {
            n = i + 1;
            break;
        }
    }
    float tot = 0.0f;
    for (int32_t i = 0; i < n; i++) { /* :156-159 */
        tot += c[i].p;
        out_ids[i] = c[i].id;
        out_probs[i] = c[i].p;
    }
    *total_p = tot;
    free(l);
    free(c);
    return n;
}

/* The draw (token_sampler.rs:160-173) with the uniform variate passed in: p = u * total_p stands for
 * rng.gen_range(0.0..=total_p).  Returns the token id, *prob = its probability / total_p. */
int32_t orc_sample_pick(const int32_t *ids, const float *probs, int32_t n, float total_p, float u, float *prob) {
    float p = total_p > 0.0f ? u * total_p : 0.0f;
    float acc = 0.0f;
    for (int32_t i = 0; i < n; i++) {
        acc += probs[i];
        if (acc >= p) {
            if (prob) *prob = probs[i] / total_p;
            return ids[i];
        }
    }
    if (prob) *prob = 0.0f;
    return 0;
}

int32_t orc_sample_greedy(const float *logits_in, int vocab, float temperature, float *prob, int32_t *n_ties) {
    float *l = (float *)malloc(sizeof(float) * (size_t)vocab);
    memcpy(l, logits_in, sizeof(float) * (size_t)vocab);
    /* token_sampler.rs:99-102 */
    if (temperature > 0.0f) {
        float inv = 1.0f / temperature;
        for (int i = 0; i < vocab; i++) l[i] = l[i] * inv;
    }
    /* token_sampler.rs:112-123: after the transpose the tensor is 1 x vocab, and both loops run over
     * 0..logits.rows() == 0..1, so only token 0 takes part: maxv = l[0]; l[0] -= maxv. */
    {
        float maxv = -INFINITY;
        float v = l[0];
        if (v > maxv) maxv = v;
        l[0] = l[0] - maxv;
    }
    /* token_sampler.rs:124 softmax (tensor.rs:479-494) */
    float sum = 0.0f;
    for (int i = 0; i < vocab; i++) sum += expf(l[i]);
    int32_t best = -1;
    float bestp = 0.0f;
    int32_t ties = 0;
    for (int i = 0; i < vocab; i++) {
        float p = expf(l[i]) / sum;
        l[i] = p;
        /* token_sampler.rs:131-145: descending by probability, NaN last */
        if (isnan(p)) continue;
        if (best < 0 || p > bestp) {
            best = i;
            bestp = p;
            ties = 1;
        } else if (p == bestp) {
            ties++;
        }
    }
    if (best < 0) { /* all NaN: the sort leaves an unspecified order; report id 0 like the fall-through (:173) */
        best = 0;
        bestp = l[0];
        ties = vocab;
    }
    if (prob) *prob = bestp; /* v.1 / total_p with total_p == v.1 gives 1.0 in the reference; we report the raw p */
    if (n_ties) *n_ties = ties;
    free(l);
    return best;
}

/* ------------------------------------------------------------------------------------------ */
/* model                                                                                       */
/* ------------------------------------------------------------------------------------------ */

typedef struct {
    void *w[8];      /* indexed by kind ORC_WQ..ORC_W3 (1..7): f16 bits if force_f16 else f32 */
    float *attn_norm;
    float *ffn_norm;
} orc_layer;

struct orc_model {
    orc_params p;
    int head_dim;
    float *tok_emb;  /* [vocab x dim] f32 */
    float *norm;     /* [dim] */
    float *output;   /* [vocab x dim] f32 */
    orc_layer *layers;
    double *freqs_cis; /* [max_seq_len x head_dim/2 x 2] */
};

struct orc_caches {
    int n_layers, n_heads, head_dim, max_seq_len, is_f16;
    void *k; /* [layer][head][head_dim][max_seq_len] */
    void *v;
};

static __thread float *g_layer_tap = NULL;
void orc_set_layer_tap(float *buf) { g_layer_tap = buf; }

orc_model *orc_model_create(const orc_params *p) {
    if (p->dim <= 0 || p->n_heads <= 0 || p->dim % p->n_heads != 0) return NULL; /* transformer.rs:252 */
    orc_model *m = (orc_model *)calloc(1, sizeof(orc_model));
    m->p = *p;
    m->head_dim = p->dim / p->n_heads;
    m->layers = (orc_layer *)calloc((size_t)p->n_layers, sizeof(orc_layer));
    m->freqs_cis = (double *)malloc(sizeof(double) * (size_t)p->max_seq_len * (size_t)(m->head_dim / 2) * 2);
    orc_freqs_cis(m->head_dim, p->max_seq_len, 10000.0, m->freqs_cis); /* transformer.rs:311 */
    return m;
}

void orc_model_free(orc_model *m) {
    if (!m) return;
    for (int l = 0; l < m->p.n_layers; l++) {
        for (int k = 0; k < 8; k++) free(m->layers[l].w[k]);
        free(m->layers[l].attn_norm);
        free(m->layers[l].ffn_norm);
    }
    free(m->layers);
    free(m->tok_emb);
    free(m->norm);
    free(m->output);
    free(m->freqs_cis);
    free(m);
}

static float *to_f32_copy(const void *src, size_t n, int src_dtype) {
    float *dst = (float *)malloc(sizeof(float) * n);
    if (src_dtype == ORC_F16) {
        orc_f16_to_f32_array((const uint16_t *)src, dst, n);
    } else {
        memcpy(dst, src, sizeof(float) * n);
    }
    return dst;
}

int orc_model_set_tensor(orc_model *m, int kind, int layer, const void *src, int rows, int cols, int src_dtype) {
    const orc_params *p = &m->p;
    size_t n = (size_t)rows * (size_t)cols;
    int d = p->dim, F = p->ffn_hidden, V = p->vocab_size;
    int er, ec;
    switch (kind) {
    case ORC_TOK_EMB: er = V; ec = d; break;
    case ORC_OUTPUT: er = V; ec = d; break;
    case ORC_WQ: case ORC_WK: case ORC_WV: case ORC_WO: er = d; ec = d; break;
    case ORC_W1: case ORC_W3: er = F; ec = d; break;
    case ORC_W2: er = d; ec = F; break;
    case ORC_ATTN_NORM: case ORC_FFN_NORM: case ORC_NORM: er = 1; ec = d; break;
    default: return 1;
    }
    if (rows != er || cols != ec) return 2;
    if (kind >= ORC_WQ && kind <= ORC_FFN_NORM && (layer < 0 || layer >= p->n_layers)) return 3;
    if (kind == ORC_TOK_EMB) { free(m->tok_emb); m->tok_emb = to_f32_copy(src, n, src_dtype); return 0; }
    if (kind == ORC_OUTPUT) { free(m->output); m->output = to_f32_copy(src, n, src_dtype); return 0; }
    if (kind == ORC_NORM) { free(m->norm); m->norm = to_f32_copy(src, n, src_dtype); return 0; }
    orc_layer *L = &m->layers[layer];
    if (kind == ORC_ATTN_NORM) { free(L->attn_norm); L->attn_norm = to_f32_copy(src, n, src_dtype); return 0; }
    if (kind == ORC_FFN_NORM) { free(L->ffn_norm); L->ffn_norm = to_f32_copy(src, n, src_dtype); return 0; }
    free(L->w[kind]);
    if (p->force_f16) {
        uint16_t *dst = (uint16_t *)malloc(sizeof(uint16_t) * n);
        if (src_dtype == ORC_F16) memcpy(dst, src, sizeof(uint16_t) * n);
        else orc_f32_to_f16_array((const float *)src, dst, n); /* Tensor::to_f16 */
        L->w[kind] = dst;
    } else {
        L->w[kind] = to_f32_copy(src, n, src_dtype);
    }
    return 0;
}

orc_caches *orc_caches_create(const orc_model *m) {
    orc_caches *c = (orc_caches *)calloc(1, sizeof(orc_caches));
    c->n_layers = m->p.n_layers;
    c->n_heads = m->p.n_heads;
    c->head_dim = m->head_dim;
    c->max_seq_len = m->p.max_seq_len;
    c->is_f16 = m->p.force_f16 ? 1 : 0; /* transformer.rs:138-142 */
    size_t n = (size_t)c->n_layers * c->n_heads * c->head_dim * c->max_seq_len;
    size_t es = c->is_f16 ? 2 : 4;
    c->k = calloc(n, es); /* Tensor::zeros */
    c->v = calloc(n, es);
    return c;
}

orc_caches *orc_caches_true_clone(const orc_caches *s) {
    orc_caches *c = (orc_caches *)malloc(sizeof(orc_caches));
    *c = *s;
    size_t n = (size_t)c->n_layers * c->n_heads * c->head_dim * c->max_seq_len;
    size_t es = c->is_f16 ? 2 : 4;
    c->k = malloc(n * es);
    c->v = malloc(n * es);
    memcpy(c->k, s->k, n * es);
    memcpy(c->v, s->v, n * es);
    return c;
}

void orc_caches_shift_left(orc_caches *c, int shifts) {
    /* transformer.rs:180-197: per shift, column seq_idx takes column seq_idx + 1 for seq_idx < cols - 1;
     * the last column keeps its value. */
    size_t rows = (size_t)c->n_layers * c->n_heads * c->head_dim;
    size_t T = (size_t)c->max_seq_len;
    size_t es = c->is_f16 ? 2 : 4;
    for (int s = 0; s < shifts; s++) {
        for (size_t r = 0; r < rows; r++) {
            char *kr = (char *)c->k + r * T * es;
            char *vr = (char *)c->v + r * T * es;
            memmove(kr, kr + es, (T - 1) * es);
            memmove(vr, vr + es, (T - 1) * es);
        }
    }
}

void orc_caches_free(orc_caches *c) {
    if (!c) return;
    free(c->k);
    free(c->v);
    free(c);
}

static inline size_t cache_row_off(const orc_caches *c, int layer, int head, int j) {
    return (((size_t)layer * c->n_heads + head) * c->head_dim + j) * (size_t)c->max_seq_len;
}

void orc_caches_read(const orc_caches *c, int layer, int head, int which, float *out) {
    size_t off = cache_row_off(c, layer, head, 0);
    size_t n = (size_t)c->head_dim * c->max_seq_len;
    const void *base = which ? c->v : c->k;
    if (c->is_f16) orc_f16_to_f32_array((const uint16_t *)base + off, out, n);
    else memcpy(out, (const float *)base + off, n * sizeof(float));
}

static inline void cache_set(orc_caches *c, void *base, size_t idx, float v) {
    if (c->is_f16) ((uint16_t *)base)[idx] = _cvtss_sh(v, 0); /* Tensor::set_f32 on an f16 tensor (tensor.rs:373-376) */
    else ((float *)base)[idx] = v;
}

/* x [n x k] (f32) times W^T where W is the stored projection [n_w x k]; result f32 [n x n_w].
 * f16 mode: x is rounded to f16 first (to_same_type, tensor.rs:1198-1208), the product is rounded to f16
 * by the kernel (tensor.rs:1623-1643) and widened back to f32 (to_f32 / into_dtype). */
static void project(const orc_model *m, const float *x, int n, const void *w, int n_w, int k, float *out, int serial_if_one_row) {
    if (m->p.force_f16) {
        uint16_t *xh = (uint16_t *)malloc(sizeof(uint16_t) * (size_t)n * k);
        uint16_t *oh = (uint16_t *)malloc(sizeof(uint16_t) * (size_t)n * n_w);
        orc_f32_to_f16_array(x, xh, (size_t)n * k);
        orc_matmul_transposed_f16(xh, n, (const uint16_t *)w, n_w, k, oh);
        orc_f16_to_f32_array(oh, out, (size_t)n * n_w);
        free(xh);
        free(oh);
    } else {
        matmul_transposed_f32_impl(x, n, (const float *)w, n_w, k, out, !(serial_if_one_row && n == 1 && g_ref_threading));
    }
}

/* Transformer::forward (transformer.rs:343-383) with the places marked where a layer split cuts it: tokens != NULL starts
 * from the embedding gather, else from the stream x_in; blocks first..=last run; x_out != NULL receives the stream after
 * them; logits_out != NULL adds the final norm and the head. */
static int forward_span(const orc_model *m, orc_caches *c, const int32_t *tokens, const float *x_in, int n, int start_pos, int first, int last,
                        float *x_out, float *logits_out) {
    const orc_params *p = &m->p;
    const int d = p->dim, H = p->n_heads, hd = m->head_dim, F = p->ffn_hidden, V = p->vocab_size;
    if (n < 1) return 1;
    if (n > 1 && start_pos != 0) return 2;      /* mask is n x n, scores are n x (start_pos+n): add panics (tensor.rs:576-584) */
    if (start_pos + n > p->max_seq_len) return 3;
    for (int i = 0; tokens && i < n; i++) {
        if (tokens[i] < 0 || tokens[i] >= V) return 4; /* BTreeMap get().unwrap() (embedding.rs:50-52) */
    }
    const int T = start_pos + n;

    float *x = (float *)malloc(sizeof(float) * (size_t)n * d);
    float *xn = (float *)malloc(sizeof(float) * (size_t)n * d);
    float *q = (float *)malloc(sizeof(float) * (size_t)n * d);
    float *k = (float *)malloc(sizeof(float) * (size_t)n * d);
    float *v = (float *)malloc(sizeof(float) * (size_t)n * d);
    float *att = (float *)malloc(sizeof(float) * (size_t)n * d);
    float *atto = (float *)malloc(sizeof(float) * (size_t)n * d);
    float *h = (float *)malloc(sizeof(float) * (size_t)n * d);
    float *g = (float *)malloc(sizeof(float) * (size_t)n * F);
    float *u = (float *)malloc(sizeof(float) * (size_t)n * F);
    float *ffn = (float *)malloc(sizeof(float) * (size_t)n * d);

    /* embedding gather + concat (transformer.rs:361-367) */
    if (tokens) {
        for (int i = 0; i < n; i++) memcpy(x + (size_t)i * d, m->tok_emb + (size_t)tokens[i] * d, sizeof(float) * d);
    } else {
        memcpy(x, x_in, sizeof(float) * (size_t)n * d);
    }

    const float inv_sqrt_hd = 1.0f / sqrtf((float)hd); /* transformer.rs:770 */

    for (int l = first; l <= last; l++) {
        const orc_layer *L = &m->layers[l];
        /* attention_norm (transformer.rs:432) */
        for (int i = 0; i < n; i++) orc_rmsnorm_row(x + (size_t)i * d, L->attn_norm, d, p->norm_eps, xn + (size_t)i * d);
        /* wq / wk / wv (transformer.rs:694-702) */
        project(m, xn, n, L->w[ORC_WQ], d, d, q, 0);
        project(m, xn, n, L->w[ORC_WK], d, d, k, 0);
        project(m, xn, n, L->w[ORC_WV], d, d, v, 0);
        /* RoPE per token row (transformer.rs:708-725) */
        for (int i = 0; i < n; i++) {
            const double *fc = m->freqs_cis + (size_t)(start_pos + i) * (hd / 2) * 2;
            orc_rope_row(q + (size_t)i * d, H, hd, fc);
            orc_rope_row(k + (size_t)i * d, H, hd, fc);
        }
        /* per head (transformer.rs:727-781) */
#pragma omp parallel for schedule(dynamic, 1)
        for (int hh = 0; hh < H; hh++) {
            /* cache write (transformer.rs:754-761) */
            for (int pos = start_pos; pos < start_pos + n; pos++) {
                for (int j = 0; j < hd; j++) {
                    size_t idx = cache_row_off(c, l, hh, j) + (size_t)pos;
                    cache_set(c, c->k, idx, k[(size_t)(pos - start_pos) * d + (size_t)hh * hd + j]);
                    cache_set(c, c->v, idx, v[(size_t)(pos - start_pos) * d + (size_t)hh * hd + j]);
                }
            }
            /* keys / values: clip_cols(T) then into f32 (transformer.rs:762-766) -> [hd x T] */
            float *keys = (float *)malloc(sizeof(float) * (size_t)hd * T);
            float *vals = (float *)malloc(sizeof(float) * (size_t)hd * T);
            for (int j = 0; j < hd; j++) {
                size_t off = cache_row_off(c, l, hh, j);
                if (c->is_f16) {
                    orc_f16_to_f32_array((const uint16_t *)c->k + off, keys + (size_t)j * T, (size_t)T);
                    orc_f16_to_f32_array((const uint16_t *)c->v + off, vals + (size_t)j * T, (size_t)T);
                } else {
                    memcpy(keys + (size_t)j * T, (const float *)c->k + off, sizeof(float) * T);
                    memcpy(vals + (size_t)j * T, (const float *)c->v + off, sizeof(float) * T);
                }
            }
            /* xq_row: this head's query rows [n x hd] */
            float *qh = (float *)malloc(sizeof(float) * (size_t)n * hd);
            for (int i = 0; i < n; i++) memcpy(qh + (size_t)i * hd, q + (size_t)i * d + (size_t)hh * hd, sizeof(float) * hd);
            float *s = (float *)malloc(sizeof(float) * (size_t)n * T);
            float *pr = (float *)malloc(sizeof(float) * (size_t)n * T);
            /* xq_row.matrix_mul(&keys) (tensor.rs:979-997): rows == 1 -> vector_matrix_mul, else matrix_mul_inplace */
            if (n == 1) orc_vector_matrix_mul_f32(qh, keys, hd, T, s);
            else orc_matmul_f32_seqk(qh, n, keys, T, hd, s);
            for (size_t i = 0; i < (size_t)n * T; i++) s[i] = s[i] * inv_sqrt_hd; /* scalar_multiply_f32 */
            if (n > 1) {
                /* full_triu(n, n, start_pos + 1, -inf) (tensor.rs:496-508) then add (tensor.rs:573-593) */
                for (int r = 0; r < n; r++) {
                    for (int cc = 0; cc < T; cc++) {
                        float mv = (cc >= r + start_pos + 1) ? -INFINITY : 0.0f;
                        s[(size_t)r * T + cc] = s[(size_t)r * T + cc] + mv;
                    }
                }
            }
            for (int r = 0; r < n; r++) orc_softmax_row(s + (size_t)r * T, T, pr + (size_t)r * T);
            /* softmax(..).matrix_mul_transposed(&values) -> f32 tiled kernel: dot8 over T (tensor.rs:1282-1475) */
            for (int r = 0; r < n; r++) {
                for (int j = 0; j < hd; j++) {
                    att[(size_t)r * d + (size_t)hh * hd + j] = orc_dot8_f32(pr + (size_t)r * T, vals + (size_t)j * T, T);
                }
            }
            free(keys);
            free(vals);
            free(qh);
            free(s);
            free(pr);
        }
        /* wo per row (transformer.rs:783-819); same arithmetic as one n-row product */
        project(m, att, n, L->w[ORC_WO], d, d, atto, 0);
        /* h = x + att_out (transformer.rs:442) */
        for (size_t i = 0; i < (size_t)n * d; i++) h[i] = x[i] + atto[i];
        /* ffn_norm (transformer.rs:443) */
        for (int i = 0; i < n; i++) orc_rmsnorm_row(h + (size_t)i * d, L->ffn_norm, d, p->norm_eps, xn + (size_t)i * d);
        /* feed forward (transformer.rs:536-583) */
        project(m, xn, n, L->w[ORC_W1], F, d, g, 1);
        project(m, xn, n, L->w[ORC_W3], F, d, u, 1);
        for (size_t i = 0; i < (size_t)n * F; i++) {
            float sv = orc_silu(g[i]); /* silu (tensor.rs:826-827) */
            g[i] = sv * u[i];          /* hadamard_product (tensor.rs:729) */
        }
        project(m, g, n, L->w[ORC_W2], d, F, ffn, 1);
        /* h + ffn_out (transformer.rs:445) */
        for (size_t i = 0; i < (size_t)n * d; i++) x[i] = h[i] + ffn[i];
        if (g_layer_tap) memcpy(g_layer_tap + (size_t)l * n * d, x, sizeof(float) * (size_t)n * d);
    }
    if (x_out) memcpy(x_out, x, sizeof(float) * (size_t)n * d);
    if (logits_out) {
        /* final norm on all rows, last row, output head (transformer.rs:378-381; tensor.rs:1837-1918) */
        for (int i = 0; i < n; i++) orc_rmsnorm_row(x + (size_t)i * d, m->norm, d, p->norm_eps, xn + (size_t)i * d);
        matmul_transposed_f32_impl(xn + (size_t)(n - 1) * d, 1, m->output, V, d, logits_out, !g_ref_threading);
    }

    free(x); free(xn); free(q); free(k); free(v); free(att); free(atto); free(h); free(g); free(u); free(ffn);
    return 0;
}

int orc_forward(const orc_model *m, orc_caches *c, const int32_t *tokens, int n, int start_pos, float *logits_out) {
    return forward_span(m, c, tokens, NULL, n, start_pos, 0, m->p.n_layers - 1, NULL, logits_out);
}

int orc_forward_layers(const orc_model *m, orc_caches *c, const float *x_in, int n, int start_pos, int first_layer, int last_layer, float *x_out) {
    if (first_layer < 0 || last_layer < first_layer || last_layer >= m->p.n_layers) return 5;
    return forward_span(m, c, NULL, x_in, n, start_pos, first_layer, last_layer, x_out, NULL);
}

int orc_embed(const orc_model *m, const int32_t *tokens, int n, float *x_out) {
    for (int i = 0; i < n; i++) {
        if (tokens[i] < 0 || tokens[i] >= m->p.vocab_size) return 4;
        memcpy(x_out + (size_t)i * m->p.dim, m->tok_emb + (size_t)tokens[i] * m->p.dim, sizeof(float) * m->p.dim);
    }
    return 0;
}

int orc_head(const orc_model *m, const float *x, int n, float *logits_out) {
    /* an empty span: no block runs, the stream goes straight to the final norm and the head */
    if (n < 1) return 1;
    return forward_span(m, NULL, NULL, x, n, 0, 0, -1, NULL, logits_out);
}
