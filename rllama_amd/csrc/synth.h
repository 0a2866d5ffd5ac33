/*
 * synth.h -- portable counter-based generator for synthetic model weights and token ids.
 *
 * The reference ships no model fixtures and seeds nothing (rand::thread_rng() everywhere, e.g.
 * tensor.rs:1985-1994), so the random-init LLaMA-shape models that the parity tests and the benchmark
 * run on are defined here: element `idx` of stream `stream` under `seed` is a pure function of
 * (seed, stream, idx).  The same source compiles for the host (gcc / host pass of hipcc) and for gfx950,
 * and it uses only operations that IEEE-754 fixes bit for bit on both -- +, -, *, /, sqrt in binary64
 * with FMA contraction switched off, and integer arithmetic; the logarithm is evaluated here, not by a
 * math library -- so a tensor generated on the GPU is bit-identical to the one generated on the host.
 *
 * Normal deviates: Marsaglia's polar method on a pair of uniform variates per attempt, up to
 * SYNTH_MAX_ATTEMPTS attempts per pair of outputs (elements 2p and 2p+1 share pair p).
 * Value = deviate * std, rounded binary64 -> binary32 -> binary16 (RNE both times).
 */
#ifndef RLLAMA_SYNTH_H
#define RLLAMA_SYNTH_H

#include <stdint.h>

#if defined(__HIPCC__)
#define SYNTH_FN __host__ __device__ static inline
#else
#define SYNTH_FN static inline
#endif

#define SYNTH_MAX_ATTEMPTS 32

/* Stream ids: tensor streams are SYNTH_STREAM_TENSOR(kind, layer); token ids have their own stream. */
#define SYNTH_STREAM_TENSOR(kind, layer) ((uint64_t)(kind) * 4096u + (uint64_t)(layer) + 1u)
#define SYNTH_STREAM_TOKENS 0xF0000000u

SYNTH_FN uint64_t synth_mix64(uint64_t z) {
    /* splitmix64 output function */
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

SYNTH_FN uint64_t synth_key(uint64_t seed, uint64_t stream) {
    return synth_mix64(seed * 0x9E3779B97F4A7C15ull + synth_mix64(stream + 0x9E3779B97F4A7C15ull));
}

/* ctr-th output of the splitmix64 sequence whose state starts at key */
SYNTH_FN uint64_t synth_u64(uint64_t key, uint64_t ctr) {
    return synth_mix64(key + (ctr + 1u) * 0x9E3779B97F4A7C15ull);
}

SYNTH_FN double synth_bits_to_double(uint64_t b) {
    union { uint64_t u; double d; } c;
    c.u = b;
    return c.d;
}

SYNTH_FN uint64_t synth_double_to_bits(double d) {
    union { uint64_t u; double d; } c;
    c.d = d;
    return c.u;
}

/* natural logarithm of a positive normal binary64, fixed operation order, no library call, no FMA */
SYNTH_FN double synth_log(double s) {
#if defined(__clang__)
#pragma clang fp contract(off)
#endif
    uint64_t b = synth_double_to_bits(s);
    int e = (int)((b >> 52) & 0x7ff) - 1022;                                   /* s = m * 2^e, m in [0.5, 1) */
    double m = synth_bits_to_double((b & 0x000fffffffffffffull) | 0x3fe0000000000000ull);
    if (m < 0.70710678118654752440) {
        m = m * 2.0;
        e = e - 1;
    }
    double t = (m - 1.0) / (m + 1.0);                                          /* |t| <= 0.1716 */
    double t2 = t * t;
    /* atanh series: log(m) = 2 t (1 + t2/3 + t2^2/5 + ... + t2^11/23), Horner */
    double p = 1.0 / 23.0;
    p = p * t2 + 1.0 / 21.0;
    p = p * t2 + 1.0 / 19.0;
    p = p * t2 + 1.0 / 17.0;
    p = p * t2 + 1.0 / 15.0;
    p = p * t2 + 1.0 / 13.0;
    p = p * t2 + 1.0 / 11.0;
    p = p * t2 + 1.0 / 9.0;
    p = p * t2 + 1.0 / 7.0;
    p = p * t2 + 1.0 / 5.0;
    p = p * t2 + 1.0 / 3.0;
    p = p * t2 + 1.0;
    double lm = 2.0 * t * p;
    return (double)e * 0.69314718055994530942 + lm;
}

SYNTH_FN double synth_sqrt(double x) {
#if defined(__HIP_DEVICE_COMPILE__)
    return __builtin_sqrt(x); /* correctly rounded binary64 square root on gfx9 */
#else
    return __builtin_sqrt(x);
#endif
}

/* round-to-nearest-even binary32 -> binary16, integer ops only (same on host and device) */
SYNTH_FN uint16_t synth_f32_to_f16(float v) {
    union { uint32_t u; float f; } c;
    c.f = v;
    uint32_t x = c.u;
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t absx = x & 0x7fffffffu;
    if (absx >= 0x7f800000u) return (uint16_t)(sign | (absx > 0x7f800000u ? 0x7e00u : 0x7c00u));
    if (absx >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);
    if (absx < 0x33000001u) return (uint16_t)sign;
    int32_t ex = (int32_t)(absx >> 23) - 127;
    uint32_t mant = (absx & 0x7fffffu) | 0x800000u;
    uint32_t shift = ex < -14 ? (uint32_t)(13 + (-14 - ex)) : 13u;
    uint32_t hexp = ex < -14 ? 0u : (uint32_t)(ex + 15);
    uint32_t q = mant >> shift;
    uint32_t rem = mant & ((1u << shift) - 1u);
    uint32_t halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (q & 1u))) q += 1;
    uint32_t h = hexp == 0 ? q : ((hexp - 1) << 10) + q;
    return (uint16_t)(sign | h);
}

/* Standard normal deviates of pair `pair` of the stream (binary64): elements 2*pair and 2*pair + 1. */
SYNTH_FN void synth_normal_pair(uint64_t key, uint64_t pair, double *z0, double *z1) {
#if defined(__clang__)
#pragma clang fp contract(off)
#endif
    for (uint32_t a = 0; a < SYNTH_MAX_ATTEMPTS; a++) {
        uint64_t c = (pair * SYNTH_MAX_ATTEMPTS + a) * 2u;
        uint64_t r1 = synth_u64(key, c);
        uint64_t r2 = synth_u64(key, c + 1u);
        double u = (double)(r1 >> 11) * (1.0 / 9007199254740992.0) * 2.0 - 1.0; /* exact: multiples of 2^-52 in [-1, 1) */
        double v = (double)(r2 >> 11) * (1.0 / 9007199254740992.0) * 2.0 - 1.0;
        double uu = u * u;
        double vv = v * v;
        double s = uu + vv;
        if (s < 1.0 && s > 0.0) {
            double num = -2.0 * synth_log(s);
            double f = synth_sqrt(num / s);
            *z0 = u * f;
            *z1 = v * f;
            return;
        }
    }
    *z0 = 0.0;
    *z1 = 0.0;
}

SYNTH_FN uint16_t synth_scale_to_f16(double z, double std) {
#if defined(__clang__)
#pragma clang fp contract(off)
#endif
    double s = z * std;
    return synth_f32_to_f16((float)s);
}

/* f16 bits of N(0, std^2) element idx */
SYNTH_FN uint16_t synth_normal_f16(uint64_t key, uint64_t idx, double std) {
    double z0, z1;
    synth_normal_pair(key, idx >> 1, &z0, &z1);
    return synth_scale_to_f16((idx & 1u) ? z1 : z0, std);
}

/* token id uniform in [lo, hi) */
SYNTH_FN int32_t synth_token(uint64_t key, uint64_t idx, int32_t lo, int32_t hi) {
    uint64_t r = synth_u64(key, idx) >> 32;
    return lo + (int32_t)((r * (uint64_t)(hi - lo)) >> 32);
}

#endif
