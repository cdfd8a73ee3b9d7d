/*
 * CPU oracle for GGML_OP_FLASH_ATTN_EXT - see fattn_oracle.h for what is pinned
 * and what is recalled.  Test infrastructure only; never linked into the product.
 */
#include "fattn_oracle.h"

#include <float.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif
#if defined(__F16C__)
#include <immintrin.h>
#endif

/* ------------------------------------------------------------------ fp16 -- */

/* IEEE-754 binary32 -> binary16, round-to-nearest-even, overflow to inf, NaN kept
 * quiet.  This is what ggml's GGML_FP32_TO_FP16 computes on every platform and what
 * the reference's ggml_cast(F32 -> F16) of the mask relies on (src/core/fastconformer.h:918,
 * src/crispasr.cpp:3141). */
static uint16_t fp32_to_fp16_soft(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    const uint32_t absx = x & 0x7fffffffu;
    if (absx >= 0x7f800000u) {                         /* inf / nan */
        return (uint16_t)(sign | (absx > 0x7f800000u ? 0x7e00u : 0x7c00u));
    }
    if (absx >= 0x477ff000u) {                         /* >= 65520 rounds to inf */
        return (uint16_t)(sign | 0x7c00u);
    }
    if (absx < 0x33000001u) {                          /* <= 2^-25 rounds to zero */
        return (uint16_t)sign;
    }
    int32_t  e = (int32_t)(absx >> 23) - 127;          /* unbiased exponent */
    uint32_t m = (absx & 0x007fffffu) | 0x00800000u;   /* 24-bit significand */
    uint32_t shift;
    uint32_t base;
    if (e < -14) {                                     /* subnormal half */
        shift = (uint32_t)(13 + (-14 - e));
        base  = 0;
    } else {
        shift = 13;
        base  = (uint32_t)(e + 15) << 10;
        m &= 0x007fffffu;
    }
    uint32_t q    = m >> shift;
    uint32_t rem  = m & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) {
        q++;                                           /* carries into the exponent correctly */
    }
    return (uint16_t)(sign | (base + q));
}

static float fp16_to_fp32_soft(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    const uint32_t e    = (h >> 10) & 0x1fu;
    const uint32_t m    = h & 0x3ffu;
    uint32_t x;
    if (e == 0) {
        if (m == 0) {
            x = sign;
        } else {                                       /* subnormal: m * 2^-24 */
            float f = (float)m * 5.9604644775390625e-08f;
            memcpy(&x, &f, 4);
            x |= sign;
        }
    } else if (e == 31) {
        x = sign | 0x7f800000u | (m << 13);
    } else {
        x = sign | ((e + 112u) << 23) | (m << 13);
    }
    float f;
    memcpy(&f, &x, 4);
    return f;
}

uint16_t ora_fp32_to_fp16(float f) { return fp32_to_fp16_soft(f); }
float    ora_fp16_to_fp32(uint16_t h) { return fp16_to_fp32_soft(h); }

/* fast paths used inside the hot loops; the tests check them against the soft ones */
static inline float h2f(uint16_t h) {
#if defined(__F16C__)
    return _cvtsh_ss(h);
#else
    return fp16_to_fp32_soft(h);
#endif
}
static inline uint16_t f2h(float f) {
#if defined(__F16C__)
    return _cvtss_sh(f, _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC);
#else
    return fp32_to_fp16_soft(f);
#endif
}

void ora_fp32_to_fp16_row(const float * x, uint16_t * y, int64_t n) {
    for (int64_t i = 0; i < n; i++) y[i] = f2h(x[i]);
}
void ora_fp16_to_fp32_row(const uint16_t * x, float * y, int64_t n) {
    for (int64_t i = 0; i < n; i++) y[i] = h2f(x[i]);
}

/* ------------------------------------------------------------------ Q8_0 -- */

/* Block of 32: d = amax/127 kept in f32 for the division, stored as fp16;
 * q = round(x * (1/d)) with the unrounded f32 d
 * (tools/upstream-prs/09-metal-q8_0-bit-match.md:24-31; "block-32" layout
 * src/core/attention.h:79-83).  ggml-cpu's SIMD quantisers round to nearest even,
 * its scalar quantize_row_q8_0_ref rounds half away from zero: both selectable. */
void ora_quantize_row_q8_0(const float * x, ora_block_q8_0 * y, int64_t n, int rounding) {
    const int64_t nb = n / ORA_QK8_0;
    for (int64_t i = 0; i < nb; i++) {
        float amax = 0.0f;
        for (int j = 0; j < ORA_QK8_0; j++) {
            const float a = fabsf(x[i * ORA_QK8_0 + j]);
            if (a > amax) amax = a;
        }
        const float d  = amax / 127.0f;
        const float id = d != 0.0f ? 1.0f / d : 0.0f;
        y[i].d = fp32_to_fp16_soft(d);
        for (int j = 0; j < ORA_QK8_0; j++) {
            const float x0 = x[i * ORA_QK8_0 + j] * id;
            y[i].qs[j] = (int8_t)(rounding == ORA_ROUND_HALF_AWAY ? roundf(x0) : nearbyintf(x0));
        }
    }
}

/* x = q * d  (f32 product of the exact int8 and the exact fp16 scale) */
void ora_dequantize_row_q8_0(const ora_block_q8_0 * x, float * y, int64_t n) {
    const int64_t nb = n / ORA_QK8_0;
    for (int64_t i = 0; i < nb; i++) {
        const float d = fp16_to_fp32_soft(x[i].d);
        for (int j = 0; j < ORA_QK8_0; j++) y[i * ORA_QK8_0 + j] = (float)x[i].qs[j] * d;
    }
}

/* --------------------------------------------------- Q4_0 Q4_1 Q5_0 Q5_1 -- */

/* ggml's scalar quantisers as recalled (quantize_row_q4_0_ref and siblings; the types are the ones
 * src/core/attention.h:79-105 lets CRISPASR_KV_QUANT name).  Symmetric types: the scale comes from the value of
 * largest magnitude WITH its sign (the first such value in the block), d = max / -8 (or -16), so that value maps to
 * quant 0 and the other end of the range clips at 15 (31); q = min(15, trunc(x/d + 8.5)).  Types with a minimum:
 * d = (max - min) / 15 (or 31), q = trunc((x - min)/d + 0.5).  The products and sums are single f32 operations in
 * that order (this file is built without contraction into fused multiply-adds). */
static void quantize_block_sym(const float * x, int levels, uint16_t * d_out, uint8_t * q) {
    float amax = 0.0f, max = 0.0f;
    for (int j = 0; j < 32; j++) {
        const float v = x[j];
        if (amax < fabsf(v)) { amax = fabsf(v); max = v; }
    }
    const float d  = max / (float)(-(levels / 2));
    const float id = d != 0.0f ? 1.0f / d : 0.0f;
    *d_out = fp32_to_fp16_soft(d);
    for (int j = 0; j < 32; j++) {
        const float x0 = x[j] * id;
        const int   qi = (int)(int8_t)(x0 + ((float)(levels / 2) + 0.5f));
        q[j] = (uint8_t)(qi < levels - 1 ? qi : levels - 1);
    }
}

static void quantize_block_min(const float * x, int levels, uint16_t * d_out, uint16_t * m_out, uint8_t * q) {
    float min = FLT_MAX, max = -FLT_MAX;
    for (int j = 0; j < 32; j++) {
        if (x[j] < min) min = x[j];
        if (x[j] > max) max = x[j];
    }
    const float d  = (max - min) / (float)(levels - 1);
    const float id = d != 0.0f ? 1.0f / d : 0.0f;
    *d_out = fp32_to_fp16_soft(d);
    *m_out = fp32_to_fp16_soft(min);
    for (int j = 0; j < 32; j++) {
        const float x0 = (x[j] - min) * id;
        const int   qi = (int)(uint8_t)(x0 + 0.5f);
        q[j] = (uint8_t)(qi < levels - 1 ? qi : levels - 1);
    }
}

static void pack_nibbles(const uint8_t * q, uint8_t * qs, uint8_t * qh) {
    uint32_t h = 0;
    for (int j = 0; j < 16; j++) {
        qs[j] = (uint8_t)((q[j] & 0x0F) | ((q[j + 16] & 0x0F) << 4));
        h |= (uint32_t)((q[j] & 0x10) >> 4) << j;
        h |= (uint32_t)((q[j + 16] & 0x10) >> 4) << (j + 16);
    }
    if (qh) { qh[0] = (uint8_t)h; qh[1] = (uint8_t)(h >> 8); qh[2] = (uint8_t)(h >> 16); qh[3] = (uint8_t)(h >> 24); }
}

static void unpack_nibbles(const uint8_t * qs, const uint8_t * qh, uint8_t * q) {
    const uint32_t h = qh ? (uint32_t)qh[0] | (uint32_t)qh[1] << 8 | (uint32_t)qh[2] << 16 | (uint32_t)qh[3] << 24 : 0;
    for (int j = 0; j < 16; j++) {
        q[j]      = (uint8_t)((qs[j] & 0x0F) | (((h >> j) & 1) << 4));
        q[j + 16] = (uint8_t)((qs[j] >> 4) | (((h >> (j + 16)) & 1) << 4));
    }
}

size_t ora_block_bytes(int type) {
    switch (type) {
        case ORA_TYPE_Q4_0: return sizeof(ora_block_q4_0);
        case ORA_TYPE_Q4_1: return sizeof(ora_block_q4_1);
        case ORA_TYPE_Q5_0: return sizeof(ora_block_q5_0);
        case ORA_TYPE_Q5_1: return sizeof(ora_block_q5_1);
        case ORA_TYPE_Q8_0: return sizeof(ora_block_q8_0);
        default:            return 0;
    }
}

int ora_quantize_row(int type, const float * x, void * y, int64_t n) {
    if (type == ORA_TYPE_Q8_0) { ora_quantize_row_q8_0(x, (ora_block_q8_0 *)y, n, ORA_ROUND_NEAREST_EVEN); return 0; }
    if (!ora_block_bytes(type)) return -2;
    uint8_t q[32];
    for (int64_t i = 0; i < n / 32; i++) {
        const float * xb = x + i * 32;
        if (type == ORA_TYPE_Q4_0) {
            ora_block_q4_0 * b = (ora_block_q4_0 *)y + i;
            quantize_block_sym(xb, 16, &b->d, q);
            pack_nibbles(q, b->qs, NULL);
        } else if (type == ORA_TYPE_Q4_1) {
            ora_block_q4_1 * b = (ora_block_q4_1 *)y + i;
            quantize_block_min(xb, 16, &b->d, &b->m, q);
            pack_nibbles(q, b->qs, NULL);
        } else if (type == ORA_TYPE_Q5_0) {
            ora_block_q5_0 * b = (ora_block_q5_0 *)y + i;
            quantize_block_sym(xb, 32, &b->d, q);
            pack_nibbles(q, b->qs, b->qh);
        } else {
            ora_block_q5_1 * b = (ora_block_q5_1 *)y + i;
            quantize_block_min(xb, 32, &b->d, &b->m, q);
            pack_nibbles(q, b->qs, b->qh);
        }
    }
    return 0;
}

int ora_dequantize_row(int type, const void * x, float * y, int64_t n) {
    if (type == ORA_TYPE_Q8_0) { ora_dequantize_row_q8_0((const ora_block_q8_0 *)x, y, n); return 0; }
    if (!ora_block_bytes(type)) return -2;
    uint8_t q[32];
    for (int64_t i = 0; i < n / 32; i++) {
        float * yb = y + i * 32;
        if (type == ORA_TYPE_Q4_0) {
            const ora_block_q4_0 * b = (const ora_block_q4_0 *)x + i;
            const float d = fp16_to_fp32_soft(b->d);
            unpack_nibbles(b->qs, NULL, q);
            for (int j = 0; j < 32; j++) yb[j] = (float)((int)q[j] - 8) * d;
        } else if (type == ORA_TYPE_Q4_1) {
            const ora_block_q4_1 * b = (const ora_block_q4_1 *)x + i;
            const float d = fp16_to_fp32_soft(b->d), m = fp16_to_fp32_soft(b->m);
            unpack_nibbles(b->qs, NULL, q);
            for (int j = 0; j < 32; j++) yb[j] = (float)q[j] * d + m;
        } else if (type == ORA_TYPE_Q5_0) {
            const ora_block_q5_0 * b = (const ora_block_q5_0 *)x + i;
            const float d = fp16_to_fp32_soft(b->d);
            unpack_nibbles(b->qs, b->qh, q);
            for (int j = 0; j < 32; j++) yb[j] = (float)((int)q[j] - 16) * d;
        } else {
            const ora_block_q5_1 * b = (const ora_block_q5_1 *)x + i;
            const float d = fp16_to_fp32_soft(b->d), m = fp16_to_fp32_soft(b->m);
            unpack_nibbles(b->qs, b->qh, q);
            for (int j = 0; j < 32; j++) yb[j] = (float)q[j] * d + m;
        }
    }
    return 0;
}

/* ------------------------------------------------------------------- RNG -- */

static inline uint64_t splitmix64_at(uint64_t seed, uint64_t idx) {
    uint64_t z = seed * 0xD1342543DE82EF95ull + (idx + 1) * 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

void ora_randn(uint64_t seed, int64_t n, float * out) {
    const double two_pi = 6.283185307179586476925286766559;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) {
        const uint64_t a  = splitmix64_at(seed, 2 * (uint64_t)i);
        const uint64_t b  = splitmix64_at(seed, 2 * (uint64_t)i + 1);
        const double   u1 = ((double)(a >> 11) + 1.0) * (1.0 / 9007199254740992.0); /* (0,1] */
        const double   u2 = (double)(b >> 11) * (1.0 / 9007199254740992.0);         /* [0,1) */
        out[i] = (float)(sqrt(-2.0 * log(u1)) * cos(two_pi * u2));
    }
}

int64_t ora_randint(uint64_t seed, int64_t i, int64_t lo, int64_t hi) {
    const uint64_t span = (uint64_t)(hi - lo + 1);
    return lo + (int64_t)(splitmix64_at(seed ^ 0xA5A5A5A5A5A5A5A5ull, (uint64_t)i) % span);
}

int ora_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ------------------------------------------------------- flash_attn_ext -- */

static inline const char * row_ptr(const ora_tensor * t, int64_t i1, int64_t i2, int64_t i3) {
    return (const char *)t->data + i1 * t->nb[1] + i2 * t->nb[2] + i3 * t->nb[3];
}

static int type_ok(int t) { return t == ORA_TYPE_F32 || t == ORA_TYPE_F16 || ora_block_bytes(t) != 0; }

/* one K or V row -> f32 (exact for every storage type) */
static void row_to_f32(const char * p, int type, int64_t n, float * out) {
    if (type == ORA_TYPE_F32) {
        memcpy(out, p, (size_t)n * 4);
    } else if (type == ORA_TYPE_F16) {
        const uint16_t * h = (const uint16_t *)p;
        for (int64_t i = 0; i < n; i++) out[i] = h2f(h[i]);
    } else {
        ora_dequantize_row(type, p, out, n);
    }
}

/* ALiBi slope of head h; 1 when max_bias == 0.  Every call site of the reference
 * passes max_bias = 0 (e.g. src/crispasr.cpp:2821, src/core/attention.h:992).
 * The formula is ggml's as recalled; at max_bias = 8 it is the published ALiBi head-slope
 * construction (slopes of the closest power of two, then every other slope of twice that set),
 * which is what the tests hold it to for power-of-two and other head counts. */
static float alibi_slope(float max_bias, int64_t h, int64_t n_head) {
    if (max_bias <= 0.0f) return 1.0f;
    const uint32_t n_head_log2 = 1u << (uint32_t)floor(log2((double)n_head));
    const float m0 = powf(2.0f, -(max_bias) / n_head_log2);
    const float m1 = powf(2.0f, -(max_bias / 2.0f) / n_head_log2);
    return h < (int64_t)n_head_log2 ? powf(m0, (float)(h + 1)) : powf(m1, (float)(2 * (h - n_head_log2) + 1));
}

float ora_alibi_slope(float max_bias, int64_t h, int64_t n_head) { return alibi_slope(max_bias, h, n_head); }

/* Q8_0 x Q8_0 dot product of n values, as the reference's note on its bit-matching GPU kernels describes
 * ggml_vec_dot_q8_0_q8_0_generic (tools/upstream-prs/09-metal-q8_0-bit-match.md:29-36): per block of 32 an
 * int8 x int8 -> int32 sum, then sumf += sumi * (d_x * d_y) in f32, the scales being the stored f16 values. */
static float vec_dot_q8_0_q8_0(const ora_block_q8_0 * x, const ora_block_q8_0 * y, int64_t n) {
    float sumf = 0.0f;
    for (int64_t ib = 0; ib < n / ORA_QK8_0; ib++) {
        int sumi = 0;
        for (int e = 0; e < ORA_QK8_0; e++) sumi += (int)x[ib].qs[e] * (int)y[ib].qs[e];
        sumf += (float)sumi * (h2f(x[ib].d) * h2f(y[ib].d));
    }
    return sumf;
}
float ora_vec_dot_q8_0_q8_0(const ora_block_q8_0 * x, const ora_block_q8_0 * y, int64_t n) { return vec_dot_q8_0_q8_0(x, y, n); }

typedef struct {
    const ora_tensor *q, *k, *v, *mask;
    float * dst;
    float   scale, max_bias, softcap;
    int64_t D, DV, Nq, Hq, B, Nkv, Hkv, Bk;
} fa_args;

/* fp64 two-pass softmax(scale*q.k [softcap] + slope*mask) . V, exact dequantisation.
 * Math and operand roles: src/core/fastconformer.h:883-885 (mask is added after the
 * scale), src/core/attention.h:923-933 (consecutive q heads share a kv head),
 * src/crispasr.cpp:3485-3487 (-inf mask entries are excluded keys),
 * src/crispasr.cpp:2823 + src/core/attention.h:1000 (output is [DV, Hq, Nq, B]). */
static void fa_row_exact(const fa_args * a, int64_t iq1, int64_t iq2, int64_t iq3,
                         double * s, float * tmp, double * acc) {
    const int64_t ik2 = iq2 / (a->Hq / a->Hkv);
    const int64_t ik3 = iq3 / (a->B / a->Bk);
    const float * qrow = (const float *)row_ptr(a->q, iq1, iq2, iq3);
    const uint16_t * mrow = NULL;
    if (a->mask) {
        mrow = (const uint16_t *)row_ptr(a->mask, iq1, iq2 % a->mask->ne[2], iq3 % a->mask->ne[3]);
    }
    const double slope = alibi_slope(a->max_bias, iq2, a->Hq);
    double smax = -INFINITY;
    for (int64_t j = 0; j < a->Nkv; j++) {
        double mv = 0.0;
        if (mrow) {
            mv = slope * (double)fp16_to_fp32_soft(mrow[j]);
            if (mv == -INFINITY) { s[j] = -INFINITY; continue; }
        }
        row_to_f32(row_ptr(a->k, j, ik2, ik3), a->k->type, a->D, tmp);
        double dot = 0.0;
        for (int64_t d = 0; d < a->D; d++) dot += (double)qrow[d] * (double)tmp[d];
        double sc = dot * (double)a->scale;
        if (a->softcap != 0.0f) sc = (double)a->softcap * tanh(sc / (double)a->softcap);
        sc += mv;
        s[j] = sc;
        if (sc > smax) smax = sc;
    }
    for (int64_t d = 0; d < a->DV; d++) acc[d] = 0.0;
    double sum = 0.0;
    if (smax > -INFINITY) {
        for (int64_t j = 0; j < a->Nkv; j++) {
            if (s[j] == -INFINITY) continue;
            const double p = exp(s[j] - smax);
            sum += p;
            row_to_f32(row_ptr(a->v, j, ik2, ik3), a->v->type, a->DV, tmp);
            for (int64_t d = 0; d < a->DV; d++) acc[d] += p * (double)tmp[d];
        }
    }
    float * out = a->dst + ((iq3 * a->Nq + iq1) * a->Hq + iq2) * a->DV;
    const double inv = sum > 0.0 ? 1.0 / sum : 0.0;
    for (int64_t d = 0; d < a->DV; d++) out[d] = (float)(acc[d] * inv);
}

/* f32 online softmax in key order, the way ggml-cpu walks one query row
 * (recurrence as in src/core/cpu_attention.h:53-83).  The Q row is converted to K's vec_dot_type:
 * F32 for F32/F16 K in the fork (tools/upstream-prs/01-cpu-f16-saturation.md:17-23), Q8_0 for Q8_0 K,
 * the row quantiser and the block dot product being the ones the reference's note
 * tools/upstream-prs/09-metal-q8_0-bit-match.md:24-36 writes down; that FLASH_ATTN_EXT routes a Q8_0 K
 * through them is recalled.  K of the narrower block types is not taken in this mode (ggml-cpu's integer block dot
 * products for them are written down nowhere in the reference's tree): the entry point refuses it. */
static void fa_row_ggml_like(const fa_args * a, int64_t iq1, int64_t iq2, int64_t iq3,
                             float * tmp, float * acc32, ora_block_q8_0 * qq) {
    const int64_t ik2 = iq2 / (a->Hq / a->Hkv);
    const int64_t ik3 = iq3 / (a->B / a->Bk);
    const float * qrow = (const float *)row_ptr(a->q, iq1, iq2, iq3);
    const uint16_t * mrow = NULL;
    if (a->mask) {
        mrow = (const uint16_t *)row_ptr(a->mask, iq1, iq2 % a->mask->ne[2], iq3 % a->mask->ne[3]);
    }
    const float slope = alibi_slope(a->max_bias, iq2, a->Hq);
    float scale = a->scale;
    if (a->softcap != 0.0f) scale /= a->softcap;

    const int     ktype  = a->k->type;
    const int     vtype  = a->v->type;
    const int64_t D      = a->D;
    const int64_t DV     = a->DV;

    if (ktype == ORA_TYPE_Q8_0) ora_quantize_row_q8_0(qrow, qq, D, ORA_ROUND_NEAREST_EVEN);

    float S = 0.0f;
    float M = -INFINITY;
    memset(acc32, 0, (size_t)DV * 4);

    for (int64_t j = 0; j < a->Nkv; j++) {
        const float mv = mrow ? slope * h2f(mrow[j]) : 0.0f;
        if (mv == -INFINITY) continue;

        const char * kp = row_ptr(a->k, j, ik2, ik3);
        float s = 0.0f;
        if (ktype == ORA_TYPE_F32) {
            const float * kf = (const float *)kp;
#pragma omp simd reduction(+ : s)
            for (int64_t d = 0; d < D; d++) s += kf[d] * qrow[d];
        } else if (ktype == ORA_TYPE_F16) {
            const uint16_t * kh = (const uint16_t *)kp;
#if defined(__F16C__) && defined(__AVX2__) && defined(__FMA__)
            __m256 vs = _mm256_setzero_ps();
            int64_t d = 0;
            for (; d + 8 <= D; d += 8) {
                const __m256 kf = _mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)(kh + d)));
                vs = _mm256_fmadd_ps(kf, _mm256_loadu_ps(qrow + d), vs);
            }
            __m128 lo = _mm_add_ps(_mm256_castps256_ps128(vs), _mm256_extractf128_ps(vs, 1));
            lo = _mm_add_ps(lo, _mm_movehl_ps(lo, lo));
            lo = _mm_add_ss(lo, _mm_movehdup_ps(lo));
            s = _mm_cvtss_f32(lo);
            for (; d < D; d++) s += h2f(kh[d]) * qrow[d];
#else
            for (int64_t d = 0; d < D; d++) s += h2f(kh[d]) * qrow[d];
#endif
        } else {
            s = vec_dot_q8_0_q8_0((const ora_block_q8_0 *)kp, qq, D);
        }
        s *= scale;
        if (a->softcap != 0.0f) s = a->softcap * tanhf(s);
        s += mv;

        const float Mold = M;
        float ms = 1.0f, vs = 1.0f;
        const char * vp = row_ptr(a->v, j, ik2, ik3);
        if (s > M) {
            M  = s;
            ms = expf(Mold - M);
            for (int64_t d = 0; d < DV; d++) acc32[d] *= ms;
        } else {
            vs = expf(s - M);
        }
        const float * vf;
        if (vtype == ORA_TYPE_F32) {
            vf = (const float *)vp;
        } else {
            row_to_f32(vp, vtype, DV, tmp);
            vf = tmp;
        }
        for (int64_t d = 0; d < DV; d++) acc32[d] += vf[d] * vs;
        S = S * ms + vs;
    }
    const float S_inv = S == 0.0f ? 0.0f : 1.0f / S;
    float * out = a->dst + ((iq3 * a->Nq + iq1) * a->Hq + iq2) * a->DV;
    for (int64_t d = 0; d < DV; d++) out[d] = acc32[d] * S_inv;
}

int ora_flash_attn_ext(const ora_tensor * q, const ora_tensor * k, const ora_tensor * v,
                       const ora_tensor * mask, float * dst,
                       float scale, float max_bias, float logit_softcap,
                       int mode, int n_threads) {
    if (!q || !k || !v || !dst) return -1;
    if (mask && !mask->data) mask = NULL;
    if (q->type != ORA_TYPE_F32 || !type_ok(k->type) || !type_ok(v->type)) return -2;
    if (mask && mask->type != ORA_TYPE_F16) return -2;

    fa_args a;
    a.q = q; a.k = k; a.v = v; a.mask = mask; a.dst = dst;
    a.scale = scale; a.max_bias = max_bias; a.softcap = logit_softcap;
    a.D = q->ne[0]; a.Nq = q->ne[1]; a.Hq = q->ne[2]; a.B = q->ne[3];
    a.DV = v->ne[0]; a.Nkv = k->ne[1]; a.Hkv = k->ne[2]; a.Bk = k->ne[3];

    /* contract of the constructor (ggml_flash_attn_ext), as the call sites use it */
    if (k->ne[0] != a.D || v->ne[1] != a.Nkv || v->ne[2] != a.Hkv || v->ne[3] != a.Bk) return -3;
    if (a.Hkv <= 0 || a.Bk <= 0 || a.Hq % a.Hkv != 0 || a.B % a.Bk != 0) return -3;
    if ((ora_block_bytes(k->type) && a.D % ORA_QK8_0) || (ora_block_bytes(v->type) && a.DV % ORA_QK8_0)) return -3;
    if (a.D > 512) return -3;
    if (mask) {
        if (mask->ne[0] < a.Nkv || mask->ne[1] < a.Nq) return -4;
        if (a.Hq % mask->ne[2] != 0 || a.B % mask->ne[3] != 0) return -4;
        if (mask->nb[0] != 2) return -4;
    }
    if (max_bias > 0.0f && !mask) return -5;
    if (q->nb[0] != 4) return -6;
    if (mode != ORA_MODE_EXACT && mode != ORA_MODE_GGML_LIKE) return -7;
    /* ggml-like mode takes K as F32, F16 or Q8_0: nothing in the reference's tree says how ggml-cpu multiplies a query row
     * with Q4_0 .. Q5_1 blocks */
    if (mode == ORA_MODE_GGML_LIKE && ora_block_bytes(k->type) && k->type != ORA_TYPE_Q8_0) return -7;

    const int64_t n_rows = a.Nq * a.Hq * a.B;
    int nt = n_threads > 0 ? n_threads : 1;
#ifndef _OPENMP
    nt = 1;
#endif

#pragma omp parallel num_threads(nt)
    {
        const int64_t Dm = a.D > a.DV ? a.D : a.DV;
        double *        s     = mode == ORA_MODE_EXACT ? (double *)malloc((size_t)(a.Nkv > 0 ? a.Nkv : 1) * 8) : NULL;
        double *        acc   = (double *)malloc((size_t)Dm * 8);
        float *         tmp   = (float *)malloc((size_t)Dm * 4);
        float *         acc32 = (float *)malloc((size_t)Dm * 4);
        ora_block_q8_0 * qq   = (ora_block_q8_0 *)malloc(sizeof(ora_block_q8_0) * (size_t)(a.D / ORA_QK8_0 + 1));
#pragma omp for schedule(dynamic, 16)
        for (int64_t ir = 0; ir < n_rows; ir++) {
            const int64_t iq3 = ir / (a.Hq * a.Nq);
            const int64_t iq2 = (ir - iq3 * a.Hq * a.Nq) / a.Nq;
            const int64_t iq1 = ir - iq3 * a.Hq * a.Nq - iq2 * a.Nq;
            if (mode == ORA_MODE_EXACT) {
                fa_row_exact(&a, iq1, iq2, iq3, s, tmp, acc);
            } else {
                fa_row_ggml_like(&a, iq1, iq2, iq3, tmp, acc32, qq);
            }
        }
        free(s); free(acc); free(tmp); free(acc32); free(qq);
    }
    return 0;
}

/* --------------------------------------------------------- KV-cache write -- */

/* ggml_cpy of an F32 tensor into a view of the KV cache (src/crispasr.cpp:2810-2811,
 * 3185-3203; src/core/attention.h:342-378, 850-867).  Element (i0,i1,i2,i3) of src goes
 * to the same index of dst; for Q8_0 a dst row is ne0/32 consecutive blocks. */
int ora_cpy_f32(const ora_tensor * src, void * dst_data, int32_t dst_type, const int64_t dst_nb[4],
                int rounding) {
    if (!src || src->type != ORA_TYPE_F32 || !type_ok(dst_type)) return -2;
    if (ora_block_bytes(dst_type) && src->ne[0] % ORA_QK8_0) return -3;
    const int64_t n0 = src->ne[0];
    float * tmp = (float *)malloc((size_t)(n0 > 0 ? n0 : 1) * 4);
    for (int64_t i3 = 0; i3 < src->ne[3]; i3++)
    for (int64_t i2 = 0; i2 < src->ne[2]; i2++)
    for (int64_t i1 = 0; i1 < src->ne[1]; i1++) {
        const char * sp = (const char *)src->data + i1 * src->nb[1] + i2 * src->nb[2] + i3 * src->nb[3];
        char *       dp = (char *)dst_data + i1 * dst_nb[1] + i2 * dst_nb[2] + i3 * dst_nb[3];
        for (int64_t i0 = 0; i0 < n0; i0++) tmp[i0] = *(const float *)(sp + i0 * src->nb[0]);
        if (dst_type == ORA_TYPE_F32) {
            for (int64_t i0 = 0; i0 < n0; i0++) *(float *)(dp + i0 * dst_nb[0]) = tmp[i0];
        } else if (dst_type == ORA_TYPE_F16) {
            for (int64_t i0 = 0; i0 < n0; i0++) *(uint16_t *)(dp + i0 * dst_nb[0]) = fp32_to_fp16_soft(tmp[i0]);
        } else if (dst_type == ORA_TYPE_Q8_0) {
            ora_quantize_row_q8_0(tmp, (ora_block_q8_0 *)dp, n0, rounding);
        } else {
            ora_quantize_row(dst_type, tmp, dp, n0);
        }
    }
    free(tmp);
    return 0;
}

/* ------------------------------------------------ FastConformer rel-pos mask -- */

/* The F16 mask that core_conformer::build_block hands to ggml_flash_attn_ext, restated node by
 * node (src/core/fastconformer.h:876-918):
 *   BD_raw    = ggml_mul_mat(ggml_cont(R), Q_v)      ne = [NR, Nq, H], NR = 2T-1 (here Nq+Nkv-1)
 *   BD        = rel_shift(BD_raw)                    a VIEW (fastconformer.h:98-102): ne = [T, T, H],
 *                                                    nb1 = nb1_raw - nb0, nb2 = nb2_raw, offset (T-1)*nb0
 *   BD_scaled = ggml_scale(ggml_cont(BD), scale)     f32
 *   BD_scaled = ggml_add(BD_scaled, local_attn_mask) optional f32 [T, T] (0 / -inf / -1e9), all heads
 *   BD_mask   = ggml_cast(BD_scaled, F16)            round to nearest even, overflow to -inf
 * The view is applied literally, as byte offsets into the BD_raw buffer, so that its index map
 * (element (j, i) of BD = element (T-1+j-i, i) of BD_raw) is a consequence, not an assumption.
 * The dot products are accumulated in double and rounded once to f32 (ggml's own summation order
 * inside mul_mat is not fixed by anything in the reference's tree).
 * Generalised to Nq != Nkv: the view offset is (Nq-1)*nb0 and NR = Nq+Nkv-1.
 * dst: f16 [Nkv, Nq, H, B] contiguous.  add may be NULL; F32 or F16, ne = [Nkv, Nq, 1|H, 1|B]. */
int ora_relpos_bias(const ora_tensor * qv, const ora_tensor * r, const ora_tensor * add,
                    float scale, int64_t n_kv, uint16_t * dst, int n_threads) {
    if (!qv || !r || !dst) return -1;
    if (add && !add->data) add = NULL;
    if (qv->type != ORA_TYPE_F32 || (r->type != ORA_TYPE_F32 && r->type != ORA_TYPE_F16)) return -2;
    if (add && add->type != ORA_TYPE_F32 && add->type != ORA_TYPE_F16) return -2;
    const int64_t D = qv->ne[0], Nq = qv->ne[1], H = qv->ne[2], B = qv->ne[3];
    const int64_t NR = Nq + n_kv - 1;
    if (r->ne[0] != D || r->ne[1] != NR || r->ne[2] <= 0 || r->ne[3] <= 0 || H % r->ne[2] || B % r->ne[3]) return -3;
    if (add && (add->ne[0] < n_kv || add->ne[1] < Nq || H % add->ne[2] || B % add->ne[3])) return -4;
    int nt = n_threads > 0 ? n_threads : 1;
#ifndef _OPENMP
    nt = 1;
#endif
#pragma omp parallel num_threads(nt)
    {
        float * raw  = (float *)malloc((size_t)(NR * Nq > 0 ? NR * Nq : 1) * sizeof(float));
        float * qrow = (float *)malloc((size_t)(D > 0 ? D : 1) * sizeof(float));
        float * rrow = (float *)malloc((size_t)(D > 0 ? D : 1) * sizeof(float));
#pragma omp for schedule(dynamic, 1)
        for (int64_t hb = 0; hb < H * B; hb++) {
            const int64_t h = hb % H, b = hb / H;
            /* BD_raw[p, i] = <R[:, p], Q_v[:, i]>, contiguous: nb0 = 4, nb1 = NR*4 */
            for (int64_t i = 0; i < Nq; i++) {
                row_to_f32(row_ptr(qv, i, h, b), ORA_TYPE_F32, D, qrow);
                for (int64_t p = 0; p < NR; p++) {
                    row_to_f32(row_ptr(r, p, h % r->ne[2], b % r->ne[3]), r->type, D, rrow);
                    double acc = 0.0;
                    for (int64_t d = 0; d < D; d++) acc += (double)rrow[d] * (double)qrow[d];
                    raw[i * NR + p] = (float)acc;
                }
            }
            /* the rel_shift view of that buffer, then scale, add, cast */
            const int64_t nb0 = 4, nb1 = NR * 4 - nb0, off = (Nq - 1) * nb0;
            for (int64_t i = 0; i < Nq; i++)
                for (int64_t j = 0; j < n_kv; j++) {
                    const float bd = *(const float *)((const char *)raw + off + j * nb0 + i * nb1);
                    float x = bd * scale;
                    if (add) {
                        const char * ap = (const char *)add->data + j * add->nb[0] + i * add->nb[1] +
                                          (h % add->ne[2]) * add->nb[2] + (b % add->ne[3]) * add->nb[3];
                        x += add->type == ORA_TYPE_F32 ? *(const float *)ap : h2f(*(const uint16_t *)ap);
                    }
                    dst[((b * H + h) * Nq + i) * n_kv + j] = f2h(x);
                }
        }
        free(raw); free(qrow); free(rrow);
    }
    return 0;
}
