/*
 * oracle.c -- CPU restatement of the reference's quantized MUL_MAT path (see oracle.h for scope and pinning).
 * TEST INFRASTRUCTURE ONLY: never linked into, loaded by, or used as a fallback for the product library.
 *
 * Reference paths are relative to the reference's cactus/ directory.  Build with -ffp-contract=off: the only
 * fused multiply-adds are the explicit fmaf() calls that mirror the reference's _mm256_fmadd_ps/_mm_fmadd_ps.
 */
#include "oracle.h"

#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

/* ---------------------------------------------------------------- block layouts (ggml-common.h:167-172,
 * 209-214, 285-296, 320-326, 329-334).  On-disk == in-memory; all little endian. */
#pragma pack(push, 1)
typedef struct { uint16_t d; uint8_t qs[16]; } blk_q4_0;
typedef struct { uint16_t d; int8_t qs[32]; } blk_q8_0;
typedef struct { uint16_t d; uint16_t dmin; uint8_t scales[12]; uint8_t qs[128]; } blk_q4_K;
typedef struct { uint8_t ql[128]; uint8_t qh[64]; int8_t scales[16]; uint16_t d; } blk_q6_K;
typedef struct { float d; int8_t qs[256]; int16_t bsums[16]; } blk_q8_K;
/* further weight types: ggml-common.h:187-193 (q5_0), :303-314 (q5_K), :405-410 (iq4_nl) */
typedef struct { uint16_t d; uint8_t qh[4]; uint8_t qs[16]; } blk_q5_0;
typedef struct { uint16_t d; uint16_t dmin; uint8_t scales[12]; uint8_t qh[32]; uint8_t qs[128]; } blk_q5_K;
typedef struct { uint16_t d; uint8_t qs[16]; } blk_iq4_nl;
/* min-based types and their activation format: ggml-common.h:175-185 (q4_1), :196-207 (q5_1), :216-227 (q8_1) */
typedef struct { uint16_t d; uint16_t m; uint8_t qs[16]; } blk_q4_1;
typedef struct { uint16_t d; uint16_t m; uint8_t qh[4]; uint8_t qs[16]; } blk_q5_1;
typedef struct { uint16_t d; uint16_t s; int8_t qs[32]; } blk_q8_1;
/* 2- and 3-bit K-quants: ggml-common.h:254-266 (q2_K), :273-278 (q3_K) */
typedef struct { uint8_t scales[16]; uint8_t qs[64]; uint16_t d; uint16_t dmin; } blk_q2_K;
typedef struct { uint8_t hmask[32]; uint8_t qs[64]; uint8_t scales[12]; uint16_t d; } blk_q3_K;
/* ggml-common.h:412-417: the non-linear 4-bit code points with 6-bit sub-block scales */
typedef struct { uint16_t d; uint16_t scales_h; uint8_t scales_l[4]; uint8_t qs[128]; } blk_iq4_xs;
#pragma pack(pop)

_Static_assert(sizeof(blk_q4_0) == 18, "q4_0");
_Static_assert(sizeof(blk_q8_0) == 34, "q8_0");
_Static_assert(sizeof(blk_q4_K) == 144, "q4_K");
_Static_assert(sizeof(blk_q6_K) == 210, "q6_K");
_Static_assert(sizeof(blk_q8_K) == 292, "q8_K");
_Static_assert(sizeof(blk_q5_0) == 22, "q5_0");
_Static_assert(sizeof(blk_q5_K) == 176, "q5_K");
_Static_assert(sizeof(blk_iq4_nl) == 18, "iq4_nl");
_Static_assert(sizeof(blk_q4_1) == 20, "q4_1");
_Static_assert(sizeof(blk_q5_1) == 24, "q5_1");
_Static_assert(sizeof(blk_q8_1) == 36, "q8_1");
_Static_assert(sizeof(blk_q2_K) == 84, "q2_K");
_Static_assert(sizeof(blk_q3_K) == 110, "q3_K");
_Static_assert(sizeof(blk_iq4_xs) == 136, "iq4_xs");

/* ggml-quants.c:2428: the 16 code points of the non-linear 4-bit types. */
static const int8_t iq4nl_values[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};

int orc_block_elems(int type) {
    switch (type) {
        case ORC_TYPE_F32: case ORC_TYPE_F16: return 1;
        case ORC_TYPE_Q4_0: case ORC_TYPE_Q8_0: case ORC_TYPE_Q5_0: case ORC_TYPE_IQ4_NL:
        case ORC_TYPE_Q4_1: case ORC_TYPE_Q5_1: case ORC_TYPE_Q8_1: return 32;
        case ORC_TYPE_Q4_K: case ORC_TYPE_Q5_K: case ORC_TYPE_Q6_K: case ORC_TYPE_Q8_K: return 256;
        case ORC_TYPE_Q2_K: case ORC_TYPE_Q3_K: case ORC_TYPE_IQ4_XS: return 256;
        default: return 0;
    }
}
size_t orc_block_bytes(int type) {
    switch (type) {
        case ORC_TYPE_F32: return 4;
        case ORC_TYPE_F16: return 2;
        case ORC_TYPE_Q4_0: return 18;
        case ORC_TYPE_Q8_0: return 34;
        case ORC_TYPE_Q4_K: return 144;
        case ORC_TYPE_Q6_K: return 210;
        case ORC_TYPE_Q8_K: return 292;
        case ORC_TYPE_Q5_0: return 22;
        case ORC_TYPE_Q5_K: return 176;
        case ORC_TYPE_IQ4_NL: return 18;
        case ORC_TYPE_Q4_1: return 20;
        case ORC_TYPE_Q5_1: return 24;
        case ORC_TYPE_Q8_1: return 36;
        case ORC_TYPE_Q2_K: return 84;
        case ORC_TYPE_Q3_K: return 110;
        case ORC_TYPE_IQ4_XS: return 136;
        default: return 0;
    }
}
size_t orc_row_size(int type, int64_t k) {
    int be = orc_block_elems(type);
    return be ? (size_t)(k / be) * orc_block_bytes(type) : 0;
}
int orc_vec_dot_type(int type) {
    switch (type) { /* ggml-cpu/ggml-cpu.c:213,245,272,284; :229 (q5_0), :278 (q5_K), :340 (iq4_nl) */
        case ORC_TYPE_Q4_0: case ORC_TYPE_Q8_0: case ORC_TYPE_Q5_0: case ORC_TYPE_IQ4_NL: return ORC_TYPE_Q8_0;
        case ORC_TYPE_Q4_K: case ORC_TYPE_Q5_K: case ORC_TYPE_Q6_K: return ORC_TYPE_Q8_K;
        case ORC_TYPE_Q2_K: case ORC_TYPE_Q3_K: return ORC_TYPE_Q8_K;   /* ggml-cpu/ggml-cpu.c:257-268 */
        case ORC_TYPE_IQ4_XS: return ORC_TYPE_Q8_K;                     /* ggml-cpu/ggml-cpu.c:340-345 */
        case ORC_TYPE_Q4_1: case ORC_TYPE_Q5_1: return ORC_TYPE_Q8_1;   /* ggml-cpu/ggml-cpu.c:221,237 */
        case ORC_TYPE_F16: return ORC_TYPE_F16;                        /* ggml-cpu/ggml-cpu.c:204-209 */
        default: return -1;
    }
}

/* ---------------------------------------------------------------- fp16 <-> fp32, IEEE round-to-nearest-even.
 * The x86 reference uses the F16C instructions (ggml-impl.h:346-353) and a 65536-entry table filled with
 * them (ggml.c:1418-1431); both are plain IEEE conversions, restated here in integer arithmetic. */
static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

float orc_fp16_to_fp32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp  = (h >> 10) & 0x1f;
    uint32_t man  = h & 0x3ffu;
    if (exp == 0) {
        if (man == 0) return u2f(sign);
        /* subnormal half: value = man * 2^-24, exact in fp32 */
        float v = (float)man * 0x1.0p-24f;
        return u2f(f2u(v) | sign);
    }
    if (exp == 31) return u2f(sign | 0x7f800000u | (man << 13));
    return u2f(sign | ((exp + 112u) << 23) | (man << 13));
}

uint16_t orc_fp32_to_fp16(float f) {
    uint32_t u = f2u(f);
    uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((a >> 13) & 0x3ffu)); /* NaN (quieted) */
    if (a >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);   /* >= 65520 rounds to inf */
    if (a < 0x33000001u) return sign;                            /* <= 2^-25 rounds to zero (tie -> even 0) */
    int32_t e = (int32_t)(a >> 23) - 127;
    uint32_t m = (a & 0x7fffffu) | 0x800000u;                    /* 24-bit significand */
    int shift;                                                   /* bits dropped from m */
    uint32_t base;
    if (e >= -14) { shift = 13; base = (uint32_t)(e + 15) << 10; m &= 0x7fffffu; }
    else          { shift = 13 + (-14 - e); base = 0; }
    uint32_t q = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) q++;
    return (uint16_t)(sign | (base + q));                        /* carry out of q bumps the exponent */
}

#define H2F(h) orc_fp16_to_fp32(h)
#define F2H(f) orc_fp32_to_fp16(f)

/* ggml-quants.c:366-371: round to nearest (ties to even) through the 1.5*2^23 magic constant. */
static inline int nearest_i(float v) {
    float t = v + 12582912.f;
    return (int)(f2u(t) & 0x007fffffu) - 0x00400000;
}
static inline int imin_(int a, int b) { return a < b ? a : b; }
static inline int imax_(int a, int b) { return a > b ? a : b; }

/* ---------------------------------------------------------------- activation quantizers */

/* ggml-cpu/ggml-cpu-quants.c:802-885 (AVX2 branch of quantize_row_q8_0):
 *   d = amax/127 ; id = amax != 0 ? 127/amax : 0 ; q = round_half_even(x*id).
 * This differs from the scalar _ref (id = 1/d, roundf) in the last ulp of id and on exact .5 ties. */
void orc_quantize_row_q8_0(const float *x, void *vy, int64_t k) {
    blk_q8_0 *y = (blk_q8_0 *)vy;
    for (int64_t b = 0; b < k / 32; b++, x += 32) {
        float amax = 0.0f;
        for (int j = 0; j < 32; j++) { float a = fabsf(x[j]); if (a > amax) amax = a; }
        const float d = amax / 127.f;
        const float id = amax != 0.0f ? 127.f / amax : 0.0f;
        y[b].d = F2H(d);
        for (int j = 0; j < 32; j++) {
            const float r = nearbyintf(x[j] * id);    /* default rounding mode: to nearest even */
            /* cvtps_epi32 turns NaN and anything outside int32 into 0x80000000 ("integer indefinite"),
             * which the two saturating packs carry down to -128; reachable when 127/amax overflows. */
            const int q = fabsf(r) < 2147483648.f ? (int)r : INT32_MIN;
            y[b].qs[j] = (int8_t)imax_(-128, imin_(127, q));
        }
    }
}

/* ggml-cpu/ggml-cpu-quants.c:1047-1140 (AVX2 branch of quantize_row_q8_1): the quants and d are those of
 * quantize_row_q8_0; s = fp16(d * sum) with the *unrounded* fp32 d and the sum of the 32 int32 conversion
 * results before the saturating packs (wrapping 32-bit adds), :1094. */
void orc_quantize_row_q8_1(const float *x, void *vy, int64_t k) {
    blk_q8_1 *y = (blk_q8_1 *)vy;
    for (int64_t b = 0; b < k / 32; b++, x += 32) {
        float amax = 0.0f;
        for (int j = 0; j < 32; j++) { float a = fabsf(x[j]); if (a > amax) amax = a; }
        const float d = amax / 127.f;
        const float id = amax != 0.0f ? 127.f / amax : 0.0f;
        y[b].d = F2H(d);
        uint32_t sum = 0;
        for (int j = 0; j < 32; j++) {
            const float r = nearbyintf(x[j] * id);
            const int q = fabsf(r) < 2147483648.f ? (int)r : INT32_MIN;
            sum += (uint32_t)q;
            y[b].qs[j] = (int8_t)imax_(-128, imin_(127, q));
        }
        y[b].s = F2H(d * (float)(int32_t)sum);
    }
}

/* F16 weights: activations are converted to fp16, round to nearest even (lm_ggml_cpu_fp32_to_fp16,
 * ggml-cpu/ggml-cpu.c:3161-3190: F16C _mm256_cvtps_ph / _mm_cvtps_ph with _MM_FROUND_TO_NEAREST_INT); weights made
 * from fp32 the same way (lm_ggml_fp32_to_fp16_row, ggml.c:417-422). */
void orc_fp32_to_fp16_row(const float *x, void *vy, int64_t k) {
    uint16_t *y = (uint16_t *)vy;
    for (int64_t i = 0; i < k; i++) y[i] = F2H(x[i]);
}

/* ggml-quants.c:188-211 (scalar reference, used for Q8_0 *weights*). */
void orc_quantize_row_q8_0_ref(const float *x, void *vy, int64_t k) {
    blk_q8_0 *y = (blk_q8_0 *)vy;
    for (int64_t b = 0; b < k / 32; b++, x += 32) {
        float amax = 0.0f;
        for (int j = 0; j < 32; j++) { float a = fabsf(x[j]); if (a > amax) amax = a; }
        const float d = amax / 127;
        const float id = d ? 1.0f / d : 0.0f;
        y[b].d = F2H(d);
        for (int j = 0; j < 32; j++) y[b].qs[j] = (int8_t)roundf(x[j] * id);
    }
}

/* ggml-cpu/ggml-cpu-quants.c:1740,1819-1821 -> ggml-quants.c:2473-2510.  An all-zero block leaves bsums
 * unwritten in the reference (they are multiplied by d == 0 downstream); here they are set to 0. */
void orc_quantize_row_q8_K(const float *x, void *vy, int64_t k) {
    blk_q8_K *y = (blk_q8_K *)vy;
    for (int64_t b = 0; b < k / 256; b++, x += 256) {
        float amax = 0.0f, mx = 0.0f;
        for (int j = 0; j < 256; j++) {
            float a = fabsf(x[j]);
            if (a > amax) { amax = a; mx = x[j]; }    /* strict >: the first largest wins, sign kept */
        }
        if (amax == 0.0f) { memset(&y[b], 0, sizeof(blk_q8_K)); continue; }
        const float iscale = -127.f / mx;
        for (int j = 0; j < 256; j++) y[b].qs[j] = (int8_t)imin_(127, nearest_i(iscale * x[j]));
        for (int g = 0; g < 16; g++) {
            int s = 0;
            for (int j = 0; j < 16; j++) s += y[b].qs[16 * g + j];
            y[b].bsums[g] = (int16_t)s;
        }
        y[b].d = 1 / iscale;
    }
}

/* ---------------------------------------------------------------- weight quantizers */

/* ggml-quants.c:25-60. */
void orc_quantize_row_q4_0_ref(const float *x, void *vy, int64_t k) {
    blk_q4_0 *y = (blk_q4_0 *)vy;
    for (int64_t b = 0; b < k / 32; b++, x += 32) {
        float amax = 0.0f, mx = 0.0f;
        for (int j = 0; j < 32; j++) {
            if (amax < fabsf(x[j])) { amax = fabsf(x[j]); mx = x[j]; }
        }
        const float d = mx / -8;
        const float id = d ? 1.0f / d : 0.0f;
        y[b].d = F2H(d);
        for (int j = 0; j < 16; j++) {
            const float lo = x[j] * id, hi = x[j + 16] * id;
            const uint8_t qlo = (uint8_t)imin_(15, (int8_t)(lo + 8.5f));
            const uint8_t qhi = (uint8_t)imin_(15, (int8_t)(hi + 8.5f));
            y[b].qs[j] = (uint8_t)(qlo | (qhi << 4));
        }
    }
}

/* ggml-quants.c:544-623 with n=32, use_mad=false.  quantize_row_q4_K_ref passes nmax=15, rmin=-1, rdelta=0.1,
 * nstep=20 (:1221); quantize_row_q5_K_ref passes nmax=31, rmin=-0.5, rdelta=0.1, nstep=15 (:1409).
 * Returns the scale, writes -min to *neg_min. */
static float fit_scale_min_32(const float *x, const float *w, uint8_t *L, float *neg_min, uint8_t *Laux,
                              int nmax, float rmin, float rdelta, int nstep) {
    const int n = 32;
    float lo = x[0], hi = x[0];
    float sum_w = w[0];
    float sum_x = sum_w * x[0];
    for (int i = 1; i < n; i++) {
        if (x[i] < lo) lo = x[i];
        if (x[i] > hi) hi = x[i];
        sum_w += w[i];
        sum_x += w[i] * x[i];
    }
    if (lo > 0) lo = 0;
    if (hi == lo) {
        for (int i = 0; i < n; i++) L[i] = 0;
        *neg_min = -lo;
        return 0.f;
    }
    float iscale = nmax / (hi - lo);
    float scale = 1 / iscale;
    float best = 0;
    for (int i = 0; i < n; i++) {
        int l = nearest_i(iscale * (x[i] - lo));
        L[i] = (uint8_t)imax_(0, imin_(nmax, l));
        float diff = scale * L[i] + lo - x[i];
        diff = diff * diff;
        best += w[i] * diff;
    }
    for (int is = 0; is <= nstep; is++) {
        iscale = (rmin + rdelta * is + nmax) / (hi - lo);
        float sum_l = 0, sum_l2 = 0, sum_xl = 0;
        for (int i = 0; i < n; i++) {
            int l = nearest_i(iscale * (x[i] - lo));
            l = imax_(0, imin_(nmax, l));
            Laux[i] = (uint8_t)l;
            sum_l  += w[i] * l;
            sum_l2 += w[i] * l * l;
            sum_xl += w[i] * l * x[i];
        }
        float D = sum_w * sum_l2 - sum_l * sum_l;
        if (D > 0) {
            float s = (sum_w * sum_xl - sum_x * sum_l) / D;
            float m = (sum_l2 * sum_x - sum_l * sum_xl) / D;
            if (m > 0) { m = 0; s = sum_xl / sum_l2; }
            float mad = 0;
            for (int i = 0; i < n; i++) {
                float diff = s * Laux[i] + m - x[i];
                diff = diff * diff;
                mad += w[i] * diff;
            }
            if (mad < best) {
                for (int i = 0; i < n; i++) L[i] = Laux[i];
                best = mad; scale = s; lo = m;
            }
        }
    }
    *neg_min = -lo;
    return scale;
}

/* ggml-quants.c:625-632: 6-bit scale and min of sub-block j from the 12 packed bytes. */
static inline void unpack_sc_m(int j, const uint8_t *q, uint8_t *sc, uint8_t *m) {
    if (j < 4) { *sc = q[j] & 63; *m = q[j + 4] & 63; }
    else {
        *sc = (uint8_t)((q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4));
        *m  = (uint8_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4));
    }
}

/* ggml-quants.c:1202-1272. */
void orc_quantize_row_q4_K_ref(const float *x, void *vy, int64_t k) {
    blk_q4_K *y = (blk_q4_K *)vy;
    uint8_t L[256], Laux[32];
    float w[32], mins[8], scales[8];
    for (int64_t b = 0; b < k / 256; b++, x += 256) {
        float max_scale = 0, max_min = 0;
        for (int j = 0; j < 8; j++) {
            const float *xs = x + 32 * j;
            float sum_x2 = 0;
            for (int l = 0; l < 32; l++) sum_x2 += xs[l] * xs[l];
            float av = sqrtf(sum_x2 / 32);
            for (int l = 0; l < 32; l++) w[l] = av + fabsf(xs[l]);
            scales[j] = fit_scale_min_32(xs, w, L + 32 * j, &mins[j], Laux, 15, -1.f, 0.1f, 20);
            if (scales[j] > max_scale) max_scale = scales[j];
            if (mins[j] > max_min) max_min = mins[j];
        }
        const float inv_scale = max_scale > 0 ? 63.f / max_scale : 0.f;
        const float inv_min   = max_min   > 0 ? 63.f / max_min   : 0.f;
        for (int j = 0; j < 8; j++) {
            uint8_t ls = (uint8_t)nearest_i(inv_scale * scales[j]);
            uint8_t lm = (uint8_t)nearest_i(inv_min * mins[j]);
            if (ls > 63) ls = 63;
            if (lm > 63) lm = 63;
            if (j < 4) { y[b].scales[j] = ls; y[b].scales[j + 4] = lm; }
            else {
                y[b].scales[j + 4] = (uint8_t)((ls & 0xF) | ((lm & 0xF) << 4));
                y[b].scales[j - 4] |= (uint8_t)((ls >> 4) << 6);
                y[b].scales[j]     |= (uint8_t)((lm >> 4) << 6);
            }
        }
        y[b].d    = F2H(max_scale / 63.f);
        y[b].dmin = F2H(max_min / 63.f);
        for (int j = 0; j < 8; j++) {
            uint8_t sc, m;
            unpack_sc_m(j, y[b].scales, &sc, &m);
            const float d = H2F(y[b].d) * sc;
            if (!d) continue;
            const float dm = H2F(y[b].dmin) * m;
            for (int i = 0; i < 32; i++) {
                int l = nearest_i((x[32 * j + i] + dm) / d);
                L[32 * j + i] = (uint8_t)imax_(0, imin_(15, l));
            }
        }
        uint8_t *q = y[b].qs;
        for (int j = 0; j < 256; j += 64, q += 32)
            for (int l = 0; l < 32; l++) q[l] = (uint8_t)(L[j + l] | (L[j + l + 32] << 4));
    }
}

/* ggml-quants.c:1389-1474. */
void orc_quantize_row_q5_K_ref(const float *x, void *vy, int64_t k) {
    blk_q5_K *y = (blk_q5_K *)vy;
    uint8_t L[256], Laux[32];
    float w[32], mins[8], scales[8];
    for (int64_t b = 0; b < k / 256; b++, x += 256) {
        float max_scale = 0, max_min = 0;
        for (int j = 0; j < 8; j++) {
            const float *xs = x + 32 * j;
            float sum_x2 = 0;
            for (int l = 0; l < 32; l++) sum_x2 += xs[l] * xs[l];
            float av = sqrtf(sum_x2 / 32);
            for (int l = 0; l < 32; l++) w[l] = av + fabsf(xs[l]);
            scales[j] = fit_scale_min_32(xs, w, L + 32 * j, &mins[j], Laux, 31, -0.5f, 0.1f, 15);
            if (scales[j] > max_scale) max_scale = scales[j];
            if (mins[j] > max_min) max_min = mins[j];
        }
        const float inv_scale = max_scale > 0 ? 63.f / max_scale : 0.f;
        const float inv_min   = max_min   > 0 ? 63.f / max_min   : 0.f;
        for (int j = 0; j < 8; j++) {
            uint8_t ls = (uint8_t)nearest_i(inv_scale * scales[j]);
            uint8_t lm = (uint8_t)nearest_i(inv_min * mins[j]);
            if (ls > 63) ls = 63;
            if (lm > 63) lm = 63;
            if (j < 4) { y[b].scales[j] = ls; y[b].scales[j + 4] = lm; }
            else {
                y[b].scales[j + 4] = (uint8_t)((ls & 0xF) | ((lm & 0xF) << 4));
                y[b].scales[j - 4] |= (uint8_t)((ls >> 4) << 6);
                y[b].scales[j]     |= (uint8_t)((lm >> 4) << 6);
            }
        }
        y[b].d    = F2H(max_scale / 63.f);
        y[b].dmin = F2H(max_min / 63.f);
        for (int j = 0; j < 8; j++) {
            uint8_t sc, m;
            unpack_sc_m(j, y[b].scales, &sc, &m);
            const float d = H2F(y[b].d) * sc;
            if (!d) continue;
            const float dm = H2F(y[b].dmin) * m;
            for (int i = 0; i < 32; i++) {
                int l = nearest_i((x[32 * j + i] + dm) / d);
                L[32 * j + i] = (uint8_t)imax_(0, imin_(31, l));
            }
        }
        memset(y[b].qh, 0, 32);
        uint8_t *ql = y[b].qs;
        uint8_t m1 = 1, m2 = 2;
        for (int n = 0; n < 256; n += 64, ql += 32) {
            for (int j = 0; j < 32; j++) {
                int l1 = L[n + j], l2 = L[n + j + 32];
                if (l1 > 15) { l1 -= 16; y[b].qh[j] |= m1; }
                if (l2 > 15) { l2 -= 16; y[b].qh[j] |= m2; }
                ql[j] = (uint8_t)(l1 | (l2 << 4));
            }
            m1 = (uint8_t)(m1 << 2); m2 = (uint8_t)(m2 << 2);
        }
    }
}

/* ggml-quants.c:62-97. */
void orc_quantize_row_q4_1_ref(const float *x, void *vy, int64_t k) {
    blk_q4_1 *y = (blk_q4_1 *)vy;
    for (int64_t b = 0; b < k / 32; b++, x += 32) {
        float mn = 3.402823466e+38f, mx = -3.402823466e+38f;
        for (int j = 0; j < 32; j++) { if (x[j] < mn) mn = x[j]; if (x[j] > mx) mx = x[j]; }
        const float d = (mx - mn) / 15;
        const float id = d ? 1.0f / d : 0.0f;
        y[b].d = F2H(d);
        y[b].m = F2H(mn);
        for (int j = 0; j < 16; j++) {
            const float x0 = (x[j] - mn) * id, x1 = (x[16 + j] - mn) * id;
            const uint8_t xi0 = (uint8_t)imin_(15, (int8_t)(x0 + 0.5f));
            const uint8_t xi1 = (uint8_t)imin_(15, (int8_t)(x1 + 0.5f));
            y[b].qs[j] = (uint8_t)(xi0 | (xi1 << 4));
        }
    }
}

/* ggml-quants.c:143-186. */
void orc_quantize_row_q5_1_ref(const float *x, void *vy, int64_t k) {
    blk_q5_1 *y = (blk_q5_1 *)vy;
    for (int64_t b = 0; b < k / 32; b++, x += 32) {
        float mn = 3.402823466e+38f, mx = -3.402823466e+38f;
        for (int j = 0; j < 32; j++) { if (x[j] < mn) mn = x[j]; if (x[j] > mx) mx = x[j]; }
        const float d = (mx - mn) / 31;
        const float id = d ? 1.0f / d : 0.0f;
        y[b].d = F2H(d);
        y[b].m = F2H(mn);
        uint32_t qh = 0;
        for (int j = 0; j < 16; j++) {
            const float x0 = (x[j] - mn) * id, x1 = (x[16 + j] - mn) * id;
            const uint8_t xi0 = (uint8_t)(x0 + 0.5f), xi1 = (uint8_t)(x1 + 0.5f);
            y[b].qs[j] = (uint8_t)((xi0 & 0x0F) | ((xi1 & 0x0F) << 4));
            qh |= ((xi0 & 0x10u) >> 4) << (j + 0);
            qh |= ((xi1 & 0x10u) >> 4) << (j + 16);
        }
        memcpy(y[b].qh, &qh, 4);
    }
}

/* ggml-quants.c:99-141. */
void orc_quantize_row_q5_0_ref(const float *x, void *vy, int64_t k) {
    blk_q5_0 *y = (blk_q5_0 *)vy;
    for (int64_t b = 0; b < k / 32; b++, x += 32) {
        float amax = 0.f, mx = 0.f;
        for (int j = 0; j < 32; j++) {
            if (amax < fabsf(x[j])) { amax = fabsf(x[j]); mx = x[j]; }
        }
        const float d = mx / -16;
        const float id = d ? 1.0f / d : 0.0f;
        y[b].d = F2H(d);
        uint32_t qh = 0;
        for (int j = 0; j < 16; j++) {
            const float x0 = x[j] * id, x1 = x[16 + j] * id;
            const uint8_t xi0 = (uint8_t)imin_(31, (int8_t)(x0 + 16.5f));
            const uint8_t xi1 = (uint8_t)imin_(31, (int8_t)(x1 + 16.5f));
            y[b].qs[j] = (uint8_t)((xi0 & 0x0F) | ((xi1 & 0x0F) << 4));
            qh |= ((xi0 & 0x10u) >> 4) << (j + 0);
            qh |= ((xi1 & 0x10u) >> 4) << (j + 16);
        }
        memcpy(y[b].qh, &qh, 4);
    }
}

/* ggml-quants.c:373-440 with the arguments quantize_row_q6_K_ref passes (n=16, nmax=32, rmse_type=1,
 * no external weights: w_i = x_i^2). */
static float fit_scale_16(const float *x, int8_t *L) {
    const int n = 16, nmax = 32;
    float mx = 0, amax = 0;
    for (int i = 0; i < n; i++) {
        float a = fabsf(x[i]);
        if (a > amax) { amax = a; mx = x[i]; }
    }
    if (amax < 1e-15f) {
        for (int i = 0; i < n; i++) L[i] = 0;
        return 0.f;
    }
    float iscale = -nmax / mx;
    float sumlx = 0, suml2 = 0;
    for (int i = 0; i < n; i++) {
        int l = nearest_i(iscale * x[i]);
        l = imax_(-nmax, imin_(nmax - 1, l));
        L[i] = (int8_t)(l + nmax);
        float w = x[i] * x[i];
        sumlx += w * x[i] * l;
        suml2 += w * l * l;
    }
    float scale = suml2 ? sumlx / suml2 : 0.0f;
    float best = scale * sumlx;
    for (int is = -9; is <= 9; is++) {
        if (is == 0) continue;
        iscale = -(nmax + 0.1f * is) / mx;
        sumlx = suml2 = 0;
        for (int i = 0; i < n; i++) {
            int l = nearest_i(iscale * x[i]);
            l = imax_(-nmax, imin_(nmax - 1, l));
            float w = x[i] * x[i];
            sumlx += w * x[i] * l;
            suml2 += w * l * l;
        }
        if (suml2 > 0 && sumlx * sumlx > best * suml2) {
            for (int i = 0; i < n; i++) {
                int l = nearest_i(iscale * x[i]);
                L[i] = (int8_t)(nmax + imax_(-nmax, imin_(nmax - 1, l)));
            }
            scale = sumlx / suml2;
            best = scale * sumlx;
        }
    }
    return scale;
}

/* ggml-quants.c:1614-1682. */
void orc_quantize_row_q6_K_ref(const float *x, void *vy, int64_t k) {
    blk_q6_K *y = (blk_q6_K *)vy;
    int8_t L[256];
    float scales[16];
    for (int64_t b = 0; b < k / 256; b++, x += 256) {
        float max_scale = 0, max_abs = 0;
        for (int g = 0; g < 16; g++) {
            const float s = fit_scale_16(x + 16 * g, L + 16 * g);
            scales[g] = s;
            const float a = fabsf(s);
            if (a > max_abs) { max_abs = a; max_scale = s; }
        }
        if (max_abs < 1e-15f) { memset(&y[b], 0, sizeof(blk_q6_K)); continue; }
        const float iscale = -128.f / max_scale;
        y[b].d = F2H(1 / iscale);
        for (int g = 0; g < 16; g++) y[b].scales[g] = (int8_t)imin_(127, nearest_i(iscale * scales[g]));
        for (int g = 0; g < 16; g++) {
            const float d = H2F(y[b].d) * y[b].scales[g];
            if (!d) continue;
            for (int i = 0; i < 16; i++) {
                int l = nearest_i(x[16 * g + i] / d);
                L[16 * g + i] = (int8_t)(imax_(-32, imin_(31, l)) + 32);
            }
        }
        uint8_t *ql = y[b].ql, *qh = y[b].qh;
        for (int j = 0; j < 256; j += 128, ql += 64, qh += 32) {
            for (int l = 0; l < 32; l++) {
                const uint8_t a = (uint8_t)L[j + l], c = (uint8_t)L[j + l + 32];
                const uint8_t e = (uint8_t)L[j + l + 64], g = (uint8_t)L[j + l + 96];
                ql[l]      = (uint8_t)((a & 0xF) | ((e & 0xF) << 4));
                ql[l + 32] = (uint8_t)((c & 0xF) | ((g & 0xF) << 4));
                qh[l] = (uint8_t)((a >> 4) | ((c >> 4) << 2) | ((e >> 4) << 4) | ((g >> 4) << 6));
            }
        }
    }
}

size_t orc_quantize_rows(int type, const float *x, void *y, int64_t nrows, int64_t k) {
    const size_t rs = orc_row_size(type, k);
    for (int64_t r = 0; r < nrows; r++) {
        void *dst = (char *)y + r * rs;
        const float *src = x + r * k;
        switch (type) {
            case ORC_TYPE_Q4_0: orc_quantize_row_q4_0_ref(src, dst, k); break;
            case ORC_TYPE_Q8_0: orc_quantize_row_q8_0_ref(src, dst, k); break;
            case ORC_TYPE_Q4_K: orc_quantize_row_q4_K_ref(src, dst, k); break;
            case ORC_TYPE_Q6_K: orc_quantize_row_q6_K_ref(src, dst, k); break;
            case ORC_TYPE_Q5_K: orc_quantize_row_q5_K_ref(src, dst, k); break;
            case ORC_TYPE_Q5_0: orc_quantize_row_q5_0_ref(src, dst, k); break;
            case ORC_TYPE_Q4_1: orc_quantize_row_q4_1_ref(src, dst, k); break;
            case ORC_TYPE_Q5_1: orc_quantize_row_q5_1_ref(src, dst, k); break;
            case ORC_TYPE_F16: orc_fp32_to_fp16_row(src, dst, k); break;
            default: return 0;
        }
    }
    return rs * (size_t)nrows;
}

/* The sixteen 6-bit scales of a q3_K super-block, still biased by 32 (ggml-quants.c:1062-1071, the same unpacking in
 * ggml-cpu/ggml-cpu-quants.c:5815-5822): byte k of the four words is scale k. */
static void q3_K_scales(const uint8_t *s12, int8_t out[16]) {
    uint32_t aux[4];
    memcpy(aux, s12, 12);
    const uint32_t tmp = aux[2];
    aux[2] = ((aux[0] >> 4) & 0x0f0f0f0fu) | (((tmp >> 4) & 0x03030303u) << 4);
    aux[3] = ((aux[1] >> 4) & 0x0f0f0f0fu) | (((tmp >> 6) & 0x03030303u) << 4);
    aux[0] = (aux[0] & 0x0f0f0f0fu) | (((tmp >> 0) & 0x03030303u) << 4);
    aux[1] = (aux[1] & 0x0f0f0f0fu) | (((tmp >> 2) & 0x03030303u) << 4);
    memcpy(out, aux, 16);
}

/* ---------------------------------------------------------------- dequantizers (closed forms)
 * q4_0 ggml-quants.c:249-267 ; q8_0 :343-357 ; q4_K :1274-1296 ; q6_K :1684-1713 ; q8_K :2512-2521 */
void orc_dequantize_row(int type, const void *vx, float *y, int64_t k) {
    if (type == ORC_TYPE_Q4_0) {
        const blk_q4_0 *x = (const blk_q4_0 *)vx;
        for (int64_t b = 0; b < k / 32; b++, y += 32) {
            const float d = H2F(x[b].d);
            for (int j = 0; j < 16; j++) {
                y[j]      = ((x[b].qs[j] & 0xF) - 8) * d;
                y[j + 16] = ((x[b].qs[j] >> 4) - 8) * d;
            }
        }
    } else if (type == ORC_TYPE_Q8_0) {
        const blk_q8_0 *x = (const blk_q8_0 *)vx;
        for (int64_t b = 0; b < k / 32; b++, y += 32) {
            const float d = H2F(x[b].d);
            for (int j = 0; j < 32; j++) y[j] = x[b].qs[j] * d;
        }
    } else if (type == ORC_TYPE_Q4_K) {
        const blk_q4_K *x = (const blk_q4_K *)vx;
        for (int64_t b = 0; b < k / 256; b++) {
            const float d = H2F(x[b].d), mn = H2F(x[b].dmin);
            const uint8_t *q = x[b].qs;
            for (int j = 0; j < 4; j++, q += 32) {
                uint8_t sc, m;
                unpack_sc_m(2 * j, x[b].scales, &sc, &m);
                const float d1 = d * sc, m1 = mn * m;
                unpack_sc_m(2 * j + 1, x[b].scales, &sc, &m);
                const float d2 = d * sc, m2 = mn * m;
                for (int l = 0; l < 32; l++) *y++ = d1 * (q[l] & 0xF) - m1;
                for (int l = 0; l < 32; l++) *y++ = d2 * (q[l] >> 4) - m2;
            }
        }
    } else if (type == ORC_TYPE_Q6_K) {
        const blk_q6_K *x = (const blk_q6_K *)vx;
        for (int64_t b = 0; b < k / 256; b++) {
            const float d = H2F(x[b].d);
            const uint8_t *ql = x[b].ql, *qh = x[b].qh;
            const int8_t *sc = x[b].scales;
            for (int h = 0; h < 2; h++, y += 128, ql += 64, qh += 32, sc += 8) {
                for (int l = 0; l < 32; l++) {
                    const int is = l / 16;
                    const int8_t q1 = (int8_t)((ql[l]      & 0xF) | (((qh[l] >> 0) & 3) << 4)) - 32;
                    const int8_t q2 = (int8_t)((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32;
                    const int8_t q3 = (int8_t)((ql[l]      >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32;
                    const int8_t q4 = (int8_t)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32;
                    y[l]      = d * sc[is + 0] * q1;
                    y[l + 32] = d * sc[is + 2] * q2;
                    y[l + 64] = d * sc[is + 4] * q3;
                    y[l + 96] = d * sc[is + 6] * q4;
                }
            }
        }
    } else if (type == ORC_TYPE_Q2_K) {                 /* ggml-quants.c:706-737 */
        const blk_q2_K *x = (const blk_q2_K *)vx;
        for (int64_t b = 0; b < k / 256; b++) {
            const float d = H2F(x[b].d), mn = H2F(x[b].dmin);
            const uint8_t *q = x[b].qs;
            int is = 0;
            for (int h = 0; h < 2; h++, q += 32) {
                for (int j = 0; j < 4; j++) {
                    for (int half = 0; half < 2; half++) {
                        const uint8_t sc = x[b].scales[is++];
                        const float dl = d * (sc & 0xF), ml = mn * (sc >> 4);
                        for (int l = 0; l < 16; l++) *y++ = dl * ((int8_t)((q[l + 16 * half] >> (2 * j)) & 3)) - ml;
                    }
                }
            }
        }
    } else if (type == ORC_TYPE_Q3_K) {                 /* ggml-quants.c:1050-1098 */
        const blk_q3_K *x = (const blk_q3_K *)vx;
        for (int64_t b = 0; b < k / 256; b++) {
            const float d_all = H2F(x[b].d);
            int8_t scales[16];
            q3_K_scales(x[b].scales, scales);
            const uint8_t *q = x[b].qs, *hm = x[b].hmask;
            uint8_t m = 1;
            int is = 0;
            for (int h = 0; h < 2; h++, q += 32) {
                for (int j = 0; j < 4; j++, m <<= 1) {
                    for (int half = 0; half < 2; half++) {
                        const float dl = d_all * (scales[is++] - 32);
                        for (int l = 16 * half; l < 16 * half + 16; l++)
                            *y++ = dl * ((int8_t)((q[l] >> (2 * j)) & 3) - ((hm[l] & m) ? 0 : 4));
                    }
                }
            }
        }
    } else if (type == ORC_TYPE_IQ4_XS) {               /* ggml-quants.c dequantize_row_iq4_xs */
        const blk_iq4_xs *x = (const blk_iq4_xs *)vx;
        for (int64_t b = 0; b < k / 256; b++) {
            const float d = H2F(x[b].d);
            const uint8_t *qs = x[b].qs;
            for (int ib = 0; ib < 8; ib++, y += 32, qs += 16) {
                const int ls = ((x[b].scales_l[ib / 2] >> 4 * (ib % 2)) & 0xf) | (((x[b].scales_h >> 2 * ib) & 3) << 4);
                const float dl = d * (ls - 32);
                for (int j = 0; j < 16; j++) {
                    y[j]      = dl * iq4nl_values[qs[j] & 0xf];
                    y[j + 16] = dl * iq4nl_values[qs[j] >> 4];
                }
            }
        }
    } else if (type == ORC_TYPE_Q8_K) {
        const blk_q8_K *x = (const blk_q8_K *)vx;
        for (int64_t b = 0; b < k / 256; b++)
            for (int j = 0; j < 256; j++) *y++ = x[b].d * x[b].qs[j];
    } else if (type == ORC_TYPE_Q5_0) {                 /* ggml-quants.c:290-313 */
        const blk_q5_0 *x = (const blk_q5_0 *)vx;
        for (int64_t b = 0; b < k / 32; b++, y += 32) {
            const float d = H2F(x[b].d);
            uint32_t qh;
            memcpy(&qh, x[b].qh, 4);
            for (int j = 0; j < 16; j++) {
                const uint8_t xh0 = (uint8_t)(((qh >> (j + 0)) << 4) & 0x10);
                const uint8_t xh1 = (uint8_t)((qh >> (j + 12)) & 0x10);
                y[j]      = (float)(((x[b].qs[j] & 0x0F) | xh0) - 16) * d;
                y[j + 16] = (float)(((x[b].qs[j] >> 4) | xh1) - 16) * d;
            }
        }
    } else if (type == ORC_TYPE_Q5_K) {                 /* ggml-quants.c:1476-1501 */
        const blk_q5_K *x = (const blk_q5_K *)vx;
        for (int64_t b = 0; b < k / 256; b++) {
            const float d = H2F(x[b].d), mn = H2F(x[b].dmin);
            const uint8_t *ql = x[b].qs, *qh = x[b].qh;
            uint8_t u1 = 1, u2 = 2;
            for (int j = 0; j < 4; j++, ql += 32) {
                uint8_t sc, m;
                unpack_sc_m(2 * j, x[b].scales, &sc, &m);
                const float d1 = d * sc, m1 = mn * m;
                unpack_sc_m(2 * j + 1, x[b].scales, &sc, &m);
                const float d2 = d * sc, m2 = mn * m;
                for (int l = 0; l < 32; l++) *y++ = d1 * ((ql[l] & 0xF) + ((qh[l] & u1) ? 16 : 0)) - m1;
                for (int l = 0; l < 32; l++) *y++ = d2 * ((ql[l] >> 4) + ((qh[l] & u2) ? 16 : 0)) - m2;
                u1 = (uint8_t)(u1 << 2); u2 = (uint8_t)(u2 << 2);
            }
        }
    } else if (type == ORC_TYPE_F16) {
        const uint16_t *x = (const uint16_t *)vx;
        for (int64_t i = 0; i < k; i++) y[i] = H2F(x[i]);
    } else if (type == ORC_TYPE_Q4_1) {                 /* ggml-quants.c:269-288 */
        const blk_q4_1 *x = (const blk_q4_1 *)vx;
        for (int64_t b = 0; b < k / 32; b++, y += 32) {
            const float d = H2F(x[b].d), m = H2F(x[b].m);
            for (int j = 0; j < 16; j++) {
                y[j]      = (x[b].qs[j] & 0x0F) * d + m;
                y[j + 16] = (x[b].qs[j] >> 4) * d + m;
            }
        }
    } else if (type == ORC_TYPE_Q5_1) {                 /* ggml-quants.c:315-341 */
        const blk_q5_1 *x = (const blk_q5_1 *)vx;
        for (int64_t b = 0; b < k / 32; b++, y += 32) {
            const float d = H2F(x[b].d), m = H2F(x[b].m);
            uint32_t qh;
            memcpy(&qh, x[b].qh, 4);
            for (int j = 0; j < 16; j++) {
                const uint8_t xh0 = (uint8_t)(((qh >> (j + 0)) << 4) & 0x10);
                const uint8_t xh1 = (uint8_t)((qh >> (j + 12)) & 0x10);
                y[j]      = (float)((x[b].qs[j] & 0x0F) | xh0) * d + m;
                y[j + 16] = (float)((x[b].qs[j] >> 4) | xh1) * d + m;
            }
        }
    } else if (type == ORC_TYPE_Q8_1) {
        const blk_q8_1 *x = (const blk_q8_1 *)vx;
        for (int64_t b = 0; b < k / 32; b++, y += 32) {
            const float d = H2F(x[b].d);
            for (int j = 0; j < 32; j++) y[j] = x[b].qs[j] * d;
        }
    } else if (type == ORC_TYPE_IQ4_NL) {               /* ggml-quants.c:2430-2446 */
        const blk_iq4_nl *x = (const blk_iq4_nl *)vx;
        for (int64_t b = 0; b < k / 32; b++, y += 32) {
            const float d = H2F(x[b].d);
            for (int j = 0; j < 16; j++) {
                y[j]      = d * iq4nl_values[x[b].qs[j] & 0xf];
                y[j + 16] = d * iq4nl_values[x[b].qs[j] >> 4];
            }
        }
    }
}

/* The 32 signed weights of one block of the 32-element types in element order (what the SIMD paths put into
 * one 256-bit register before multiplying with the Q8_0 quants). */
static void block32_ints(int type, const void *vx, int64_t b, int8_t w[32], uint16_t *dh) {
    if (type == ORC_TYPE_Q5_0) {                        /* ggml-cpu/ggml-cpu-quants.c:70-80 + q5_0 AVX2 branch */
        const blk_q5_0 *x = (const blk_q5_0 *)vx + b;
        uint32_t qh;
        memcpy(&qh, x->qh, 4);
        for (int j = 0; j < 16; j++) {
            w[j]      = (int8_t)(((x->qs[j] & 0xF) | (((qh >> j) & 1) << 4)) - 16);
            w[j + 16] = (int8_t)(((x->qs[j] >> 4) | (((qh >> (j + 16)) & 1) << 4)) - 16);
        }
        *dh = x->d;
    } else {                                            /* ORC_TYPE_IQ4_NL */
        const blk_iq4_nl *x = (const blk_iq4_nl *)vx + b;
        for (int j = 0; j < 16; j++) {
            w[j]      = iq4nl_values[x->qs[j] & 0xf];
            w[j + 16] = iq4nl_values[x->qs[j] >> 4];
        }
        *dh = x->d;
    }
}

/* ---------------------------------------------------------------- dot products (AVX2 lane structure) */

/* ggml-cpu/ggml-cpu-quants.c:43-49: horizontal sum of 8 lanes, in the order the shuffles impose. */
static inline float hsum8(const float a[8]) {
    const float r0 = a[4] + a[0], r1 = a[5] + a[1], r2 = a[6] + a[2], r3 = a[7] + a[3];
    const float s0 = r0 + r2, s1 = r1 + r3;
    return s0 + s1;
}

/* ggml-cpu/ggml-cpu-quants.c:2267-2290.  Lane j of the 8-wide accumulator takes the four products of bytes
 * 4j..4j+3 of the 32-byte vectors (low nibbles are bytes 0..15, high nibbles 16..31; :79-85,116-128). */
float orc_vec_dot_q4_0_q8_0(int64_t k, const void *vx, const void *vy, int32_t *isum) {
    const blk_q4_0 *x = (const blk_q4_0 *)vx;
    const blk_q8_0 *y = (const blk_q8_0 *)vy;
    float acc[8] = {0};
    for (int64_t b = 0; b < k / 32; b++) {
        const float d = H2F(x[b].d) * H2F(y[b].d);
        int8_t w[32];
        for (int j = 0; j < 16; j++) {
            w[j]      = (int8_t)((x[b].qs[j] & 0xF) - 8);
            w[j + 16] = (int8_t)((x[b].qs[j] >> 4) - 8);
        }
        int32_t tot = 0;
        for (int j = 0; j < 8; j++) {
            int32_t p = 0;
            for (int t = 0; t < 4; t++) p += (int32_t)w[4 * j + t] * y[b].qs[4 * j + t];
            tot += p;
            acc[j] = fmaf(d, (float)p, acc[j]);
        }
        if (isum) isum[b] = tot;
    }
    return hsum8(acc);
}

/* ggml-cpu/ggml-cpu-quants.c:3863-3880. */
float orc_vec_dot_q8_0_q8_0(int64_t k, const void *vx, const void *vy, int32_t *isum) {
    const blk_q8_0 *x = (const blk_q8_0 *)vx;
    const blk_q8_0 *y = (const blk_q8_0 *)vy;
    float acc[8] = {0};
    for (int64_t b = 0; b < k / 32; b++) {
        const float d = H2F(x[b].d) * H2F(y[b].d);
        int32_t tot = 0;
        for (int j = 0; j < 8; j++) {
            int32_t p = 0;
            for (int t = 0; t < 4; t++) p += (int32_t)x[b].qs[4 * j + t] * y[b].qs[4 * j + t];
            tot += p;
            acc[j] = fmaf(d, (float)p, acc[j]);
        }
        if (isum) isum[b] = tot;
    }
    return hsum8(acc);
}

/* The shuffle the SIMD paths use to unpack the 12 scale bytes (ggml-cpu/ggml-cpu-quants.c:7048-7053):
 * out[0..7] = 6-bit scales, out[8..15] = 6-bit mins.  Equivalent to unpack_sc_m for j = 0..7. */
static void unpack_scales_kmask(const uint8_t *s12, uint8_t out[16]) {
    uint32_t u[4];
    memcpy(u, s12, 12);
    u[3] = ((u[2] >> 4) & 0x0f0f0f0fu) | (((u[1] >> 6) & 0x03030303u) << 4);
    const uint32_t t = u[1] & 0x3f3f3f3fu;
    u[1] = (u[2] & 0x0f0f0f0fu) | (((u[0] >> 6) & 0x03030303u) << 4);
    u[2] = t;
    u[0] &= 0x3f3f3f3fu;
    memcpy(out, u, 16);
}

/* ggml-cpu/ggml-cpu-quants.c:7036-7099. */
float orc_vec_dot_q4_K_q8_K(int64_t k, const void *vx, const void *vy, int32_t *isum, int32_t *imin) {
    const blk_q4_K *x = (const blk_q4_K *)vx;
    const blk_q8_K *y = (const blk_q8_K *)vy;
    float acc[8] = {0};
    float accm[4] = {0};
    for (int64_t b = 0; b < k / 256; b++) {
        const float d = y[b].d * H2F(x[b].d);
        const float dmin = -y[b].d * H2F(x[b].dmin);
        uint8_t sm[16];
        unpack_scales_kmask(x[b].scales, sm);
        const uint8_t *sc = sm, *mn = sm + 8;

        /* mins: pairwise bsums as int16 (hadd), then madd by pairs of mins -> 4 int32 lanes */
        int32_t mtot = 0;
        for (int i = 0; i < 4; i++) {
            const int16_t s0 = (int16_t)(y[b].bsums[4 * i + 0] + y[b].bsums[4 * i + 1]);
            const int16_t s1 = (int16_t)(y[b].bsums[4 * i + 2] + y[b].bsums[4 * i + 3]);
            const int32_t p = (int32_t)mn[2 * i] * s0 + (int32_t)mn[2 * i + 1] * s1;
            mtot += p;
            accm[i] = fmaf(dmin, (float)p, accm[i]);
        }

        int32_t lane[8] = {0};
        const uint8_t *q4 = x[b].qs;
        const int8_t *q8 = y[b].qs;
        for (int j = 0; j < 4; j++, q4 += 32, q8 += 64) {
            for (int m = 0; m < 8; m++) {
                int32_t pl = 0, ph = 0;
                for (int t = 0; t < 4; t++) {
                    pl += (int32_t)(q4[4 * m + t] & 0xF) * q8[4 * m + t];
                    ph += (int32_t)(q4[4 * m + t] >> 4) * q8[32 + 4 * m + t];
                }
                lane[m] += (int32_t)sc[2 * j] * pl + (int32_t)sc[2 * j + 1] * ph;
            }
        }
        int32_t tot = 0;
        for (int m = 0; m < 8; m++) { tot += lane[m]; acc[m] = fmaf(d, (float)lane[m], acc[m]); }
        if (isum) isum[b] = tot;
        if (imin) imin[b] = mtot;
    }
    const float m0 = accm[0] + accm[2], m1 = accm[1] + accm[3];
    return hsum8(acc) + (m0 + m1);
}

/* ggml-cpu/ggml-cpu-quants.c:8972-9049. */
float orc_vec_dot_q6_K_q8_K(int64_t k, const void *vx, const void *vy, int32_t *isum) {
    const blk_q6_K *x = (const blk_q6_K *)vx;
    const blk_q8_K *y = (const blk_q8_K *)vy;
    float acc[8] = {0};
    for (int64_t b = 0; b < k / 256; b++) {
        const float d = y[b].d * H2F(x[b].d);
        int32_t lane[8] = {0};
        const uint8_t *ql = x[b].ql, *qh = x[b].qh;
        const int8_t *q8 = y[b].qs, *sc = x[b].scales;
        for (int h = 0; h < 2; h++, ql += 64, qh += 32, q8 += 128, sc += 8) {
            for (int v = 0; v < 4; v++) {                 /* the four 32-value vectors of this half */
                for (int m = 0; m < 8; m++) {
                    int32_t p = 0;
                    for (int t = 0; t < 4; t++) {
                        const int i = 4 * m + t;
                        int q;
                        switch (v) {
                            case 0:  q = (ql[i]      & 0xF) | (((qh[i] >> 0) & 3) << 4); break;
                            case 1:  q = (ql[i + 32] & 0xF) | (((qh[i] >> 2) & 3) << 4); break;
                            case 2:  q = (ql[i]      >> 4) | (((qh[i] >> 4) & 3) << 4); break;
                            default: q = (ql[i + 32] >> 4) | (((qh[i] >> 6) & 3) << 4); break;
                        }
                        p += (q - 32) * (int32_t)q8[32 * v + i];
                    }
                    lane[m] += (int32_t)sc[2 * v + (m >= 4)] * p;
                }
            }
        }
        int32_t tot = 0;
        for (int m = 0; m < 8; m++) { tot += lane[m]; acc[m] = fmaf(d, (float)lane[m], acc[m]); }
        if (isum) isum[b] = tot;
    }
    return hsum8(acc);
}

/* q5_0: ggml-cpu/ggml-cpu-quants.c AVX2 branch of lm_ggml_vec_dot_q5_0_q8_0 (:2924...): one 8-lane accumulator,
 * lane j takes the four products of elements 4j..4j+3, fmadd with d = dx * dy. */
float orc_vec_dot_q5_0_q8_0(int64_t k, const void *vx, const void *vy, int32_t *isum) {
    const blk_q8_0 *y = (const blk_q8_0 *)vy;
    float acc[8] = {0};
    for (int64_t b = 0; b < k / 32; b++) {
        int8_t w[32];
        uint16_t dh;
        block32_ints(ORC_TYPE_Q5_0, vx, b, w, &dh);
        const float d = H2F(dh) * H2F(y[b].d);
        int32_t tot = 0;
        for (int j = 0; j < 8; j++) {
            int32_t p = 0;
            for (int t = 0; t < 4; t++) p += (int32_t)w[4 * j + t] * y[b].qs[4 * j + t];
            tot += p;
            acc[j] = fmaf(d, (float)p, acc[j]);
        }
        if (isum) isum[b] = tot;
    }
    return hsum8(acc);
}

/* iq4_nl: AVX2 branch of lm_ggml_vec_dot_iq4_nl_q8_0 (ggml-cpu/ggml-cpu-quants.c:12798-12826): blocks are taken
 * two at a time into two 8-lane accumulators (d = dy * dx), added lane-wise at the end; an odd last block
 * goes through the scalar tail (:12869-12878: sumf += d * (sumi1 + sumi2)). */
float orc_vec_dot_iq4_nl_q8_0(int64_t k, const void *vx, const void *vy, int32_t *isum) {
    const blk_q8_0 *y = (const blk_q8_0 *)vy;
    const int64_t nb = k / 32;
    float acc1[8] = {0}, acc2[8] = {0};
    int64_t b = 0;
    for (; b + 1 < nb; b += 2) {
        for (int h = 0; h < 2; h++) {
            int8_t w[32];
            uint16_t dh;
            block32_ints(ORC_TYPE_IQ4_NL, vx, b + h, w, &dh);
            const float d = H2F(y[b + h].d) * H2F(dh);
            float *acc = h ? acc2 : acc1;
            int32_t tot = 0;
            for (int j = 0; j < 8; j++) {
                int32_t p = 0;
                for (int t = 0; t < 4; t++) p += (int32_t)w[4 * j + t] * y[b + h].qs[4 * j + t];
                tot += p;
                acc[j] = fmaf(d, (float)p, acc[j]);
            }
            if (isum) isum[b + h] = tot;
        }
    }
    float s8[8];
    for (int j = 0; j < 8; j++) s8[j] = acc1[j] + acc2[j];
    float sumf = hsum8(s8);
    for (; b < nb; b++) {
        int8_t w[32];
        uint16_t dh;
        block32_ints(ORC_TYPE_IQ4_NL, vx, b, w, &dh);
        const float d = H2F(y[b].d) * H2F(dh);
        int32_t s1 = 0, s2 = 0;
        for (int j = 0; j < 16; j++) { s1 += y[b].qs[j] * w[j]; s2 += y[b].qs[j + 16] * w[j + 16]; }
        if (isum) isum[b] = s1 + s2;
        sumf += d * (float)(s1 + s2);
    }
    return sumf;
}

/* F16 x F16: lm_ggml_vec_dot_f16 (ggml-cpu/vec.cpp:122-162) with the AVX2 mapping of ggml-cpu/simd-mappings.h
 * (LM_GGML_F16_STEP 32, four 8-lane fp32 accumulators, fmadd of the widened halves; reduction :251-269:
 * acc0 += acc2, acc1 += acc3, acc0 += acc1, low half + high half, two horizontal adds).  Elements past the last
 * multiple of 32 are added in double precision (:152-154). */
float orc_vec_dot_f16(int64_t k, const void *vx, const void *vy) {
    const uint16_t *x = (const uint16_t *)vx, *y = (const uint16_t *)vy;
    float acc[4][8] = {{0}};
    const int64_t np = k & ~(int64_t)31;
    for (int64_t i = 0; i < np; i += 32)
        for (int j = 0; j < 4; j++)
            for (int l = 0; l < 8; l++) acc[j][l] = fmaf(H2F(x[i + 8 * j + l]), H2F(y[i + 8 * j + l]), acc[j][l]);
    float t[4];
    for (int l = 0; l < 8; l++) { acc[0][l] = acc[0][l] + acc[2][l]; acc[1][l] = acc[1][l] + acc[3][l]; }
    for (int l = 0; l < 8; l++) acc[0][l] = acc[0][l] + acc[1][l];
    for (int l = 0; l < 4; l++) t[l] = acc[0][l] + acc[0][l + 4];
    const float h0 = t[0] + t[1], h1 = t[2] + t[3];
    double sumf = (double)(h0 + h1);
    for (int64_t i = np; i < k; i++) sumf += (double)(H2F(x[i]) * H2F(y[i]));
    return (float)sumf;
}

/* q4_1 / q5_1 x q8_1: AVX2 branches of lm_ggml_vec_dot_q4_1_q8_1 and lm_ggml_vec_dot_q5_1_q8_1
 * (ggml-cpu/ggml-cpu-quants.c): unsigned weights u (nibble, or nibble | bit << 4), lane j takes the four
 * products of elements 4j..4j+3, acc = fmadd(dx*dy, float(p), acc); the min term is the scalar
 * summs += m * s (separate multiply and add), added after the horizontal sum. */
static float dot_min32(int type, int64_t k, const void *vx, const void *vy, int32_t *isum) {
    const blk_q8_1 *y = (const blk_q8_1 *)vy;
    float acc[8] = {0};
    float summs = 0.f;
    for (int64_t b = 0; b < k / 32; b++) {
        uint8_t w[32];
        uint16_t dh, mh;
        if (type == ORC_TYPE_Q4_1) {
            const blk_q4_1 *x = (const blk_q4_1 *)vx + b;
            for (int j = 0; j < 16; j++) { w[j] = x->qs[j] & 0xF; w[j + 16] = x->qs[j] >> 4; }
            dh = x->d; mh = x->m;
        } else {
            const blk_q5_1 *x = (const blk_q5_1 *)vx + b;
            uint32_t qh;
            memcpy(&qh, x->qh, 4);
            for (int j = 0; j < 16; j++) {
                w[j]      = (uint8_t)((x->qs[j] & 0xF) | (((qh >> j) & 1) << 4));
                w[j + 16] = (uint8_t)((x->qs[j] >> 4) | (((qh >> (j + 16)) & 1) << 4));
            }
            dh = x->d; mh = x->m;
        }
        const float prod = H2F(mh) * H2F(y[b].s);
        summs = summs + prod;
        const float d = H2F(dh) * H2F(y[b].d);
        int32_t tot = 0;
        for (int j = 0; j < 8; j++) {
            int32_t p = 0;
            for (int t = 0; t < 4; t++) p += (int32_t)w[4 * j + t] * y[b].qs[4 * j + t];
            tot += p;
            acc[j] = fmaf(d, (float)p, acc[j]);
        }
        if (isum) isum[b] = tot;
    }
    return hsum8(acc) + summs;
}
float orc_vec_dot_q4_1_q8_1(int64_t k, const void *vx, const void *vy, int32_t *isum) { return dot_min32(ORC_TYPE_Q4_1, k, vx, vy, isum); }
float orc_vec_dot_q5_1_q8_1(int64_t k, const void *vx, const void *vy, int32_t *isum) { return dot_min32(ORC_TYPE_Q5_1, k, vx, vy, isum); }

/* q5_K: AVX2 branch of lm_ggml_vec_dot_q5_K_q8_K (ggml-cpu/ggml-cpu-quants.c:7786-7860): as q4_K for the d term
 * (one integer 8-lane sum per super-block, one fmadd), but the min term is a scalar
 * `summs += dmin * hsum` (separate multiply and add) added after the horizontal sum. */
float orc_vec_dot_q5_K_q8_K(int64_t k, const void *vx, const void *vy, int32_t *isum, int32_t *imin) {
    const blk_q5_K *x = (const blk_q5_K *)vx;
    const blk_q8_K *y = (const blk_q8_K *)vy;
    float acc[8] = {0};
    float summs = 0.f;
    for (int64_t b = 0; b < k / 256; b++) {
        const float d = y[b].d * H2F(x[b].d);
        const float dmin = -y[b].d * H2F(x[b].dmin);
        uint8_t sm[16];
        unpack_scales_kmask(x[b].scales, sm);
        const uint8_t *sc = sm, *mn = sm + 8;
        int32_t mtot = 0;
        for (int j = 0; j < 8; j++)
            mtot += (int32_t)mn[j] * (int16_t)(y[b].bsums[2 * j] + y[b].bsums[2 * j + 1]);
        const float prod = dmin * (float)mtot;
        summs = summs + prod;

        int32_t lane[8] = {0};
        const uint8_t *q5 = x[b].qs, *qh = x[b].qh;
        const int8_t *q8 = y[b].qs;
        for (int j = 0; j < 4; j++, q5 += 32, q8 += 64) {
            for (int m = 0; m < 8; m++) {
                int32_t pl = 0, ph = 0;
                for (int t = 0; t < 4; t++) {
                    const int e = 4 * m + t;
                    const int lo = (q5[e] & 0xF) + (((qh[e] >> (2 * j)) & 1) << 4);
                    const int hi = (q5[e] >> 4) + (((qh[e] >> (2 * j + 1)) & 1) << 4);
                    pl += lo * q8[e];
                    ph += hi * q8[32 + e];
                }
                lane[m] += (int32_t)sc[2 * j] * pl + (int32_t)sc[2 * j + 1] * ph;
            }
        }
        int32_t tot = 0;
        for (int m = 0; m < 8; m++) { tot += lane[m]; acc[m] = fmaf(d, (float)lane[m], acc[m]); }
        if (isum) isum[b] = tot;
        if (imin) imin[b] = mtot;
    }
    return hsum8(acc) + summs;
}

/* ggml-cpu/ggml-cpu-quants.c:4831-4894 (AVX2).  Eight int32 lanes: lane m of a 32-value vector v of half h holds
 * scale[8h + 2v + (m >= 4)] * sum_{t<4} q2 * q8 over bytes 4m .. 4m+3; the mins go first, into the same eight float
 * lanes, as mins[2m] * bsums[2m] + mins[2m+1] * bsums[2m+1]. */
float orc_vec_dot_q2_K_q8_K(int64_t k, const void *vx, const void *vy, int32_t *isum, int32_t *imin) {
    const blk_q2_K *x = (const blk_q2_K *)vx;
    const blk_q8_K *y = (const blk_q8_K *)vy;
    float acc[8] = {0};
    for (int64_t b = 0; b < k / 256; b++) {
        const float d = y[b].d * H2F(x[b].d);
        const float dmin = -y[b].d * H2F(x[b].dmin);
        int32_t mtot = 0;
        for (int m = 0; m < 8; m++) {
            const int32_t p = (int32_t)(x[b].scales[2 * m] >> 4) * y[b].bsums[2 * m] + (int32_t)(x[b].scales[2 * m + 1] >> 4) * y[b].bsums[2 * m + 1];
            mtot += p;
            acc[m] = fmaf(dmin, (float)p, acc[m]);
        }
        int32_t lane[8] = {0};
        const uint8_t *q2 = x[b].qs;
        const int8_t *q8 = y[b].qs;
        for (int h = 0; h < 2; h++, q2 += 32, q8 += 128) {
            for (int v = 0; v < 4; v++) {
                for (int m = 0; m < 8; m++) {
                    int32_t p = 0;
                    for (int t = 0; t < 4; t++) p += (int32_t)((q2[4 * m + t] >> (2 * v)) & 3) * q8[32 * v + 4 * m + t];
                    lane[m] += (int32_t)(x[b].scales[8 * h + 2 * v + (m >= 4)] & 0xF) * p;
                }
            }
        }
        int32_t tot = 0;
        for (int m = 0; m < 8; m++) { tot += lane[m]; acc[m] = fmaf(d, (float)lane[m], acc[m]); }
        if (isum) isum[b] = tot;
        if (imin) imin[b] = mtot;
    }
    return hsum8(acc);
}

/* ggml-cpu/ggml-cpu-quants.c:5806-5911 (AVX2): as q2_K without mins; the quant is the two low bits minus 4 where the
 * high bit is clear, the scales are biased by 32. */
float orc_vec_dot_q3_K_q8_K(int64_t k, const void *vx, const void *vy, int32_t *isum) {
    const blk_q3_K *x = (const blk_q3_K *)vx;
    const blk_q8_K *y = (const blk_q8_K *)vy;
    float acc[8] = {0};
    for (int64_t b = 0; b < k / 256; b++) {
        const float d = y[b].d * H2F(x[b].d);
        int8_t sc[16];
        q3_K_scales(x[b].scales, sc);
        int32_t lane[8] = {0};
        const uint8_t *q3 = x[b].qs, *hm = x[b].hmask;
        const int8_t *q8 = y[b].qs;
        for (int h = 0; h < 2; h++, q3 += 32, q8 += 128) {
            for (int v = 0; v < 4; v++) {
                const uint8_t bit = (uint8_t)(1u << (4 * h + v));
                for (int m = 0; m < 8; m++) {
                    int32_t p = 0;
                    for (int t = 0; t < 4; t++) {
                        const int i = 4 * m + t;
                        const int q = (int)((q3[i] >> (2 * v)) & 3) - ((hm[i] & bit) ? 0 : 4);
                        p += q * (int32_t)q8[32 * v + i];
                    }
                    lane[m] += (int32_t)(sc[8 * h + 2 * v + (m >= 4)] - 32) * p;
                }
            }
        }
        int32_t tot = 0;
        for (int m = 0; m < 8; m++) { tot += lane[m]; acc[m] = fmaf(d, (float)lane[m], acc[m]); }
        if (isum) isum[b] = tot;
    }
    return hsum8(acc);
}

/* ggml-cpu/ggml-cpu-quants.c lm_ggml_vec_dot_iq4_xs_q8_K, AVX2 branch: a 32-value sub-block is 16 qs bytes, the code points of
 * the low nibbles (elements 0..15) then those of the high nibbles (16..31) against 32 consecutive q8; lane m of eight holds
 * (ls - 32) * sum over bytes 4m .. 4m+3 of that vector; the super-block's scale is h2f(d) * y.d. */
float orc_vec_dot_iq4_xs_q8_K(int64_t k, const void *vx, const void *vy, int32_t *isum) {
    const blk_iq4_xs *x = (const blk_iq4_xs *)vx;
    const blk_q8_K *y = (const blk_q8_K *)vy;
    float acc[8] = {0};
    for (int64_t b = 0; b < k / 256; b++) {
        const float d = H2F(x[b].d) * y[b].d;
        int32_t lane[8] = {0};
        const uint8_t *qs = x[b].qs;
        const int8_t *q8 = y[b].qs;
        for (int ib = 0; ib < 8; ib++, qs += 16, q8 += 32) {
            const int ls = (((x[b].scales_l[ib / 2] >> 4 * (ib % 2)) & 0xf) | (((x[b].scales_h >> 2 * ib) & 3) << 4)) - 32;
            for (int m = 0; m < 8; m++) {
                int32_t p = 0;
                for (int t = 0; t < 4; t++) {
                    const int e = 4 * m + t;                          /* element of the sub-block */
                    const int nib = e < 16 ? (qs[e] & 0xf) : (qs[e - 16] >> 4);
                    p += (int32_t)iq4nl_values[nib] * q8[e];
                }
                lane[m] += ls * p;
            }
        }
        int32_t tot = 0;
        for (int m = 0; m < 8; m++) { tot += lane[m]; acc[m] = fmaf(d, (float)lane[m], acc[m]); }
        if (isum) isum[b] = tot;
    }
    return hsum8(acc);
}

float orc_vec_dot(int type, int64_t k, const void *vx, const void *vy) {
    switch (type) {
        case ORC_TYPE_Q4_0: return orc_vec_dot_q4_0_q8_0(k, vx, vy, NULL);
        case ORC_TYPE_Q8_0: return orc_vec_dot_q8_0_q8_0(k, vx, vy, NULL);
        case ORC_TYPE_Q4_K: return orc_vec_dot_q4_K_q8_K(k, vx, vy, NULL, NULL);
        case ORC_TYPE_Q6_K: return orc_vec_dot_q6_K_q8_K(k, vx, vy, NULL);
        case ORC_TYPE_Q5_0: return orc_vec_dot_q5_0_q8_0(k, vx, vy, NULL);
        case ORC_TYPE_IQ4_NL: return orc_vec_dot_iq4_nl_q8_0(k, vx, vy, NULL);
        case ORC_TYPE_Q5_K: return orc_vec_dot_q5_K_q8_K(k, vx, vy, NULL, NULL);
        case ORC_TYPE_Q4_1: return orc_vec_dot_q4_1_q8_1(k, vx, vy, NULL);
        case ORC_TYPE_Q5_1: return orc_vec_dot_q5_1_q8_1(k, vx, vy, NULL);
        case ORC_TYPE_F16: return orc_vec_dot_f16(k, vx, vy);
        case ORC_TYPE_Q2_K: return orc_vec_dot_q2_K_q8_K(k, vx, vy, NULL, NULL);
        case ORC_TYPE_Q3_K: return orc_vec_dot_q3_K_q8_K(k, vx, vy, NULL);
        case ORC_TYPE_IQ4_XS: return orc_vec_dot_iq4_xs_q8_K(k, vx, vy, NULL);
        default: return NAN;
    }
}

double orc_vec_dot_exact(int type, int64_t k, const void *vx, const void *vy, double *sum_abs) {
    double s = 0, sa = 0;
    const int be = orc_block_elems(type);
    if (!be) return NAN;
    const int64_t nb = k / be;
    int32_t *is = (int32_t *)malloc(sizeof(int32_t) * (size_t)(nb > 0 ? nb : 1) * 2);
    if (type == ORC_TYPE_Q4_0 || type == ORC_TYPE_Q8_0) {
        if (type == ORC_TYPE_Q4_0) orc_vec_dot_q4_0_q8_0(k, vx, vy, is);
        else                       orc_vec_dot_q8_0_q8_0(k, vx, vy, is);
        const blk_q8_0 *y = (const blk_q8_0 *)vy;
        for (int64_t b = 0; b < nb; b++) {
            const uint16_t hx = type == ORC_TYPE_Q4_0 ? ((const blk_q4_0 *)vx)[b].d : ((const blk_q8_0 *)vx)[b].d;
            const double t = (double)H2F(hx) * (double)H2F(y[b].d) * (double)is[b];
            s += t; sa += fabs(t);
        }
    } else if (type == ORC_TYPE_Q5_0 || type == ORC_TYPE_IQ4_NL) {
        if (type == ORC_TYPE_Q5_0) orc_vec_dot_q5_0_q8_0(k, vx, vy, is);
        else                       orc_vec_dot_iq4_nl_q8_0(k, vx, vy, is);
        const blk_q8_0 *y = (const blk_q8_0 *)vy;
        for (int64_t b = 0; b < nb; b++) {
            const uint16_t hx = type == ORC_TYPE_Q5_0 ? ((const blk_q5_0 *)vx)[b].d : ((const blk_iq4_nl *)vx)[b].d;
            const double t = (double)H2F(hx) * (double)H2F(y[b].d) * (double)is[b];
            s += t; sa += fabs(t);
        }
    } else if (type == ORC_TYPE_F16) {
        const uint16_t *x = (const uint16_t *)vx, *y = (const uint16_t *)vy;
        for (int64_t i = 0; i < k; i++) {
            const double t = (double)H2F(x[i]) * (double)H2F(y[i]);
            s += t; sa += fabs(t);
        }
    } else if (type == ORC_TYPE_Q4_1 || type == ORC_TYPE_Q5_1) {
        dot_min32(type, k, vx, vy, is);
        const blk_q8_1 *y = (const blk_q8_1 *)vy;
        for (int64_t b = 0; b < nb; b++) {
            const uint16_t dh = type == ORC_TYPE_Q4_1 ? ((const blk_q4_1 *)vx)[b].d : ((const blk_q5_1 *)vx)[b].d;
            const uint16_t mh = type == ORC_TYPE_Q4_1 ? ((const blk_q4_1 *)vx)[b].m : ((const blk_q5_1 *)vx)[b].m;
            const double t1 = (double)H2F(dh) * (double)H2F(y[b].d) * (double)is[b];
            const double t2 = (double)H2F(mh) * (double)H2F(y[b].s);
            s += t1 + t2; sa += fabs(t1) + fabs(t2);
        }
    } else if (type == ORC_TYPE_Q5_K) {
        const blk_q5_K *x = (const blk_q5_K *)vx;
        const blk_q8_K *y = (const blk_q8_K *)vy;
        for (int64_t b = 0; b < nb; b++) {
            const double d = (double)y[b].d * (double)H2F(x[b].d), dm = (double)y[b].d * (double)H2F(x[b].dmin);
            for (int j = 0; j < 8; j++) {
                uint8_t sc, m;
                unpack_sc_m(j, x[b].scales, &sc, &m);
                const uint8_t *q5 = x[b].qs + 32 * (j / 2);
                const int8_t *q8 = y[b].qs + 32 * j;
                int64_t dot = 0;
                for (int l = 0; l < 32; l++) {
                    const int q = ((j & 1) ? (q5[l] >> 4) : (q5[l] & 0xF)) + (((x[b].qh[l] >> j) & 1) << 4);
                    dot += (int64_t)q * q8[l];
                }
                const double t1 = d * (double)sc * (double)dot;
                const double t2 = dm * (double)m * (double)(y[b].bsums[2 * j] + y[b].bsums[2 * j + 1]);
                s += t1 - t2; sa += fabs(t1) + fabs(t2);
            }
        }
    } else if (type == ORC_TYPE_Q4_K) {
        /* terms at sub-block granularity (32 values with their own 6-bit scale and min) */
        const blk_q4_K *x = (const blk_q4_K *)vx;
        const blk_q8_K *y = (const blk_q8_K *)vy;
        for (int64_t b = 0; b < nb; b++) {
            const double d = (double)y[b].d * (double)H2F(x[b].d), dm = (double)y[b].d * (double)H2F(x[b].dmin);
            for (int j = 0; j < 8; j++) {
                uint8_t sc, m;
                unpack_sc_m(j, x[b].scales, &sc, &m);
                const uint8_t *q4 = x[b].qs + 32 * (j / 2);
                const int8_t *q8 = y[b].qs + 32 * j;
                int64_t dot = 0;
                for (int l = 0; l < 32; l++) dot += (int64_t)((j & 1) ? (q4[l] >> 4) : (q4[l] & 0xF)) * q8[l];
                const double t1 = d * (double)sc * (double)dot;
                const double t2 = dm * (double)m * (double)(y[b].bsums[2 * j] + y[b].bsums[2 * j + 1]);
                s += t1 - t2; sa += fabs(t1) + fabs(t2);
            }
        }
    } else if (type == ORC_TYPE_Q6_K) {
        /* terms at sub-block granularity (16 values with their own int8 scale) */
        const int64_t n6 = k;
        float *wi = (float *)malloc(sizeof(float) * (size_t)(n6 > 0 ? n6 : 1));
        blk_q6_K *tmp = (blk_q6_K *)malloc(sizeof(blk_q6_K) * (size_t)(nb > 0 ? nb : 1));
        const blk_q6_K *x = (const blk_q6_K *)vx;
        const blk_q8_K *y = (const blk_q8_K *)vy;
        /* dequantize with d = 1 and unit scales to recover the integers q-32 in element order */
        memcpy(tmp, x, sizeof(blk_q6_K) * (size_t)nb);
        for (int64_t b = 0; b < nb; b++) { tmp[b].d = 0x3c00; for (int g = 0; g < 16; g++) tmp[b].scales[g] = 1; }
        orc_dequantize_row(ORC_TYPE_Q6_K, tmp, wi, k);
        for (int64_t b = 0; b < nb; b++) {
            const double d = (double)y[b].d * (double)H2F(x[b].d);
            for (int g = 0; g < 16; g++) {
                int64_t dot = 0;
                for (int l = 0; l < 16; l++) dot += (int64_t)wi[256 * b + 16 * g + l] * y[b].qs[16 * g + l];
                const double t = d * (double)x[b].scales[g] * (double)dot;
                s += t; sa += fabs(t);
            }
        }
        free(wi); free(tmp);
    } else if (type == ORC_TYPE_Q2_K || type == ORC_TYPE_Q3_K) {
        /* terms at sub-block granularity (16 values): d*sc_g*dot_g, and for q2_K dmin*m_g*bsum_g */
        float *wi = (float *)malloc(sizeof(float) * (size_t)(k > 0 ? k : 1));
        const blk_q8_K *y = (const blk_q8_K *)vy;
        for (int64_t b = 0; b < nb; b++) {
            double d, dm = 0;
            int sc[16], mn[16];
            if (type == ORC_TYPE_Q2_K) {
                blk_q2_K t = ((const blk_q2_K *)vx)[b];
                d = (double)y[b].d * (double)H2F(t.d); dm = (double)y[b].d * (double)H2F(t.dmin);
                for (int g = 0; g < 16; g++) { sc[g] = t.scales[g] & 0xF; mn[g] = t.scales[g] >> 4; t.scales[g] = 1; }
                t.d = 0x3c00; t.dmin = 0;                 /* d = 1, unit scales, no mins: the integers q in element order */
                orc_dequantize_row(ORC_TYPE_Q2_K, &t, wi + 256 * b, 256);
            } else {
                blk_q3_K t = ((const blk_q3_K *)vx)[b];
                int8_t s8[16];
                d = (double)y[b].d * (double)H2F(t.d);
                q3_K_scales(t.scales, s8);
                for (int g = 0; g < 16; g++) { sc[g] = s8[g] - 32; mn[g] = 0; }
                /* scales of 33 - 32 = 1 in every position: low nibbles 1, high bit pairs 2 */
                for (int i = 0; i < 8; i++) t.scales[i] = 0x11;
                for (int i = 8; i < 12; i++) t.scales[i] = 0xAA;
                t.d = 0x3c00;
                orc_dequantize_row(ORC_TYPE_Q3_K, &t, wi + 256 * b, 256);
            }
            for (int g = 0; g < 16; g++) {
                int64_t dot = 0;
                for (int l = 0; l < 16; l++) dot += (int64_t)wi[256 * b + 16 * g + l] * y[b].qs[16 * g + l];
                const double t1 = d * (double)sc[g] * (double)dot;
                const double t2 = dm * (double)mn[g] * (double)y[b].bsums[g];
                s += t1 - t2; sa += fabs(t1) + fabs(t2);
            }
        }
        free(wi);
    } else if (type == ORC_TYPE_IQ4_XS) {
        /* terms at sub-block granularity (32 values with their own 6-bit scale) */
        const blk_iq4_xs *x = (const blk_iq4_xs *)vx;
        const blk_q8_K *y = (const blk_q8_K *)vy;
        for (int64_t b = 0; b < nb; b++) {
            const double d = (double)H2F(x[b].d) * (double)y[b].d;
            for (int ib = 0; ib < 8; ib++) {
                const int ls = (((x[b].scales_l[ib / 2] >> 4 * (ib % 2)) & 0xf) | (((x[b].scales_h >> 2 * ib) & 3) << 4)) - 32;
                int64_t dot = 0;
                for (int j = 0; j < 16; j++) {
                    dot += (int64_t)iq4nl_values[x[b].qs[16 * ib + j] & 0xf] * y[b].qs[32 * ib + j];
                    dot += (int64_t)iq4nl_values[x[b].qs[16 * ib + j] >> 4] * y[b].qs[32 * ib + 16 + j];
                }
                const double t = d * (double)ls * (double)dot;
                s += t; sa += fabs(t);
            }
        }
    } else { s = NAN; }
    free(is);
    if (sum_abs) *sum_abs = sa;
    return s;
}

/* ---------------------------------------------------------------- MUL_MAT (ggml-cpu/ggml-cpu.c:1257-1449) */
typedef struct {
    int type; int64_t K, N, n; const char *W; const char *wd; float *y; double *sa;
    int64_t r0, r1;
} mm_job;

static void *mm_worker(void *p) {
    mm_job *j = (mm_job *)p;
    const size_t wrs = orc_row_size(j->type, j->K);
    const size_t ars = orc_row_size(orc_vec_dot_type(j->type), j->K);
    for (int64_t t = 0; t < j->n; t++) {
        for (int64_t r = j->r0; r < j->r1; r++) {
            const void *wr = j->W + (size_t)r * wrs;
            const void *ar = j->wd + (size_t)t * ars;
            j->y[t * j->N + r] = orc_vec_dot(j->type, j->K, wr, ar);
            if (j->sa) orc_vec_dot_exact(j->type, j->K, wr, ar, &j->sa[t * j->N + r]);
        }
    }
    return NULL;
}

void orc_mul_mat(int type, int64_t K, int64_t N, int64_t n, const void *W, const float *x, float *y,
                 void *wdata, double *sum_abs, int nthreads) {
    const int vdt = orc_vec_dot_type(type);
    if (vdt < 0) return;
    const size_t ars = orc_row_size(vdt, K);
    char *wd = wdata ? (char *)wdata : (char *)malloc(ars * (size_t)(n > 0 ? n : 1));
    for (int64_t t = 0; t < n; t++) {
        if (vdt == ORC_TYPE_Q8_0)      orc_quantize_row_q8_0(x + t * K, wd + (size_t)t * ars, K);
        else if (vdt == ORC_TYPE_Q8_1) orc_quantize_row_q8_1(x + t * K, wd + (size_t)t * ars, K);
        else if (vdt == ORC_TYPE_F16)  orc_fp32_to_fp16_row(x + t * K, wd + (size_t)t * ars, K);
        else                           orc_quantize_row_q8_K(x + t * K, wd + (size_t)t * ars, K);
    }
    if (nthreads < 1) nthreads = 1;
    if (nthreads > 256) nthreads = 256;
    if ((int64_t)nthreads > N) nthreads = (int)(N > 0 ? N : 1);
    pthread_t th[256];
    mm_job jobs[256];
    for (int i = 0; i < nthreads; i++) {
        jobs[i] = (mm_job){type, K, N, n, (const char *)W, wd, y, sum_abs, N * i / nthreads, N * (i + 1) / nthreads};
        if (i > 0) pthread_create(&th[i], NULL, mm_worker, &jobs[i]);
    }
    mm_worker(&jobs[0]);
    for (int i = 1; i < nthreads; i++) pthread_join(th[i], NULL);
    if (!wdata) free(wd);
}

/* LM_GGML_OP_MUL_MAT_ID (reference ggml-cpu/ggml-cpu.c:1460-1710): n_as expert matrices of N rows each, stored one
 * after the other; for token t and slot s the expert is ids[t][s], the activation row is x[t][s % ne11] (quantized to
 * the weight type's vec_dot type like in MUL_MAT), and y[t][s][r] = vec_dot(expert row r, that activation row).  The
 * reference groups the (token, slot) pairs by expert only to schedule them; every output is this one vec_dot. */
int orc_mul_mat_id(int type, int64_t K, int64_t N, int64_t n_as, const void *W, const float *x, int64_t ne11,
                   const int32_t *ids, int64_t n_used, int64_t n_tokens, float *y, double *sum_abs, int nthreads) {
    const size_t rs = orc_row_size(type, K);
    if (orc_vec_dot_type(type) < 0 || ne11 < 1) return -1;
    for (int64_t t = 0; t < n_tokens; t++)
        for (int64_t s = 0; s < n_used; s++) {
            const int32_t e = ids[t * n_used + s];
            if (e < 0 || e >= n_as) return -2;                     /* the reference asserts */
            const float *xr = x + (size_t)(t * ne11 + s % ne11) * K;
            const size_t o = (size_t)(t * n_used + s) * N;
            orc_mul_mat(type, K, N, 1, (const char *)W + (size_t)e * N * rs, xr, y + o, NULL, sum_abs ? sum_abs + o : NULL,
                        nthreads);
        }
    return 0;
}

/* ---- the element-wise ops next to the matmuls of an FFN block ---- */

/* lm_ggml_compute_forward_rms_norm_f32 (reference ggml-cpu/ops.cpp:3270-3316): per row, the sum of the float squares
 * in double, in element order; mean and scale in float; y = x * scale (lm_ggml_vec_scale_f32: one float multiply). */
void orc_rms_norm_f32(const float *x, float *y, int64_t n_rows, int64_t ne0, float eps) {
    for (int64_t r = 0; r < n_rows; r++) {
        const float *xr = x + r * ne0;
        double sum = 0.0;
        for (int64_t i = 0; i < ne0; i++) sum += (double)(xr[i] * xr[i]);
        const float mean = (float)(sum / (double)ne0);
        const float scale = 1.0f / sqrtf(mean + eps);
        for (int64_t i = 0; i < ne0; i++) y[r * ne0 + i] = xr[i] * scale;
    }
}

/* One lane of lm_ggml_v_expf, AVX2 + FMA form (reference ggml-cpu/vec.h:615-656): round-to-nearest via the 1.5 * 2^23
 * shift, two-step range reduction, degree-5 polynomial, exponent assembled in the integer domain; |n| > 126 takes the
 * two-factor scaling path, |n| > 192 saturates through s1 * s1.  The lanes of a vector do not interact (the early
 * return computes the same value as the select). */
static float v_expf_lane(float x) {
    const float r = 0x1.8p23f;
    const float z = fmaf(x, 0x1.715476p+0f, r);
    const float n = z - r;
    const float b = fmaf(-n, 0x1.7f7d1cp-20f, fmaf(-n, 0x1.62e4p-1f, x));
    uint32_t zb, one_b;
    memcpy(&zb, &z, 4);
    const float one = 1.0f;
    memcpy(&one_b, &one, 4);
    const uint32_t e = zb << 23;
    const uint32_t kb = e + one_b;
    float k;
    memcpy(&k, &kb, 4);
    const float u = b * b;
    const float j = fmaf(fmaf(fmaf(0x1.0e4020p-7f, b, 0x1.573e2ep-5f), u, fmaf(0x1.555e66p-3f, b, 0x1.fffdb6p-2f)), u,
                         0x1.ffffecp-1f * b);
    if (!(fabsf(n) > 126.0f)) return fmaf(j, k, k);
    const uint32_t g = (n <= 0.0f) ? 0x82000000u : 0u;
    const uint32_t s1b = g + 0x7f000000u, s2b = e - g;
    float s1, s2;
    memcpy(&s1, &s1b, 4);
    memcpy(&s2, &s2b, 4);
    if (fabsf(n) > 192.0f) return s1 * s1;
    return fmaf(s2, j, s2) * s1;
}

/* lm_ggml_vec_silu_f32 (reference ggml-cpu/vec.cpp:164-186), AVX2 build: x / (1 + v_expf(-x)) for the first
 * n - n % 8 elements of a row, x / (1 + expf(-x)) with the C library's expf for the rest. */
void orc_silu_f32(const float *x, float *y, int64_t n_rows, int64_t ne0) {
    for (int64_t r = 0; r < n_rows; r++) {
        const float *xr = x + r * ne0;
        float *yr = y + r * ne0;
        int64_t i = 0;
        for (; i + 7 < ne0; i += 8)
            for (int l = 0; l < 8; l++) yr[i + l] = xr[i + l] / (1.0f + v_expf_lane(0.0f - xr[i + l]));
        for (; i < ne0; i++) yr[i] = xr[i] / (1.0f + expf(-xr[i]));
    }
}

/* LM_GGML_UNARY_OP_GELU on F32 rows: lm_ggml_vec_gelu_f32 in its LM_GGML_GELU_FP16 form (reference ggml-cpu/vec.h:16, 452-466):
 * 0 at or below -10, x at or above 10, else the entry fp16(x) of a 65536-entry fp16 table, widened.  The table is what
 * lm_ggml_cpu_init fills (ggml-cpu/ggml-cpu.c:3474-3481): entry h = fp16(lm_ggml_gelu_f32(fp32(h))) with
 * lm_ggml_gelu_f32(x) = 0.5 x (1 + tanhf(sqrt(2/pi) x (1 + 0.044715 x x))) (vec.h:428-435) and the C library's tanhf. */
void orc_gelu_table(uint16_t *table) {
    static const float coef_a = 0.044715f, sqrt_2_over_pi = 0.79788456080286535587989211986876f;
    for (uint32_t i = 0; i < 65536u; i++) {
        const float x = H2F((uint16_t)i);
        table[i] = F2H(0.5f * x * (1.0f + tanhf(sqrt_2_over_pi * x * (1.0f + coef_a * x * x))));
    }
}
void orc_gelu_f32(const float *x, float *y, int64_t n) {
    static uint16_t table[65536];
    static int ready = 0;
    if (!ready) { orc_gelu_table(table); ready = 1; }
    for (int64_t i = 0; i < n; i++) {
        if (x[i] <= -10.0f) y[i] = 0.0f;
        else if (x[i] >= 10.0f) y[i] = x[i];
        else y[i] = H2F(table[F2H(x[i])]);
    }
}

/* lm_ggml_compute_forward_soft_max_f32 (reference ggml-cpu/ops.cpp:4731-4827) with lm_ggml_vec_soft_max_f32's AVX2 branch
 * (ggml-cpu/vec.cpp:198-208, 233-238).  Row i1 of x [n_rows][ne00]: w = x * scale + slope * mask[i1 % ne01] (mask fp32
 * or fp16, one [ne01][ne00] matrix shared by all heads), max over the row, e = lm_ggml_v_expf(w - max) in groups of 8
 * with the group summed in float as ((e0+e4)+(e2+e6)) + ((e1+e5)+(e3+e7)) and the groups added in double in row
 * order, the tail (ne00 % 8) through the C library's expf; y = e * (float)(1.0 / sum).  ALiBi: head h = (i1 / ne01) %
 * n_head gets slope m0^(h+1) or m1^(2(h - n_head_log2) + 1); max_bias == 0 means slope 1. */
void orc_soft_max_f32(const float *x, const void *mask, int mask_is_f16, int64_t ne00, int64_t ne01, int64_t n_head,
                      int64_t n_rows, float scale, float max_bias, float *y) {
    const uint32_t n_head_log2 = 1u << (uint32_t)floor(log2((double)n_head));
    const float m0 = powf(2.0f, -(max_bias) / n_head_log2);
    const float m1 = powf(2.0f, -(max_bias / 2.0f) / n_head_log2);
    float *w = (float *)malloc(sizeof(float) * (size_t)(ne00 > 0 ? ne00 : 1));
    for (int64_t i1 = 0; i1 < n_rows; i1++) {
        const uint32_t h = (uint32_t)((i1 / ne01) % n_head);
        const float slope = (max_bias > 0.0f) ? (h < n_head_log2 ? powf(m0, h + 1) : powf(m1, 2 * (h - n_head_log2) + 1)) : 1.0f;
        const float *xr = x + i1 * ne00;
        float *yr = y + i1 * ne00;
        for (int64_t i = 0; i < ne00; i++) w[i] = xr[i] * scale;
        if (mask) {
            const int64_t mr = (i1 % ne01) * ne00;
            if (mask_is_f16) for (int64_t i = 0; i < ne00; i++) w[i] += slope * H2F(((const uint16_t *)mask)[mr + i]);
            else             for (int64_t i = 0; i < ne00; i++) w[i] += slope * ((const float *)mask)[mr + i];
        }
        float mx = -INFINITY;
        for (int64_t i = 0; i < ne00; i++) mx = mx > w[i] ? mx : w[i];
        double sum = 0.0;
        int64_t i = 0;
        for (; i + 7 < ne00; i += 8) {
            float e[8];
            for (int l = 0; l < 8; l++) e[l] = yr[i + l] = v_expf_lane(w[i + l] - mx);
            const float a0 = e[0] + e[4], a1 = e[1] + e[5], a2 = e[2] + e[6], a3 = e[3] + e[7];
            sum += (double)((a0 + a2) + (a1 + a3));
        }
        for (; i < ne00; i++) {
            const float v = expf(w[i] - mx);
            sum += (double)v;
            yr[i] = v;
        }
        const float inv = (float)(1.0 / sum);
        for (int64_t k = 0; k < ne00; k++) yr[k] *= inv;
    }
    free(w);
}

/* lm_ggml_compute_forward_rope_f32 (reference ggml-cpu/ops.cpp:5178-5361) for the text modes (mode 0: adjacent pairs,
 * LM_GGML_ROPE_TYPE_NEOX = 2: pairs half a rotation apart), with lm_ggml_rope_cache_init / rope_yarn (ops.cpp:5080-5118)
 * and lm_ggml_rope_yarn_corr_dims (ggml.c:3749-3761).  x, y [ne2][ne1][ne0] contiguous (token, head, channel); pos
 * [ne2]; freq_factors [n_dims / 2] or NULL.  theta runs through the float recurrence theta *= theta_scale from
 * theta = pos; cosf / sinf are the C library's. */
void orc_rope_f32(const float *x, const int32_t *pos, const float *freq_factors, int64_t ne0, int64_t ne1, int64_t ne2,
                  int n_dims, int mode, int n_ctx_orig, float freq_base, float freq_scale, float ext_factor,
                  float attn_factor, float beta_fast, float beta_slow, float *y) {
    const float theta_scale = powf(freq_base, -2.0f / n_dims);
    float corr[2];
    {
        const float lo = n_dims * logf(n_ctx_orig / (beta_fast * 2 * (float)M_PI)) / (2 * logf(freq_base));
        const float hi = n_dims * logf(n_ctx_orig / (beta_slow * 2 * (float)M_PI)) / (2 * logf(freq_base));
        const float start = floorf(lo), end = ceilf(hi);
        corr[0] = 0 > start ? 0 : start;
        corr[1] = (n_dims - 1) < end ? (float)(n_dims - 1) : end;
    }
    const int neox = mode & 2;
    float *cache = (float *)malloc(sizeof(float) * (size_t)(ne0 + 2));
    for (int64_t i2 = 0; i2 < ne2; i2++) {
        float theta = (float)(int64_t)pos[i2];
        for (int64_t i0 = 0; i0 < ne0; i0 += 2) {
            const float ff = freq_factors ? freq_factors[i0 / 2] : 1.0f;
            const float theta_extrap = theta / ff;
            const float theta_interp = freq_scale * theta_extrap;
            float th = theta_interp, mscale = attn_factor;
            if (ext_factor != 0.0f) {
                const float d = corr[1] - corr[0];
                const float yv = ((int)i0 / 2 - corr[0]) / (0.001f > d ? 0.001f : d);
                const float ramp = 1 - (1 < (0 > yv ? 0 : yv) ? 1 : (0 > yv ? 0 : yv));
                const float ramp_mix = ramp * ext_factor;
                th = theta_interp * (1 - ramp_mix) + theta_extrap * ramp_mix;
                mscale *= 1.0f + 0.1f * logf(1.0f / freq_scale);
            }
            cache[i0 + 0] = cosf(th) * mscale;
            cache[i0 + 1] = sinf(th) * mscale;
            theta *= theta_scale;
        }
        for (int64_t i1 = 0; i1 < ne1; i1++) {
            const float *src = x + (i2 * ne1 + i1) * ne0;
            float *dst = y + (i2 * ne1 + i1) * ne0;
            for (int64_t i0 = 0; i0 < n_dims; i0 += 2) {
                const float c = cache[i0], sn = cache[i0 + 1];
                const int64_t a = neox ? i0 / 2 : i0, b = neox ? i0 / 2 + n_dims / 2 : i0 + 1;
                const float x0 = src[a], x1 = src[b];
                dst[a] = x0 * c - x1 * sn;
                dst[b] = x0 * sn + x1 * c;
            }
            for (int64_t i0 = n_dims; i0 < ne0; i0++) dst[i0] = src[i0];
        }
    }
    free(cache);
}
