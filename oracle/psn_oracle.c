/*
 * psn_oracle.c -- CPU restatement of the quantized GGUF compute path.
 * TEST INFRASTRUCTURE ONLY (see psn_oracle.h for provenance and parity status).
 *
 * Block formats restated from the published GGUF definitions:
 *   Q8_0 { fp16 d; int8 qs[32]; }                                34 B / 32 w
 *   Q4_0 { fp16 d; uint8 qs[16]; }                               18 B / 32 w
 *   Q4_K { fp16 d; fp16 dmin; uint8 scales[12]; uint8 qs[128]; } 144 B / 256 w
 *   Q6_K { uint8 ql[128]; uint8 qh[64]; int8 scales[16]; fp16 d; } 210 B / 256 w
 *   Q8_K { fp32 d; int8 qs[256]; int16 bsums[16]; }              292 B / 256 x
 * Built with -ffp-contract=off so that a*b+c is two roundings everywhere.
 */
#include "psn_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define QK 32
#define QKK 256

#pragma pack(push, 1)
typedef struct { uint16_t d; int8_t qs[QK]; } blk_q8_0;
typedef struct { uint16_t d; uint8_t qs[QK / 2]; } blk_q4_0;
typedef struct { uint16_t d; uint16_t dmin; uint8_t scales[12]; uint8_t qs[QKK / 2]; } blk_q4_K;
typedef struct { uint16_t d; uint16_t dmin; uint8_t scales[12]; uint8_t qh[QKK / 8]; uint8_t qs[QKK / 2]; } blk_q5_K;
typedef struct { uint8_t ql[QKK / 2]; uint8_t qh[QKK / 4]; int8_t scales[QKK / 16]; uint16_t d; } blk_q6_K;
typedef struct { float d; int8_t qs[QKK]; int16_t bsums[QKK / 16]; } blk_q8_K;
#pragma pack(pop)

_Static_assert(sizeof(blk_q8_0) == 34, "q8_0");
_Static_assert(sizeof(blk_q4_0) == 18, "q4_0");
_Static_assert(sizeof(blk_q4_K) == 144, "q4_K");
_Static_assert(sizeof(blk_q5_K) == 176, "q5_K");
_Static_assert(sizeof(blk_q6_K) == 210, "q6_K");
_Static_assert(sizeof(blk_q8_K) == 292, "q8_K");

/* ---------------------------------------------------------------- scalars */

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* IEEE-754 binary32 -> binary16, round to nearest even, NaN kept quiet */
uint16_t orc_fp32_to_fp16(float f) {
    uint32_t u = f2u(f);
    uint32_t sign = (u >> 16) & 0x8000u;
    uint32_t mag = u & 0x7fffffffu;
    if (mag >= 0x7f800000u) {                       /* inf / nan */
        return (uint16_t)(sign | 0x7c00u | (mag > 0x7f800000u ? 0x0200u | ((mag >> 13) & 0x3ffu) : 0));
    }
    if (mag >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);   /* rounds to >= 65520 -> inf */
    if (mag < 0x33000001u) return (uint16_t)sign;                /* <= 2^-25 -> 0 (tie to even) */
    int32_t e = (int32_t)(mag >> 23) - 127;
    uint32_t man = (mag & 0x7fffffu) | 0x800000u;               /* 24-bit significand */
    uint32_t shift, half;
    if (e < -14) {                                               /* subnormal half */
        shift = (uint32_t)(13 + (-14 - e));                      /* 14..24 */
        uint32_t q = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1u);
        half = 1u << (shift - 1);
        if (rem > half || (rem == half && (q & 1u))) q++;
        return (uint16_t)(sign | q);                             /* carry into exponent is correct */
    }
    shift = 13;
    uint32_t q = ((uint32_t)(e + 15) << 10) | ((man >> shift) & 0x3ffu);
    uint32_t rem = man & 0x1fffu;
    half = 0x1000u;
    if (rem > half || (rem == half && (q & 1u))) q++;            /* may carry to next exponent / inf */
    return (uint16_t)(sign | q);
}

float orc_fp16_to_fp32(uint16_t h) {
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1fu;
    uint32_t m = h & 0x3ffu;
    if (e == 0) {
        if (m == 0) return u2f(sign);
        /* subnormal: value = m * 2^-24 */
        float v = (float)m * u2f(0x33800000u);                   /* 2^-24, exact */
        return sign ? -v : v;
    }
    if (e == 31) return u2f(sign | 0x7f800000u | (m << 13));
    return u2f(sign | ((e + 112u) << 23) | (m << 13));
}

/* round half to even through the 1.5*2^23 magic add; |f| < 2^22 */
int32_t orc_nearest_int(float f) {
    float v = f + 12582912.f;
    int32_t i = (int32_t)f2u(v);
    return (i & 0x007fffff) - 0x00400000;
}

static inline float h2f(uint16_t h) { return orc_fp16_to_fp32(h); }
static inline int imin(int a, int b) { return a < b ? a : b; }
static inline int imax(int a, int b) { return a > b ? a : b; }

int64_t orc_block_elems(int32_t t) {
    switch (t) {
        case ORC_Q4_0: case ORC_Q8_0: return QK;
        case ORC_Q4_K: case ORC_Q5_K: case ORC_Q6_K: case ORC_Q8_K: return QKK;
        default: return 0;
    }
}
int64_t orc_block_bytes(int32_t t) {
    switch (t) {
        case ORC_Q4_0: return sizeof(blk_q4_0);
        case ORC_Q8_0: return sizeof(blk_q8_0);
        case ORC_Q4_K: return sizeof(blk_q4_K);
        case ORC_Q5_K: return sizeof(blk_q5_K);
        case ORC_Q6_K: return sizeof(blk_q6_K);
        case ORC_Q8_K: return sizeof(blk_q8_K);
        default: return 0;
    }
}
int64_t orc_row_bytes(int32_t t, int64_t k) {
    int64_t be = orc_block_elems(t);
    if (be == 0 || k < 0 || k % be) return -1;
    return k / be * orc_block_bytes(t);
}

/* ------------------------------------------------------------- quantizers */

/* Q8_0: d = amax/127, q = round-half-away(x/d) */
static void quant_q8_0(const float *x, blk_q8_0 *y, int64_t k) {
    for (int64_t b = 0; b < k / QK; b++) {
        float amax = 0.f;
        for (int j = 0; j < QK; j++) { float a = fabsf(x[b * QK + j]); if (a > amax) amax = a; }
        float d = amax / 127.f;
        float id = d != 0.f ? 1.f / d : 0.f;
        y[b].d = orc_fp32_to_fp16(d);
        for (int j = 0; j < QK; j++) y[b].qs[j] = (int8_t)roundf(x[b * QK + j] * id);
    }
}

/* Q4_0: d = (signed value of largest magnitude)/-8, q = min(15, trunc(x/d + 8.5)) */
static void quant_q4_0(const float *x, blk_q4_0 *y, int64_t k) {
    for (int64_t b = 0; b < k / QK; b++) {
        const float *xb = x + b * QK;
        float amax = 0.f, vmax = 0.f;
        for (int j = 0; j < QK; j++) { float a = fabsf(xb[j]); if (a > amax) { amax = a; vmax = xb[j]; } }
        float d = vmax / -8.f;
        float id = d != 0.f ? 1.f / d : 0.f;
        y[b].d = orc_fp32_to_fp16(d);
        for (int j = 0; j < QK / 2; j++) {
            int lo = imin(15, (int)(int8_t)(xb[j] * id + 8.5f));
            int hi = imin(15, (int)(int8_t)(xb[j + QK / 2] * id + 8.5f));
            y[b].qs[j] = (uint8_t)(lo | (hi << 4));
        }
    }
}

/* Q8_K: iscale = -127/(signed max), q = min(127, nearest_int(iscale*x)), d = 1/iscale (fp32) */
static void quant_q8_K(const float *x, blk_q8_K *y, int64_t k) {
    for (int64_t b = 0; b < k / QKK; b++) {
        const float *xb = x + b * QKK;
        float amax = 0.f, vmax = 0.f;
        for (int j = 0; j < QKK; j++) { float a = fabsf(xb[j]); if (a > amax) { amax = a; vmax = xb[j]; } }
        if (amax == 0.f) { memset(&y[b], 0, sizeof(blk_q8_K)); continue; }
        float iscale = -127.f / vmax;
        for (int j = 0; j < QKK; j++) y[b].qs[j] = (int8_t)imin(127, orc_nearest_int(iscale * xb[j]));
        for (int g = 0; g < QKK / 16; g++) {
            int s = 0;
            for (int j = 0; j < 16; j++) s += y[b].qs[g * 16 + j];
            y[b].bsums[g] = (int16_t)s;
        }
        y[b].d = 1.f / iscale;
    }
}

/* Weighted least-squares fit x ~ scale*L - min_out, L in [0,nmax], trying nstep+1
 * candidate grid spacings.  Published reference search for the K-quants with a min. */
static float fit_scale_min(int n, int nmax, const float *x, const float *w, uint8_t *L,
                           float *min_out, uint8_t *Ltry, float rmin, float rdelta, int nstep) {
    float lo = x[0], hi = x[0], sw = w[0], swx = w[0] * x[0];
    for (int i = 1; i < n; i++) {
        if (x[i] < lo) lo = x[i];
        if (x[i] > hi) hi = x[i];
        sw += w[i];
        swx += w[i] * x[i];
    }
    if (lo > 0.f) lo = 0.f;
    if (hi == lo) {
        for (int i = 0; i < n; i++) L[i] = 0;
        *min_out = -lo;
        return 0.f;
    }
    float iscale = (float)nmax / (hi - lo);
    float scale = 1.f / iscale;
    float best = 0.f;
    for (int i = 0; i < n; i++) {
        int l = imax(0, imin(nmax, orc_nearest_int(iscale * (x[i] - lo))));
        L[i] = (uint8_t)l;
        float e = scale * (float)l + lo - x[i];
        best += w[i] * (e * e);
    }
    for (int s = 0; s <= nstep; s++) {
        iscale = (rmin + rdelta * (float)s + (float)nmax) / (hi - lo);
        float sl = 0.f, sl2 = 0.f, sxl = 0.f;
        for (int i = 0; i < n; i++) {
            int l = imax(0, imin(nmax, orc_nearest_int(iscale * (x[i] - lo))));
            Ltry[i] = (uint8_t)l;
            sl += w[i] * (float)l;
            sl2 += w[i] * (float)l * (float)l;
            sxl += w[i] * (float)l * x[i];
        }
        float det = sw * sl2 - sl * sl;
        if (det > 0.f) {
            float sc = (sw * sxl - swx * sl) / det;
            float mn = (sl2 * swx - sl * sxl) / det;
            if (mn > 0.f) { mn = 0.f; sc = sxl / sl2; }
            float err = 0.f;
            for (int i = 0; i < n; i++) {
                float e = sc * (float)Ltry[i] + mn - x[i];
                err += w[i] * (e * e);
            }
            if (err < best) {
                memcpy(L, Ltry, (size_t)n);
                best = err; scale = sc; lo = mn;
            }
        }
    }
    *min_out = -lo;
    return scale;
}

static void q4k_pack_scale_min(int j, uint8_t ls, uint8_t lm, uint8_t *s12) {
    if (j < 4) {
        s12[j] = (uint8_t)((s12[j] & 0xC0) | ls);
        s12[j + 4] = (uint8_t)((s12[j + 4] & 0xC0) | lm);
    } else {
        s12[j + 4] = (uint8_t)((ls & 0xF) | ((lm & 0xF) << 4));
        s12[j - 4] = (uint8_t)((s12[j - 4] & 0x3F) | ((ls >> 4) << 6));
        s12[j] = (uint8_t)((s12[j] & 0x3F) | ((lm >> 4) << 6));
    }
}

void orc_q4k_scale_min(const uint8_t *q, uint8_t sc[8], uint8_t mn[8]) {
    for (int j = 0; j < 8; j++) {
        if (j < 4) {
            sc[j] = q[j] & 63;
            mn[j] = q[j + 4] & 63;
        } else {
            sc[j] = (uint8_t)((q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4));
            mn[j] = (uint8_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4));
        }
    }
}

/* One 32-element Q4_K sub-block: importance weights sqrt(mean x^2) + |x|, 16 levels, the
 * 21-candidate search (rmin -1, step 0.1).  x ~ scale * L - min.  Exported so that tests can
 * pin the search by what the mathematics fixes; quant_q4_K calls exactly this. */
float orc_q4k_fit_subblock(const float *x, uint8_t *L, float *min_out) {
    uint8_t Ltry[32];
    float w[32], s2 = 0.f;
    for (int l = 0; l < 32; l++) s2 += x[l] * x[l];
    float av = sqrtf(s2 / 32.f);
    for (int l = 0; l < 32; l++) w[l] = av + fabsf(x[l]);
    return fit_scale_min(32, 15, x, w, L, min_out, Ltry, -1.f, 0.1f, 20);
}

static void quant_q4_K(const float *x, blk_q4_K *y, int64_t k) {
    uint8_t L[QKK];
    float mins[8], scales[8];
    for (int64_t b = 0; b < k / QKK; b++) {
        const float *xb = x + b * QKK;
        float max_scale = 0.f, max_min = 0.f;
        for (int j = 0; j < 8; j++) {
            scales[j] = orc_q4k_fit_subblock(xb + 32 * j, L + 32 * j, &mins[j]);
            if (scales[j] > max_scale) max_scale = scales[j];
            if (mins[j] > max_min) max_min = mins[j];
        }
        float inv_scale = max_scale > 0.f ? 63.f / max_scale : 0.f;
        float inv_min = max_min > 0.f ? 63.f / max_min : 0.f;
        memset(y[b].scales, 0, 12);
        for (int j = 0; j < 8; j++) {
            uint8_t ls = (uint8_t)imin(63, orc_nearest_int(inv_scale * scales[j]));
            uint8_t lm = (uint8_t)imin(63, orc_nearest_int(inv_min * mins[j]));
            q4k_pack_scale_min(j, ls, lm, y[b].scales);
        }
        y[b].d = orc_fp32_to_fp16(max_scale / 63.f);
        y[b].dmin = orc_fp32_to_fp16(max_min / 63.f);
        uint8_t sc[8], mn[8];
        orc_q4k_scale_min(y[b].scales, sc, mn);
        for (int j = 0; j < 8; j++) {
            float d = h2f(y[b].d) * (float)sc[j];
            if (d == 0.f) continue;                       /* keeps the search's L */
            float dm = h2f(y[b].dmin) * (float)mn[j];
            for (int l = 0; l < 32; l++) {
                int q = orc_nearest_int((xb[32 * j + l] + dm) / d);
                L[32 * j + l] = (uint8_t)imax(0, imin(15, q));
            }
        }
        for (int c = 0; c < 4; c++)
            for (int l = 0; l < 32; l++)
                y[b].qs[32 * c + l] = (uint8_t)(L[64 * c + l] | (L[64 * c + 32 + l] << 4));
    }
}

/* One 32-element Q5_K sub-block: the same importance weights, 32 levels, 16 candidates from rmin -0.5. */
float orc_q5k_fit_subblock(const float *x, uint8_t *L, float *min_out) {
    uint8_t Ltry[32];
    float w[32], s2 = 0.f;
    for (int l = 0; l < 32; l++) s2 += x[l] * x[l];
    float av = sqrtf(s2 / 32.f);
    for (int l = 0; l < 32; l++) w[l] = av + fabsf(x[l]);
    return fit_scale_min(32, 31, x, w, L, min_out, Ltry, -0.5f, 0.1f, 15);
}

/* Q5_K: Q4_K's super-block with a fifth bit per weight.  Sub-block scales/mins are packed exactly as in
 * Q4_K; the low four bits of the eight sub-blocks share qs like Q4_K's nibbles (sub-blocks 2c, 2c+1 in
 * bytes 32c..32c+31), bit (2c) / (2c+1) of qh[l] is the fifth bit of element l of sub-block 2c / 2c+1. */
static void quant_q5_K(const float *x, blk_q5_K *y, int64_t k) {
    uint8_t L[QKK];
    float mins[8], scales[8];
    for (int64_t b = 0; b < k / QKK; b++) {
        const float *xb = x + b * QKK;
        float max_scale = 0.f, max_min = 0.f;
        for (int j = 0; j < 8; j++) {
            scales[j] = orc_q5k_fit_subblock(xb + 32 * j, L + 32 * j, &mins[j]);
            if (scales[j] > max_scale) max_scale = scales[j];
            if (mins[j] > max_min) max_min = mins[j];
        }
        float inv_scale = max_scale > 0.f ? 63.f / max_scale : 0.f;
        float inv_min = max_min > 0.f ? 63.f / max_min : 0.f;
        memset(y[b].scales, 0, 12);
        for (int j = 0; j < 8; j++) {
            uint8_t ls = (uint8_t)imin(63, orc_nearest_int(inv_scale * scales[j]));
            uint8_t lm = (uint8_t)imin(63, orc_nearest_int(inv_min * mins[j]));
            q4k_pack_scale_min(j, ls, lm, y[b].scales);
        }
        y[b].d = orc_fp32_to_fp16(max_scale / 63.f);
        y[b].dmin = orc_fp32_to_fp16(max_min / 63.f);
        uint8_t sc[8], mn[8];
        orc_q4k_scale_min(y[b].scales, sc, mn);
        for (int j = 0; j < 8; j++) {
            float d = h2f(y[b].d) * (float)sc[j];
            if (d == 0.f) continue;
            float dm = h2f(y[b].dmin) * (float)mn[j];
            for (int l = 0; l < 32; l++) {
                int q = orc_nearest_int((xb[32 * j + l] + dm) / d);
                L[32 * j + l] = (uint8_t)imax(0, imin(31, q));
            }
        }
        memset(y[b].qh, 0, sizeof y[b].qh);
        for (int c = 0; c < 4; c++)
            for (int l = 0; l < 32; l++) {
                int l1 = L[64 * c + l], l2 = L[64 * c + 32 + l];
                if (l1 > 15) { l1 -= 16; y[b].qh[l] |= (uint8_t)(1u << (2 * c)); }
                if (l2 > 15) { l2 -= 16; y[b].qh[l] |= (uint8_t)(2u << (2 * c)); }
                y[b].qs[32 * c + l] = (uint8_t)(l1 | (l2 << 4));
            }
    }
}

/* symmetric fit x ~ scale*(L-nmax), L-nmax in [-nmax, nmax-1], weights x^2;
 * 19 candidate spacings around -nmax/max.  Published reference search for Q6_K. */
static float fit_scale_sym(int n, int nmax, const float *x, int8_t *L) {
    float amax = 0.f, vmax = 0.f;
    for (int i = 0; i < n; i++) { float a = fabsf(x[i]); if (a > amax) { amax = a; vmax = x[i]; } }
    if (amax < 1e-15f) {
        for (int i = 0; i < n; i++) L[i] = 0;
        return 0.f;
    }
    float iscale = -(float)nmax / vmax;
    float sxl = 0.f, sl2 = 0.f;
    for (int i = 0; i < n; i++) {
        int l = imax(-nmax, imin(nmax - 1, orc_nearest_int(iscale * x[i])));
        L[i] = (int8_t)(l + nmax);
        float w = x[i] * x[i];
        sxl += w * x[i] * (float)l;
        sl2 += w * (float)l * (float)l;
    }
    float scale = sl2 != 0.f ? sxl / sl2 : 0.f;
    float best = scale * sxl;
    for (int s = -9; s <= 9; s++) {
        if (s == 0) continue;
        iscale = -((float)nmax + 0.1f * (float)s) / vmax;
        sxl = sl2 = 0.f;
        for (int i = 0; i < n; i++) {
            int l = imax(-nmax, imin(nmax - 1, orc_nearest_int(iscale * x[i])));
            float w = x[i] * x[i];
            sxl += w * x[i] * (float)l;
            sl2 += w * (float)l * (float)l;
        }
        if (sl2 > 0.f && sxl * sxl > best * sl2) {
            for (int i = 0; i < n; i++) {
                int l = imax(-nmax, imin(nmax - 1, orc_nearest_int(iscale * x[i])));
                L[i] = (int8_t)(l + nmax);
            }
            scale = sxl / sl2;
            best = scale * sxl;
        }
    }
    return scale;
}

/* One 16-element Q6_K sub-block (64 levels, weights x^2): x ~ scale * (L - 32).  Exported for
 * the tests that pin the search; quant_q6_K calls exactly this. */
float orc_q6k_fit_subblock(const float *x, int8_t *L) { return fit_scale_sym(16, 32, x, L); }

static void quant_q6_K(const float *x, blk_q6_K *y, int64_t k) {
    int8_t L[QKK];
    float scales[16];
    for (int64_t b = 0; b < k / QKK; b++) {
        const float *xb = x + b * QKK;
        float max_scale = 0.f, max_abs = 0.f;
        for (int g = 0; g < 16; g++) {
            scales[g] = orc_q6k_fit_subblock(xb + 16 * g, L + 16 * g);
            float a = fabsf(scales[g]);
            if (a > max_abs) { max_abs = a; max_scale = scales[g]; }
        }
        if (max_abs < 1e-15f) { memset(&y[b], 0, sizeof(blk_q6_K)); continue; }
        float iscale = -128.f / max_scale;
        y[b].d = orc_fp32_to_fp16(1.f / iscale);
        for (int g = 0; g < 16; g++) y[b].scales[g] = (int8_t)imin(127, orc_nearest_int(iscale * scales[g]));
        for (int g = 0; g < 16; g++) {
            float d = h2f(y[b].d) * (float)y[b].scales[g];
            if (d == 0.f) continue;
            for (int l = 0; l < 16; l++) {
                int q = orc_nearest_int(xb[16 * g + l] / d);
                L[16 * g + l] = (int8_t)(imax(-32, imin(31, q)) + 32);
            }
        }
        for (int h = 0; h < 2; h++) {
            const int8_t *Lh = L + 128 * h;
            uint8_t *ql = y[b].ql + 64 * h, *qh = y[b].qh + 32 * h;
            for (int l = 0; l < 32; l++) {
                uint8_t a = (uint8_t)Lh[l], bq = (uint8_t)Lh[l + 32], c = (uint8_t)Lh[l + 64], e = (uint8_t)Lh[l + 96];
                ql[l] = (uint8_t)((a & 0xF) | ((c & 0xF) << 4));
                ql[l + 32] = (uint8_t)((bq & 0xF) | ((e & 0xF) << 4));
                qh[l] = (uint8_t)((a >> 4) | ((bq >> 4) << 2) | ((c >> 4) << 4) | ((e >> 4) << 6));
            }
        }
    }
}

int32_t orc_quantize_row(int32_t t, const float *x, void *y, int64_t k) {
    if (orc_row_bytes(t, k) < 0) return -1;
    switch (t) {
        case ORC_Q8_0: quant_q8_0(x, (blk_q8_0 *)y, k); return 0;
        case ORC_Q4_0: quant_q4_0(x, (blk_q4_0 *)y, k); return 0;
        case ORC_Q4_K: quant_q4_K(x, (blk_q4_K *)y, k); return 0;
        case ORC_Q5_K: quant_q5_K(x, (blk_q5_K *)y, k); return 0;
        case ORC_Q6_K: quant_q6_K(x, (blk_q6_K *)y, k); return 0;
        case ORC_Q8_K: quant_q8_K(x, (blk_q8_K *)y, k); return 0;
        default: return -1;
    }
}

int32_t orc_quantize_rows(int32_t t, const float *x, void *y, int64_t n, int64_t k, int32_t nthreads) {
    int64_t rb = orc_row_bytes(t, k);
    if (rb < 0 || n < 0) return -1;
    if (nthreads < 1) nthreads = 1;
#pragma omp parallel for num_threads(nthreads) schedule(static)
    for (int64_t r = 0; r < n; r++) orc_quantize_row(t, x + r * k, (uint8_t *)y + r * rb, k);
    return 0;
}

/* ----------------------------------------------------------- dequantizers */

static void deq_q8_0(const blk_q8_0 *x, float *y, int64_t k) {
    for (int64_t b = 0; b < k / QK; b++) {
        float d = h2f(x[b].d);
        for (int j = 0; j < QK; j++) y[b * QK + j] = (float)x[b].qs[j] * d;
    }
}
static void deq_q4_0(const blk_q4_0 *x, float *y, int64_t k) {
    for (int64_t b = 0; b < k / QK; b++) {
        float d = h2f(x[b].d);
        for (int j = 0; j < QK / 2; j++) {
            y[b * QK + j] = (float)((x[b].qs[j] & 0xF) - 8) * d;
            y[b * QK + j + QK / 2] = (float)((x[b].qs[j] >> 4) - 8) * d;
        }
    }
}
static void deq_q4_K(const blk_q4_K *x, float *y, int64_t k) {
    for (int64_t b = 0; b < k / QKK; b++) {
        float d = h2f(x[b].d), dmin = h2f(x[b].dmin);
        uint8_t sc[8], mn[8];
        orc_q4k_scale_min(x[b].scales, sc, mn);
        for (int c = 0; c < 4; c++) {
            float d1 = d * (float)sc[2 * c], m1 = dmin * (float)mn[2 * c];
            float d2 = d * (float)sc[2 * c + 1], m2 = dmin * (float)mn[2 * c + 1];
            for (int l = 0; l < 32; l++) {
                uint8_t q = x[b].qs[32 * c + l];
                y[b * QKK + 64 * c + l] = d1 * (float)(q & 0xF) - m1;
                y[b * QKK + 64 * c + 32 + l] = d2 * (float)(q >> 4) - m2;
            }
        }
    }
}
static void deq_q5_K(const blk_q5_K *x, float *y, int64_t k) {
    for (int64_t b = 0; b < k / QKK; b++) {
        float d = h2f(x[b].d), dmin = h2f(x[b].dmin);
        uint8_t sc[8], mn[8];
        orc_q4k_scale_min(x[b].scales, sc, mn);
        for (int c = 0; c < 4; c++) {
            float d1 = d * (float)sc[2 * c], m1 = dmin * (float)mn[2 * c];
            float d2 = d * (float)sc[2 * c + 1], m2 = dmin * (float)mn[2 * c + 1];
            for (int l = 0; l < 32; l++) {
                uint8_t q = x[b].qs[32 * c + l], h = x[b].qh[l];
                y[b * QKK + 64 * c + l] = d1 * (float)((q & 0xF) + ((h >> (2 * c)) & 1) * 16) - m1;
                y[b * QKK + 64 * c + 32 + l] = d2 * (float)((q >> 4) + ((h >> (2 * c + 1)) & 1) * 16) - m2;
            }
        }
    }
}
static void deq_q6_K(const blk_q6_K *x, float *y, int64_t k) {
    for (int64_t b = 0; b < k / QKK; b++) {
        float d = h2f(x[b].d);
        for (int h = 0; h < 2; h++) {
            const uint8_t *ql = x[b].ql + 64 * h, *qh = x[b].qh + 32 * h;
            const int8_t *sc = x[b].scales + 8 * h;
            float *yo = y + b * QKK + 128 * h;
            for (int l = 0; l < 32; l++) {
                int is = l / 16;
                int q1 = (int)((ql[l] & 0xF) | (((qh[l] >> 0) & 3) << 4)) - 32;
                int q2 = (int)((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32;
                int q3 = (int)((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32;
                int q4 = (int)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32;
                yo[l] = d * (float)sc[is] * (float)q1;
                yo[l + 32] = d * (float)sc[is + 2] * (float)q2;
                yo[l + 64] = d * (float)sc[is + 4] * (float)q3;
                yo[l + 96] = d * (float)sc[is + 6] * (float)q4;
            }
        }
    }
}
static void deq_q8_K(const blk_q8_K *x, float *y, int64_t k) {
    for (int64_t b = 0; b < k / QKK; b++)
        for (int j = 0; j < QKK; j++) y[b * QKK + j] = x[b].d * (float)x[b].qs[j];
}

int32_t orc_dequantize_row(int32_t t, const void *x, float *y, int64_t k) {
    if (orc_row_bytes(t, k) < 0) return -1;
    switch (t) {
        case ORC_Q8_0: deq_q8_0((const blk_q8_0 *)x, y, k); return 0;
        case ORC_Q4_0: deq_q4_0((const blk_q4_0 *)x, y, k); return 0;
        case ORC_Q4_K: deq_q4_K((const blk_q4_K *)x, y, k); return 0;
        case ORC_Q5_K: deq_q5_K((const blk_q5_K *)x, y, k); return 0;
        case ORC_Q6_K: deq_q6_K((const blk_q6_K *)x, y, k); return 0;
        case ORC_Q8_K: deq_q8_K((const blk_q8_K *)x, y, k); return 0;
        default: return -1;
    }
}

/* ------------------------------------------------- integer dot products */

static float dot_q4_0_q8_0(const blk_q4_0 *w, const blk_q8_0 *x, int64_t k) {
    float acc = 0.f;
    for (int64_t b = 0; b < k / QK; b++) {
        int s = 0;
        for (int j = 0; j < QK / 2; j++) {
            s += ((int)(w[b].qs[j] & 0xF) - 8) * (int)x[b].qs[j];
            s += ((int)(w[b].qs[j] >> 4) - 8) * (int)x[b].qs[j + QK / 2];
        }
        acc += (float)s * h2f(w[b].d) * h2f(x[b].d);
    }
    return acc;
}
static float dot_q8_0_q8_0(const blk_q8_0 *w, const blk_q8_0 *x, int64_t k) {
    float acc = 0.f;
    for (int64_t b = 0; b < k / QK; b++) {
        int s = 0;
        for (int j = 0; j < QK; j++) s += (int)w[b].qs[j] * (int)x[b].qs[j];
        acc += (float)s * (h2f(w[b].d) * h2f(x[b].d));
    }
    return acc;
}
static float dot_q4_K_q8_K(const blk_q4_K *w, const blk_q8_K *x, int64_t k) {
    float acc = 0.f;
    for (int64_t b = 0; b < k / QKK; b++) {
        uint8_t sc[8], mn[8];
        orc_q4k_scale_min(w[b].scales, sc, mn);
        int32_t isum = 0, msum = 0;
        for (int c = 0; c < 4; c++) {
            int32_t s_lo = 0, s_hi = 0;
            for (int l = 0; l < 32; l++) {
                uint8_t q = w[b].qs[32 * c + l];
                s_lo += (int)(q & 0xF) * (int)x[b].qs[64 * c + l];
                s_hi += (int)(q >> 4) * (int)x[b].qs[64 * c + 32 + l];
            }
            isum += (int32_t)sc[2 * c] * s_lo + (int32_t)sc[2 * c + 1] * s_hi;
        }
        for (int j = 0; j < 8; j++) msum += (int32_t)mn[j] * ((int32_t)x[b].bsums[2 * j] + (int32_t)x[b].bsums[2 * j + 1]);
        float d = h2f(w[b].d) * x[b].d, dm = h2f(w[b].dmin) * x[b].d;
        acc += d * (float)isum - dm * (float)msum;
    }
    return acc;
}
static float dot_q5_K_q8_K(const blk_q5_K *w, const blk_q8_K *x, int64_t k) {
    float acc = 0.f;
    for (int64_t b = 0; b < k / QKK; b++) {
        uint8_t sc[8], mn[8];
        orc_q4k_scale_min(w[b].scales, sc, mn);
        int32_t isum = 0, msum = 0;
        for (int c = 0; c < 4; c++) {
            int32_t s_lo = 0, s_hi = 0;
            for (int l = 0; l < 32; l++) {
                uint8_t q = w[b].qs[32 * c + l], h = w[b].qh[l];
                s_lo += (int)((q & 0xF) + ((h >> (2 * c)) & 1) * 16) * (int)x[b].qs[64 * c + l];
                s_hi += (int)((q >> 4) + ((h >> (2 * c + 1)) & 1) * 16) * (int)x[b].qs[64 * c + 32 + l];
            }
            isum += (int32_t)sc[2 * c] * s_lo + (int32_t)sc[2 * c + 1] * s_hi;
        }
        for (int j = 0; j < 8; j++) msum += (int32_t)mn[j] * ((int32_t)x[b].bsums[2 * j] + (int32_t)x[b].bsums[2 * j + 1]);
        float d = h2f(w[b].d) * x[b].d, dm = h2f(w[b].dmin) * x[b].d;
        acc += d * (float)isum - dm * (float)msum;
    }
    return acc;
}
static float dot_q6_K_q8_K(const blk_q6_K *w, const blk_q8_K *x, int64_t k) {
    float acc = 0.f;
    for (int64_t b = 0; b < k / QKK; b++) {
        int32_t isum = 0;
        for (int h = 0; h < 2; h++) {
            const uint8_t *ql = w[b].ql + 64 * h, *qh = w[b].qh + 32 * h;
            const int8_t *sc = w[b].scales + 8 * h, *q8 = x[b].qs + 128 * h;
            int32_t part[8] = {0, 0, 0, 0, 0, 0, 0, 0};
            for (int l = 0; l < 32; l++) {
                int is = l / 16;
                int q1 = (int)((ql[l] & 0xF) | (((qh[l] >> 0) & 3) << 4)) - 32;
                int q2 = (int)((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32;
                int q3 = (int)((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32;
                int q4 = (int)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32;
                part[is + 0] += q1 * (int)q8[l];
                part[is + 2] += q2 * (int)q8[l + 32];
                part[is + 4] += q3 * (int)q8[l + 64];
                part[is + 6] += q4 * (int)q8[l + 96];
            }
            for (int g = 0; g < 8; g++) isum += (int32_t)sc[g] * part[g];
        }
        acc += h2f(w[b].d) * x[b].d * (float)isum;
    }
    return acc;
}

float orc_vec_dot_q(int32_t t, const void *w, const void *xq, int64_t k) {
    switch (t) {
        case ORC_Q4_0: return dot_q4_0_q8_0((const blk_q4_0 *)w, (const blk_q8_0 *)xq, k);
        case ORC_Q8_0: return dot_q8_0_q8_0((const blk_q8_0 *)w, (const blk_q8_0 *)xq, k);
        case ORC_Q4_K: return dot_q4_K_q8_K((const blk_q4_K *)w, (const blk_q8_K *)xq, k);
        case ORC_Q5_K: return dot_q5_K_q8_K((const blk_q5_K *)w, (const blk_q8_K *)xq, k);
        case ORC_Q6_K: return dot_q6_K_q8_K((const blk_q6_K *)w, (const blk_q8_K *)xq, k);
        default: return NAN;
    }
}

/* ---------------------------------------------------------------- matvec */

static int is_weight_type(int32_t t) { return t == ORC_Q4_0 || t == ORC_Q8_0 || t == ORC_Q4_K || t == ORC_Q5_K || t == ORC_Q6_K; }
static int32_t act_type_for(int32_t wt) { return (wt == ORC_Q4_0 || wt == ORC_Q8_0) ? ORC_Q8_0 : ORC_Q8_K; }

int32_t orc_matvec(int32_t wt, int32_t scheme, const void *W, const float *x, float *y,
                   int64_t n, int64_t k, int32_t batch, int32_t nthreads) {
    int64_t rb = orc_row_bytes(wt, k);
    if (!is_weight_type(wt) || rb < 0 || n <= 0 || k <= 0 || batch < 1) return -1;
    if (nthreads < 1) nthreads = 1;
    if (scheme == ORC_ACT_Q8) {
        int32_t at = act_type_for(wt);
        int64_t xb = orc_row_bytes(at, k);
        uint8_t *xq = (uint8_t *)malloc((size_t)(xb * batch));
        if (!xq) return -1;
        for (int32_t b = 0; b < batch; b++) orc_quantize_row(at, x + (int64_t)b * k, xq + b * xb, k);
#pragma omp parallel for num_threads(nthreads) schedule(static)
        for (int64_t r = 0; r < n; r++)
            for (int32_t b = 0; b < batch; b++)
                y[(int64_t)b * n + r] = orc_vec_dot_q(wt, (const uint8_t *)W + r * rb, xq + b * xb, k);
        free(xq);
        return 0;
    }
    if (scheme != ORC_ACT_F32) return -1;
    int failed = 0;
#pragma omp parallel num_threads(nthreads)
    {
        float *row = (float *)malloc((size_t)k * sizeof(float));
        if (!row) {
#pragma omp atomic write
            failed = 1;
        }
#pragma omp for schedule(static)
        for (int64_t r = 0; r < n; r++) {
            if (!row) continue;
            orc_dequantize_row(wt, (const uint8_t *)W + r * rb, row, k);
            for (int32_t b = 0; b < batch; b++) {
                const float *xv = x + (int64_t)b * k;
                /* eight interleaved fp32 partial sums, then a fixed tree */
                float p[8] = {0, 0, 0, 0, 0, 0, 0, 0};
                for (int64_t i = 0; i < k; i += 8)
                    for (int j = 0; j < 8; j++) p[j] += row[i + j] * xv[i + j];
                y[(int64_t)b * n + r] = ((p[0] + p[1]) + (p[2] + p[3])) + ((p[4] + p[5]) + (p[6] + p[7]));
            }
        }
        free(row);
    }
    return failed ? -1 : 0;
}

int32_t orc_matvec_f64(int32_t wt, const void *W, const float *x, double *y,
                       int64_t n, int64_t k, int32_t batch, int32_t nthreads) {
    int64_t rb = orc_row_bytes(wt, k);
    if (!is_weight_type(wt) || rb < 0 || n <= 0 || k <= 0 || batch < 1) return -1;
    if (nthreads < 1) nthreads = 1;
#pragma omp parallel num_threads(nthreads)
    {
        float *row = (float *)malloc((size_t)k * sizeof(float));
#pragma omp for schedule(static)
        for (int64_t r = 0; r < n; r++) {
            if (!row) continue;
            orc_dequantize_row(wt, (const uint8_t *)W + r * rb, row, k);
            for (int32_t b = 0; b < batch; b++) {
                double s = 0.0;
                for (int64_t i = 0; i < k; i++) s += (double)row[i] * (double)x[(int64_t)b * k + i];
                y[(int64_t)b * n + r] = s;
            }
        }
        free(row);
    }
    return 0;
}

/* --------------------------------------------------------------- prefill */

int32_t orc_prefill(int32_t wt, const void *W, const uint16_t *X, float *Y,
                    int64_t m, int64_t n, int64_t k, int32_t nthreads) {
    int64_t rb = orc_row_bytes(wt, k);
    if (!is_weight_type(wt) || rb < 0 || m <= 0 || n <= 0 || k <= 0) return -1;
    if (nthreads < 1) nthreads = 1;
    float *Xf = (float *)malloc((size_t)(m * k) * sizeof(float));
    if (!Xf) return -1;
    for (int64_t i = 0; i < m * k; i++) Xf[i] = h2f(X[i]);
#pragma omp parallel num_threads(nthreads)
    {
        float *row = (float *)malloc((size_t)k * sizeof(float));
#pragma omp for schedule(static)
        for (int64_t r = 0; r < n; r++) {
            if (!row) continue;
            orc_dequantize_row(wt, (const uint8_t *)W + r * rb, row, k);
            for (int64_t i = 0; i < k; i++) row[i] = h2f(orc_fp32_to_fp16(row[i]));
            for (int64_t mi = 0; mi < m; mi++) {
                const float *xv = Xf + mi * k;
                float p[8] = {0, 0, 0, 0, 0, 0, 0, 0};
                for (int64_t i = 0; i < k; i += 8)
                    for (int j = 0; j < 8; j++) p[j] += row[i + j] * xv[i + j];
                Y[mi * n + r] = ((p[0] + p[1]) + (p[2] + p[3])) + ((p[4] + p[5]) + (p[6] + p[7]));
            }
        }
        free(row);
    }
    free(Xf);
    return 0;
}

int32_t orc_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
