/* Host-side GGUF weight quantizer of the library: fp32 rows -> Q4_0 / Q8_0 / Q4_K / Q5_K / Q6_K blocks,
 * and the dequantizer back to fp32 (a token's embedding row, a check of what a file holds).
 *
 * This is the import step of the path (fp32 or fp16 checkpoints become the quantized tensors that
 * psn_weight_upload takes), restating the published ggml reference quantizers so that a tensor
 * quantized here is byte-identical to one quantized by the reference's CPU path:
 *   Q8_0  d = amax/127, q = round-half-away(x/d)
 *   Q4_0  d = (value of largest magnitude)/-8, q = min(15, trunc(x/d + 8.5))
 *   Q4_K / Q5_K  eight 32-element sub-blocks, each fitted x ~ scale*L - min by a weighted
 *         least-squares search over candidate grid spacings (weights sqrt(mean x^2) + |x|);
 *         6-bit sub-block scales/mins against fp16 d / dmin, then L re-derived from the stored values
 *   Q6_K  sixteen 16-element sub-blocks, symmetric fit x ~ scale*(L-32) with weights x^2 over 19
 *         candidate spacings; int8 sub-block scales against fp16 d
 * All arithmetic is fp32 in the reference's operation order (this file is built with
 * -ffp-contract=off), rounding to nearest-even where the reference's magic-number rounding does.
 * Rows are independent; a call splits them over `threads` host threads.
 */
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <thread>
#include <vector>

#include "psn.h"

namespace {

inline uint32_t float_bits(float f) {
    uint32_t u;
    std::memcpy(&u, &f, 4);
    return u;
}
inline float bits_float(uint32_t u) {
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}
/* fp32 -> fp16 bits, round to nearest even, subnormals and overflow to infinity included */
inline uint16_t to_half_bits(float f) {
    uint32_t x = float_bits(f);
    const uint32_t sign = (x >> 16) & 0x8000u;
    x &= 0x7fffffffu;
    if (x >= 0x7f800000u) return (uint16_t)(sign | (x > 0x7f800000u ? 0x7e00u : 0x7c00u));
    if (x < 0x38800000u)                                    /* below 2^-14: the sum's mantissa counts units of 2^-24 */
        return (uint16_t)(sign | (float_bits(bits_float(x) + 0.5f) - 0x3f000000u));
    x += 0xfffu + ((x >> 13) & 1u);
    return (uint16_t)(sign | std::min<uint32_t>((x - 0x38000000u) >> 13, 0x7c00u));
}
inline float from_half_bits(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16, e = (h >> 10) & 31u, m = h & 0x3ffu;
    if (e == 0) return bits_float(sign | float_bits((float)m * 5.9604644775390625e-8f));
    if (e == 31) return bits_float(sign | 0x7f800000u | (m << 13));
    return bits_float(sign | ((e + 112u) << 23) | (m << 13));
}
inline void put_half(uint8_t *p, float f) {
    const uint16_t u = to_half_bits(f);
    std::memcpy(p, &u, 2);
}
/* nearest integer, ties to even (the reference adds 1.5 * 2^23 and reads the mantissa) */
inline int rne(float f) { return (int)std::nearbyintf(f); }
inline int clampi(int v, int lo, int hi) { return v < lo ? lo : (v > hi ? hi : v); }

/* value of largest magnitude (first one wins) and that magnitude */
inline void signed_max(const float *x, int n, float &amax, float &vmax) {
    amax = 0.f;
    vmax = 0.f;
    for (int i = 0; i < n; ++i) {
        const float a = std::fabs(x[i]);
        if (a > amax) { amax = a; vmax = x[i]; }
    }
}

void row_q8_0(const float *x, uint8_t *out, int64_t k) {
    for (int64_t b = 0; b < k / 32; ++b, x += 32, out += 34) {
        float amax, vmax;
        signed_max(x, 32, amax, vmax);
        const float d = amax / 127.f, id = d != 0.f ? 1.f / d : 0.f;
        put_half(out, d);
        for (int j = 0; j < 32; ++j) out[2 + j] = (uint8_t)(int8_t)std::roundf(x[j] * id);
    }
}

void row_q4_0(const float *x, uint8_t *out, int64_t k) {
    for (int64_t b = 0; b < k / 32; ++b, x += 32, out += 18) {
        float amax, vmax;
        signed_max(x, 32, amax, vmax);
        const float d = vmax / -8.f, id = d != 0.f ? 1.f / d : 0.f;
        put_half(out, d);
        for (int j = 0; j < 16; ++j) {
            const int lo = std::min(15, (int)(int8_t)(x[j] * id + 8.5f));
            const int hi = std::min(15, (int)(int8_t)(x[j + 16] * id + 8.5f));
            out[2 + j] = (uint8_t)(lo | (hi << 4));
        }
    }
}

/* One sub-block of the formats with a minimum: levels 0..LEVELS, STEPS+1 candidate spacings
 * (LEVELS + first + 0.1*s)/(hi - lo).  Returns the scale, *neg_min = -(fitted intercept) >= 0.
 * A candidate replaces the running (scale, intercept) when its weighted error is smaller; the
 * levels of later candidates are taken against the UPDATED intercept, as in the reference. */
template <int N, int LEVELS, int STEPS>
float fit_affine(const float *x, float first, uint8_t *L, float *neg_min) {
    float w[N], s2 = 0.f;
    for (int i = 0; i < N; ++i) s2 += x[i] * x[i];
    const float av = std::sqrt(s2 / (float)N);
    for (int i = 0; i < N; ++i) w[i] = av + std::fabs(x[i]);

    float lo = x[0], hi = x[0], sw = w[0], swx = w[0] * x[0];
    for (int i = 1; i < N; ++i) {
        lo = std::min(lo, x[i]);
        hi = std::max(hi, x[i]);
        sw += w[i];
        swx += w[i] * x[i];
    }
    if (lo > 0.f) lo = 0.f;
    if (hi == lo) {
        std::memset(L, 0, N);
        *neg_min = -lo;
        return 0.f;
    }
    float inv = (float)LEVELS / (hi - lo), scale = 1.f / inv, best = 0.f;
    for (int i = 0; i < N; ++i) {
        const int l = clampi(rne(inv * (x[i] - lo)), 0, LEVELS);
        L[i] = (uint8_t)l;
        const float e = scale * (float)l + lo - x[i];
        best += w[i] * (e * e);
    }
    uint8_t cand[N];
    for (int s = 0; s <= STEPS; ++s) {
        inv = (first + 0.1f * (float)s + (float)LEVELS) / (hi - lo);
        float sl = 0.f, sl2 = 0.f, sxl = 0.f;
        for (int i = 0; i < N; ++i) {
            const int l = clampi(rne(inv * (x[i] - lo)), 0, LEVELS);
            cand[i] = (uint8_t)l;
            sl += w[i] * (float)l;
            sl2 += w[i] * (float)l * (float)l;
            sxl += w[i] * (float)l * x[i];
        }
        const float det = sw * sl2 - sl * sl;
        if (!(det > 0.f)) continue;
        float sc = (sw * sxl - swx * sl) / det, ic = (sl2 * swx - sl * sxl) / det;
        if (ic > 0.f) { ic = 0.f; sc = sxl / sl2; }
        float err = 0.f;
        for (int i = 0; i < N; ++i) {
            const float e = sc * (float)cand[i] + ic - x[i];
            err += w[i] * (e * e);
        }
        if (err < best) {
            std::memcpy(L, cand, N);
            best = err;
            scale = sc;
            lo = ic;
        }
    }
    *neg_min = -lo;
    return scale;
}

/* the 12 bytes holding eight 6-bit scales and eight 6-bit mins */
inline void pack6(uint8_t *s12, int j, int ls, int lm) {
    if (j < 4) {
        s12[j] = (uint8_t)ls;
        s12[j + 4] = (uint8_t)lm;
    } else {
        s12[j + 4] = (uint8_t)((ls & 15) | ((lm & 15) << 4));
        s12[j - 4] |= (uint8_t)((ls >> 4) << 6);
        s12[j] |= (uint8_t)((lm >> 4) << 6);
    }
}
inline void unpack6(const uint8_t *s12, int j, int &sc, int &mn) {
    if (j < 4) {
        sc = s12[j] & 63;
        mn = s12[j + 4] & 63;
    } else {
        sc = (s12[j + 4] & 15) | ((s12[j - 4] >> 6) << 4);
        mn = (s12[j + 4] >> 4) | ((s12[j] >> 6) << 4);
    }
}

/* shared head of Q4_K (LEVELS 15, 21 candidates from -1.0) and Q5_K (LEVELS 31, 16 from -0.5):
 * fits, 6-bit packing, fp16 d/dmin at block offsets 0/2, scales at 4; L re-derived from the stored values */
template <int LEVELS, int STEPS>
void kquant_head(const float *x, uint8_t *blk, float first, uint8_t *L) {
    float scales[8], mins[8], max_scale = 0.f, max_min = 0.f;
    for (int j = 0; j < 8; ++j) {
        scales[j] = fit_affine<32, LEVELS, STEPS>(x + 32 * j, first, L + 32 * j, &mins[j]);
        max_scale = std::max(max_scale, scales[j]);
        max_min = std::max(max_min, mins[j]);
    }
    const float inv_scale = max_scale > 0.f ? 63.f / max_scale : 0.f;
    const float inv_min = max_min > 0.f ? 63.f / max_min : 0.f;
    uint8_t *s12 = blk + 4;
    std::memset(s12, 0, 12);
    for (int j = 0; j < 8; ++j)
        pack6(s12, j, std::min(63, rne(inv_scale * scales[j])), std::min(63, rne(inv_min * mins[j])));
    put_half(blk, max_scale / 63.f);
    put_half(blk + 2, max_min / 63.f);
    uint16_t db, mb;
    std::memcpy(&db, blk, 2);
    std::memcpy(&mb, blk + 2, 2);
    const float d_all = from_half_bits(db), m_all = from_half_bits(mb);
    for (int j = 0; j < 8; ++j) {
        int sc, mn;
        unpack6(s12, j, sc, mn);
        const float d = d_all * (float)sc;
        if (d == 0.f) continue;                               /* the fit's levels stay */
        const float dm = m_all * (float)mn;
        for (int l = 0; l < 32; ++l) L[32 * j + l] = (uint8_t)clampi(rne((x[32 * j + l] + dm) / d), 0, LEVELS);
    }
}

void row_q4_K(const float *x, uint8_t *out, int64_t k) {
    uint8_t L[256];
    for (int64_t b = 0; b < k / 256; ++b, x += 256, out += 144) {
        kquant_head<15, 20>(x, out, -1.f, L);
        uint8_t *qs = out + 16;
        for (int c = 0; c < 4; ++c)
            for (int l = 0; l < 32; ++l) qs[32 * c + l] = (uint8_t)(L[64 * c + l] | (L[64 * c + 32 + l] << 4));
    }
}

void row_q5_K(const float *x, uint8_t *out, int64_t k) {
    uint8_t L[256];
    for (int64_t b = 0; b < k / 256; ++b, x += 256, out += 176) {
        kquant_head<31, 15>(x, out, -0.5f, L);
        uint8_t *qh = out + 16, *qs = out + 48;
        std::memset(qh, 0, 32);
        for (int c = 0; c < 4; ++c)
            for (int l = 0; l < 32; ++l) {
                const int a = L[64 * c + l], e = L[64 * c + 32 + l];
                qh[l] |= (uint8_t)(((a >> 4) << (2 * c)) | ((e >> 4) << (2 * c + 1)));
                qs[32 * c + l] = (uint8_t)((a & 15) | ((e & 15) << 4));
            }
    }
}

/* Q6_K sub-block: symmetric levels -32..31 (stored +32), weights x^2, 19 spacings (32 + 0.1*s)/max */
float fit_symmetric16(const float *x, int8_t *L) {
    float amax, vmax;
    signed_max(x, 16, amax, vmax);
    if (amax < 1e-15f) {
        std::memset(L, 0, 16);
        return 0.f;
    }
    auto sums = [&](float inv, float &sxl, float &sl2, int8_t *store) {
        sxl = sl2 = 0.f;
        for (int i = 0; i < 16; ++i) {
            const int l = clampi(rne(inv * x[i]), -32, 31);
            if (store) store[i] = (int8_t)(l + 32);
            const float w = x[i] * x[i];
            sxl += w * x[i] * (float)l;
            sl2 += w * (float)l * (float)l;
        }
    };
    float sxl, sl2;
    sums(-32.f / vmax, sxl, sl2, L);
    float scale = sl2 != 0.f ? sxl / sl2 : 0.f, best = scale * sxl;
    for (int s = -9; s <= 9; ++s) {
        if (s == 0) continue;
        const float inv = -(32.f + 0.1f * (float)s) / vmax;
        sums(inv, sxl, sl2, nullptr);
        if (sl2 > 0.f && sxl * sxl > best * sl2) {
            float a, b2;
            sums(inv, a, b2, L);
            scale = sxl / sl2;
            best = scale * sxl;
        }
    }
    return scale;
}

void row_q6_K(const float *x, uint8_t *out, int64_t k) {
    int8_t L[256];
    for (int64_t b = 0; b < k / 256; ++b, x += 256, out += 210) {
        float scales[16], max_abs = 0.f, max_scale = 0.f;
        for (int g = 0; g < 16; ++g) {
            scales[g] = fit_symmetric16(x + 16 * g, L + 16 * g);
            const float a = std::fabs(scales[g]);
            if (a > max_abs) { max_abs = a; max_scale = scales[g]; }
        }
        if (max_abs < 1e-15f) {
            std::memset(out, 0, 210);
            continue;
        }
        uint8_t *ql = out, *qh = out + 128;
        int8_t *sc8 = reinterpret_cast<int8_t *>(out + 192);
        const float inv = -128.f / max_scale;
        put_half(out + 208, 1.f / inv);
        uint16_t db;
        std::memcpy(&db, out + 208, 2);
        const float d_all = from_half_bits(db);
        for (int g = 0; g < 16; ++g) sc8[g] = (int8_t)std::min(127, rne(inv * scales[g]));
        for (int g = 0; g < 16; ++g) {
            const float d = d_all * (float)sc8[g];
            if (d == 0.f) continue;
            for (int l = 0; l < 16; ++l) L[16 * g + l] = (int8_t)(clampi(rne(x[16 * g + l] / d), -32, 31) + 32);
        }
        for (int h = 0; h < 2; ++h)
            for (int l = 0; l < 32; ++l) {
                const uint8_t a = (uint8_t)L[128 * h + l], c = (uint8_t)L[128 * h + 32 + l];
                const uint8_t e = (uint8_t)L[128 * h + 64 + l], f = (uint8_t)L[128 * h + 96 + l];
                ql[64 * h + l] = (uint8_t)((a & 15) | ((e & 15) << 4));
                ql[64 * h + 32 + l] = (uint8_t)((c & 15) | ((f & 15) << 4));
                qh[32 * h + l] = (uint8_t)((a >> 4) | ((c >> 4) << 2) | ((e >> 4) << 4) | ((f >> 4) << 6));
            }
    }
}

/* ---- the inverse direction: blocks -> fp32, the published dequantize_row_* formulas in their fp32
 *      operation order (value = (d * sub-block scale) * level - (dmin * sub-block min)) ---------- */
inline float half_at(const uint8_t *p) {
    uint16_t u;
    std::memcpy(&u, p, 2);
    return from_half_bits(u);
}

void deq_q4_0(const uint8_t *in, float *y, int64_t k) {
    for (int64_t b = 0; b < k / 32; ++b, in += 18, y += 32) {
        const float d = half_at(in);
        for (int j = 0; j < 16; ++j) {
            y[j] = (float)((in[2 + j] & 15) - 8) * d;
            y[j + 16] = (float)((in[2 + j] >> 4) - 8) * d;
        }
    }
}

void deq_q8_0(const uint8_t *in, float *y, int64_t k) {
    for (int64_t b = 0; b < k / 32; ++b, in += 34, y += 32) {
        const float d = half_at(in);
        for (int j = 0; j < 32; ++j) y[j] = (float)(int8_t)in[2 + j] * d;
    }
}

/* Q4_K (HIGH false: levels at 16) and Q5_K (fifth bits at 16, low nibbles at 48) */
template <bool HIGH>
void deq_q45_K(const uint8_t *in, float *y, int64_t k) {
    for (int64_t b = 0; b < k / 256; ++b, in += HIGH ? 176 : 144, y += 256) {
        const float d = half_at(in), dmin = half_at(in + 2);
        const uint8_t *qh = in + 16, *qs = in + (HIGH ? 48 : 16);
        for (int c = 0; c < 4; ++c) {
            int s1, m1, s2, m2;
            unpack6(in + 4, 2 * c, s1, m1);
            unpack6(in + 4, 2 * c + 1, s2, m2);
            const float d1 = d * (float)s1, n1 = dmin * (float)m1, d2 = d * (float)s2, n2 = dmin * (float)m2;
            for (int l = 0; l < 32; ++l) {
                int a = qs[32 * c + l] & 15, e = qs[32 * c + l] >> 4;
                if (HIGH) {
                    a += ((qh[l] >> (2 * c)) & 1) << 4;
                    e += ((qh[l] >> (2 * c + 1)) & 1) << 4;
                }
                y[64 * c + l] = d1 * (float)a - n1;
                y[64 * c + 32 + l] = d2 * (float)e - n2;
            }
        }
    }
}

void deq_q6_K(const uint8_t *in, float *y, int64_t k) {
    for (int64_t b = 0; b < k / 256; ++b, in += 210, y += 256) {
        const uint8_t *ql = in, *qh = in + 128;
        const int8_t *sc = reinterpret_cast<const int8_t *>(in + 192);
        const float d = half_at(in + 208);
        for (int h = 0; h < 2; ++h)
            for (int l = 0; l < 32; ++l) {
                const int g = 8 * h + l / 16, hb = qh[32 * h + l];
                const int q1 = ((ql[64 * h + l] & 15) | ((hb & 3) << 4)) - 32;
                const int q2 = ((ql[64 * h + 32 + l] & 15) | (((hb >> 2) & 3) << 4)) - 32;
                const int q3 = ((ql[64 * h + l] >> 4) | (((hb >> 4) & 3) << 4)) - 32;
                const int q4 = ((ql[64 * h + 32 + l] >> 4) | (((hb >> 6) & 3) << 4)) - 32;
                y[128 * h + l] = d * (float)sc[g] * (float)q1;
                y[128 * h + 32 + l] = d * (float)sc[g + 2] * (float)q2;
                y[128 * h + 64 + l] = d * (float)sc[g + 4] * (float)q3;
                y[128 * h + 96 + l] = d * (float)sc[g + 6] * (float)q4;
            }
    }
}

using row_fn = void (*)(const float *, uint8_t *, int64_t);

row_fn row_quantizer(int32_t qtype) {
    switch (qtype) {
        case PSN_Q4_0: return row_q4_0;
        case PSN_Q8_0: return row_q8_0;
        case PSN_Q4_K: return row_q4_K;
        case PSN_Q5_K: return row_q5_K;
        case PSN_Q6_K: return row_q6_K;
        default: return nullptr;
    }
}

}  // namespace

/* rows [n][k] fp32 -> [n][row_bytes] blocks; returns 0, or -1 when the type has no quantizer.
 * The caller (psn_quantize_rows in psn_host.cpp) has checked the shape and the buffer size. */
int psn_quantize_rows_impl(int32_t qtype, const float *x, int64_t n, int64_t k, uint8_t *out, int64_t row_bytes, int32_t threads) {
    const row_fn fn = row_quantizer(qtype);
    if (!fn) return -1;
    const int64_t nt = std::max<int64_t>(1, std::min<int64_t>(threads, n));
    if (nt == 1) {
        for (int64_t r = 0; r < n; ++r) fn(x + r * k, out + r * row_bytes, k);
        return 0;
    }
    std::vector<std::thread> pool;
    pool.reserve((size_t)nt);
    for (int64_t t = 0; t < nt; ++t)
        pool.emplace_back([=] {
            for (int64_t r = n * t / nt; r < n * (t + 1) / nt; ++r) fn(x + r * k, out + r * row_bytes, k);
        });
    for (auto &th : pool) th.join();
    return 0;
}

/* rows [n][row_bytes] blocks -> [n][k] fp32; returns 0, or -1 when the type has no dequantizer.
 * The caller (psn_dequantize_rows in psn_host.cpp) has checked the shape and the buffer size. */
int psn_dequantize_rows_impl(int32_t qtype, const uint8_t *in, int64_t n, int64_t k, float *out, int64_t row_bytes) {
    void (*fn)(const uint8_t *, float *, int64_t) = nullptr;
    switch (qtype) {
        case PSN_Q4_0: fn = deq_q4_0; break;
        case PSN_Q8_0: fn = deq_q8_0; break;
        case PSN_Q4_K: fn = deq_q45_K<false>; break;
        case PSN_Q5_K: fn = deq_q45_K<true>; break;
        case PSN_Q6_K: fn = deq_q6_K; break;
        default: return -1;
    }
    for (int64_t r = 0; r < n; ++r) fn(in + r * row_bytes, out + r * k, k);
    return 0;
}
