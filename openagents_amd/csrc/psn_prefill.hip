/*
 * psn_prefill.hip -- gfx950 quantized prefill matmul  Y[m][n] = sum_k h(deq(W)[n][k]) * X[m][k]
 * for GGUF Q4_0 / Q8_0 weights (every kernel family) and Q4_K / Q5_K / Q6_K weights (the four-wave base family),
 * fp16 activations, fp32 accumulation on v_mfma_f32_32x32x16_f16.
 *
 * A workgroup of 256 threads owns a BM x BN tile of Y and walks K in steps of 64.  Per step
 *   - the X tile (BM x 64 fp16) goes global -> LDS with 16-byte direct-to-LDS loads;
 *   - the W tile is dequantized from registers: every thread keeps one 256-weight chunk of one
 *     weight row (the same 144- or 272-byte chunk the decode kernels fetch) and turns two GGUF
 *     blocks of it into 64 fp16 values, bit-exactly h(d * q): (0x6400 | q) is the fp16 1024 + q,
 *     subtracting the bias is exact, and the fp16 multiply by the block's fp16 scale rounds once;
 *   - each wave multiplies its (BM/WM) x (BN/WN) part with 32x32x16 MFMAs, operands read from LDS
 *     as 16-byte fragments (8 consecutive k per lane for both A = X rows and B = W rows).
 * LDS rows are 128 bytes (64 fp16); the eight 16-byte chunks of a row are stored XOR-swizzled by
 * (row & 7) so that the 32 rows a fragment read touches fall into distinct banks.  Two LDS
 * buffers alternate; one barrier per K step.
 *
 * Workgroup -> tile mapping is XCD-aware: workgroup b runs on XCD b % 8, and all M tiles of one
 * N tile are placed on the same XCD back to back, so a weight panel streams from HBM into one L2.
 */
#include "psn_args.h"
#include "psn_device.h"

#define UNROLL _Pragma("unroll")

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));

/* byte offset of 16-byte chunk `chunk` (0..7) of tile row `row` */
PSN_DEV int tile_off(int row, int chunk) { return row * 128 + ((chunk ^ (row & 7)) << 4); }

PSN_DEV u32 h2_bits(half2_t v) { return __builtin_bit_cast(u32, v); }
PSN_DEV half2_t bits_h2(u32 v) { return __builtin_bit_cast(half2_t, v); }

/* four bytes of v (already masked to the wanted 0..255 values) -> four fp16 (1024 + byte) in element
 * order, minus `bias`, times the block scale */
PSN_DEV void bytes_to_h4(u32 v, u32 keep, half2_t bias, half2_t d2, u32 &lo, u32 &hi) {
    const u32 t01 = __builtin_amdgcn_perm(0x64646464u, v, 0x04010400u) & keep;   /* [b0, 0x64, b1, 0x64] */
    const u32 t23 = __builtin_amdgcn_perm(0x64646464u, v, 0x04030402u) & keep;   /* [b2, 0x64, b3, 0x64] */
    lo = h2_bits((bits_h2(t01) - bias) * d2);
    hi = h2_bits((bits_h2(t23) - bias) * d2);
}

struct PfQ4_0 {
    static constexpr int DW = 36, BYTES = 144;
    static constexpr bool KQ = false;
    static PSN_DEV void load(const uint8_t *p, u32 (&w)[DW]) {
        const uint4 *q = reinterpret_cast<const uint4 *>(p);
        UNROLL for (int i = 0; i < 9; ++i) unpack4(q[i], &w[4 * i]);
    }
    /* GGUF block B of the chunk -> 32 fp16 in element order (16 dwords) */
    template <int B>
    static PSN_DEV void deq_block(const u32 (&w)[DW], u32 (&o)[16]) {
        constexpr int base = 9 * (B >> 1);
        u32 q[4], dbits;
        if constexpr ((B & 1) == 0) {
            dbits = w[base] & 0xffffu;
            UNROLL for (int i = 0; i < 4; ++i) q[i] = align2(w[base + i + 1], w[base + i]);
        } else {
            dbits = w[base + 4] >> 16;
            UNROLL for (int i = 0; i < 4; ++i) q[i] = w[base + 5 + i];
        }
        const half2_t d2 = bits_h2(dbits | (dbits << 16));
        const half2_t bias = bits_h2(0x64086408u);               /* 1032 = 1024 + 8 */
        UNROLL for (int i = 0; i < 4; ++i) {
            bytes_to_h4(q[i], 0x640f640fu, bias, d2, o[2 * i], o[2 * i + 1]);              /* elements 4i..4i+3 */
            bytes_to_h4(q[i] >> 4, 0x640f640fu, bias, d2, o[8 + 2 * i], o[8 + 2 * i + 1]); /* elements 16+4i.. */
        }
    }
    /* half H (elements 16H .. 16H+15) of GGUF block B: one nibble plane of the block's 16 bytes */
    template <int B, int H>
    static PSN_DEV void deq_half(const u32 (&w)[DW], u32 (&o)[8]) {
        constexpr int base = 9 * (B >> 1);
        u32 q[4], dbits;
        if constexpr ((B & 1) == 0) {
            dbits = w[base] & 0xffffu;
            UNROLL for (int i = 0; i < 4; ++i) q[i] = align2(w[base + i + 1], w[base + i]);
        } else {
            dbits = w[base + 4] >> 16;
            UNROLL for (int i = 0; i < 4; ++i) q[i] = w[base + 5 + i];
        }
        const half2_t d2 = bits_h2(dbits | (dbits << 16));
        const half2_t bias = bits_h2(0x64086408u);
        UNROLL for (int i = 0; i < 4; ++i) bytes_to_h4(H ? q[i] >> 4 : q[i], 0x640f640fu, bias, d2, o[2 * i], o[2 * i + 1]);
    }
};

struct PfQ8_0 {
    static constexpr int DW = 68, BYTES = 272;
    static constexpr bool KQ = false;
    static PSN_DEV void load(const uint8_t *p, u32 (&w)[DW]) {
        const uint4 *q = reinterpret_cast<const uint4 *>(p);
        UNROLL for (int i = 0; i < 17; ++i) unpack4(q[i], &w[4 * i]);
    }
    template <int B>
    static PSN_DEV void deq_block(const u32 (&w)[DW], u32 (&o)[16]) {
        constexpr int base = 17 * (B >> 1);
        u32 q[8], dbits;
        if constexpr ((B & 1) == 0) {
            dbits = w[base] & 0xffffu;
            UNROLL for (int i = 0; i < 8; ++i) q[i] = align2(w[base + i + 1], w[base + i]);
        } else {
            dbits = w[base + 8] >> 16;
            UNROLL for (int i = 0; i < 8; ++i) q[i] = w[base + 9 + i];
        }
        const half2_t d2 = bits_h2(dbits | (dbits << 16));
        const half2_t bias = bits_h2(0x64806480u);               /* 1152 = 1024 + 128 */
        UNROLL for (int i = 0; i < 8; ++i)
            bytes_to_h4(q[i] ^ 0x80808080u, 0x64ff64ffu, bias, d2, o[2 * i], o[2 * i + 1]);   /* int8 + 128 */
    }
    template <int B, int H>
    static PSN_DEV void deq_half(const u32 (&w)[DW], u32 (&o)[8]) {
        constexpr int base = 17 * (B >> 1);
        u32 q[4], dbits;
        if constexpr ((B & 1) == 0) {
            dbits = w[base] & 0xffffu;
            UNROLL for (int i = 0; i < 4; ++i) q[i] = align2(w[base + 4 * H + i + 1], w[base + 4 * H + i]);
        } else {
            dbits = w[base + 8] >> 16;
            UNROLL for (int i = 0; i < 4; ++i) q[i] = w[base + 9 + 4 * H + i];
        }
        const half2_t d2 = bits_h2(dbits | (dbits << 16));
        const half2_t bias = bits_h2(0x64806480u);
        UNROLL for (int i = 0; i < 4; ++i) bytes_to_h4(q[i] ^ 0x80808080u, 0x64ff64ffu, bias, d2, o[2 * i], o[2 * i + 1]);
    }
};

/* ---- K-quant weights (Q4_K, Q5_K, Q6_K): a chunk is one super-block.  The reference dequantizes in fp32
 *      with one rounding per operation (d * sc, then * q, then - dmin * m); the fp16 weight the MFMA sees is
 *      that fp32 value rounded once more.  d (fp16, 11 significant bits) * sc (6 bits) * q (<= 5 bits) has at most
 *      22 significant bits, so both products are exact in fp32 and only the subtraction rounds: one fused
 *      multiply-add d1 * q - m1 returns the same fp32 value bit for bit, and converting it to fp16 with
 *      round-to-nearest-even is the second rounding (the compiler emits v_cvt_f32_ubyteN + v_fma_mix{lo,hi}_f16:
 *      two instructions per weight).  Q6_K: d * scale (19 bits) * (q - 32) (5 bits, or the power of two 32) is
 *      exact; written as fma(ds, q, -32 ds) the unsigned byte converts directly. ---- */
PSN_DEV u32 pack_h2_rn(float a, float b) {
    const half2_t v = {(_Float16)a, (_Float16)b};
    return h2_bits(v);
}
PSN_DEV void pf_kq_scales(u32 s0, u32 s1, u32 s2, u32 (&sc)[2], u32 (&mn)[2]) {
    sc[0] = s0 & 0x3f3f3f3fu;
    mn[0] = s1 & 0x3f3f3f3fu;
    sc[1] = (s2 & 0x0f0f0f0fu) | ((s0 >> 2) & 0x30303030u);
    mn[1] = ((s2 >> 4) & 0x0f0f0f0fu) | ((s1 >> 2) & 0x30303030u);
}
template <int I> PSN_DEV float pf_byte(const u32 (&v)[2]) { return (float)((v[I >> 2] >> (8 * (I & 3))) & 0xffu); }
/* four unsigned byte values of q -> d1 * q - m1, two packed pairs */
PSN_DEV void pf_affine4(u32 q, float d1, float m1, u32 &lo, u32 &hi) {
    const float v0 = __builtin_fmaf(d1, (float)(q & 0xffu), -m1), v1 = __builtin_fmaf(d1, (float)((q >> 8) & 0xffu), -m1);
    const float v2 = __builtin_fmaf(d1, (float)((q >> 16) & 0xffu), -m1), v3 = __builtin_fmaf(d1, (float)(q >> 24), -m1);
    lo = pack_h2_rn(v0, v1);
    hi = pack_h2_rn(v2, v3);
}

/* Q4_K: dword 0 = d | dmin << 16, dwords 1..3 = scales, dwords 4..35 = nibbles (sub-block 2g in the low,
 * 2g+1 in the high nibbles of bytes 32g .. 32g+31) */
struct PfQ4_K {
    static constexpr int DW = 36, BYTES = 144;
    static constexpr bool KQ = true;                          /* super-block format: deq_block is all there is */
    static PSN_DEV void load(const uint8_t *p, u32 (&w)[DW]) {
        const uint4 *q = reinterpret_cast<const uint4 *>(p);
        UNROLL for (int i = 0; i < 9; ++i) unpack4(q[i], &w[4 * i]);
    }
    template <int B>
    static PSN_DEV void deq_block(const u32 (&w)[DW], u32 (&o)[16]) {
        u32 sc[2], mn[2];
        pf_kq_scales(w[1], w[2], w[3], sc, mn);
        const float d1 = __fmul_rn(h2f_lo(w[0]), pf_byte<B>(sc)), m1 = __fmul_rn(h2f_hi(w[0]), pf_byte<B>(mn));
        UNROLL for (int i = 0; i < 8; ++i)
            pf_affine4((w[4 + 8 * (B >> 1) + i] >> (4 * (B & 1))) & 0x0f0f0f0fu, d1, m1, o[2 * i], o[2 * i + 1]);
    }
    /* elements 16 H .. 16 H + 15 of block B */
    template <int B, int H>
    static PSN_DEV void deq_half(const u32 (&w)[DW], u32 (&o)[8]) {
        u32 sc[2], mn[2];
        pf_kq_scales(w[1], w[2], w[3], sc, mn);
        const float d1 = __fmul_rn(h2f_lo(w[0]), pf_byte<B>(sc)), m1 = __fmul_rn(h2f_hi(w[0]), pf_byte<B>(mn));
        UNROLL for (int i = 0; i < 4; ++i)
            pf_affine4((w[4 + 8 * (B >> 1) + 4 * H + i] >> (4 * (B & 1))) & 0x0f0f0f0fu, d1, m1, o[2 * i], o[2 * i + 1]);
    }
};

/* Q5_K: dword 0 and the scales as Q4_K, dwords 4..11 = qh (bit j of byte l: fifth bit of element l of
 * sub-block j), dwords 12..43 = nibbles laid out as Q4_K's */
struct PfQ5_K {
    static constexpr int DW = 44, BYTES = 176;
    static constexpr bool KQ = true;
    static PSN_DEV void load(const uint8_t *p, u32 (&w)[DW]) {
        const uint4 *q = reinterpret_cast<const uint4 *>(p);
        UNROLL for (int i = 0; i < 11; ++i) unpack4(q[i], &w[4 * i]);
    }
    template <int B>
    static PSN_DEV void deq_block(const u32 (&w)[DW], u32 (&o)[16]) {
        u32 sc[2], mn[2];
        pf_kq_scales(w[1], w[2], w[3], sc, mn);
        const float d1 = __fmul_rn(h2f_lo(w[0]), pf_byte<B>(sc)), m1 = __fmul_rn(h2f_hi(w[0]), pf_byte<B>(mn));
        UNROLL for (int i = 0; i < 8; ++i) {
            const u32 nib = (w[12 + 8 * (B >> 1) + i] >> (4 * (B & 1))) & 0x0f0f0f0fu;
            const u32 top = ((w[4 + i] >> B) & 0x01010101u) << 4;
            pf_affine4(nib | top, d1, m1, o[2 * i], o[2 * i + 1]);
        }
    }
    template <int B, int H>
    static PSN_DEV void deq_half(const u32 (&w)[DW], u32 (&o)[8]) {
        u32 sc[2], mn[2];
        pf_kq_scales(w[1], w[2], w[3], sc, mn);
        const float d1 = __fmul_rn(h2f_lo(w[0]), pf_byte<B>(sc)), m1 = __fmul_rn(h2f_hi(w[0]), pf_byte<B>(mn));
        UNROLL for (int i = 0; i < 4; ++i) {
            const u32 nib = (w[12 + 8 * (B >> 1) + 4 * H + i] >> (4 * (B & 1))) & 0x0f0f0f0fu;
            const u32 top = ((w[4 + 4 * H + i] >> B) & 0x01010101u) << 4;
            pf_affine4(nib | top, d1, m1, o[2 * i], o[2 * i + 1]);
        }
    }
};

/* Q6_K: 210 bytes: ql[128] (dwords 0..31), qh[64] (32..47), int8 scales[16] (48..51), fp16 d (dword 52).
 * A super-block starts on an even byte, not on a dword: the loads are declared 2-byte aligned.  Element
 * 128 h + 32 t + l: low four bits from ql[64 h + 32 (t & 1) + l] (high nibble for t >= 2), bits 4..5 from
 * (qh[32 h + l] >> 2 t) & 3, minus 32, times d * scales[8 h + 2 t + l / 16]. */
struct __attribute__((packed, aligned(2))) pf_u4_a2 { u32 x, y, z, w; };
struct __attribute__((packed, aligned(2))) pf_u16_a2 { unsigned short v; };
struct PfQ6_K {
    static constexpr int DW = 53, BYTES = 210;
    static constexpr bool KQ = true;
    static PSN_DEV void load(const uint8_t *p, u32 (&w)[DW]) {
        const pf_u4_a2 *q = reinterpret_cast<const pf_u4_a2 *>(p);
        UNROLL for (int i = 0; i < 13; ++i) {
            const pf_u4_a2 v = q[i];
            w[4 * i] = v.x; w[4 * i + 1] = v.y; w[4 * i + 2] = v.z; w[4 * i + 3] = v.w;
        }
        w[52] = reinterpret_cast<const pf_u16_a2 *>(p + 208)->v;
    }
    template <int B>
    static PSN_DEV void deq_block(const u32 (&w)[DW], u32 (&o)[16]) {
        constexpr int h = B >> 2, t = B & 3;
        const float d = h2f_lo(w[52]);
        constexpr int si = 8 * h + 2 * t;                       /* scale of elements l < 16; l >= 16: si + 1 */
        const float ds0 = __fmul_rn(d, (float)(int)(int8_t)((w[48 + (si >> 2)] >> (8 * (si & 3))) & 0xffu));
        const float ds1 = __fmul_rn(d, (float)(int)(int8_t)((w[48 + ((si + 1) >> 2)] >> (8 * ((si + 1) & 3))) & 0xffu));
        const float dm0 = ds0 * 32.f, dm1 = ds1 * 32.f;
        UNROLL for (int i = 0; i < 8; ++i) {
            const u32 nib = (w[16 * h + 8 * (t & 1) + i] >> (4 * (t >> 1))) & 0x0f0f0f0fu;
            const u32 top = ((w[32 + 8 * h + i] >> (2 * t)) & 0x03030303u) << 4;
            const u32 q = nib | top;
            pf_affine4(q, i < 4 ? ds0 : ds1, i < 4 ? dm0 : dm1, o[2 * i], o[2 * i + 1]);
        }
    }
};

/* 64 dequantized fp16 (blocks 2P and 2P+1 of the chunk) into one swizzled tile row */
template <typename WF, int P>
PSN_DEV void stage_w_row(const u32 (&w)[WF::DW], char *tile, int row) {
    u32 o[16];
    WF::template deq_block<2 * P>(w, o);
    UNROLL for (int c = 0; c < 4; ++c)
        *reinterpret_cast<uint4 *>(tile + tile_off(row, c)) = make_uint4(o[4 * c], o[4 * c + 1], o[4 * c + 2], o[4 * c + 3]);
    WF::template deq_block<2 * P + 1>(w, o);
    UNROLL for (int c = 0; c < 4; ++c)
        *reinterpret_cast<uint4 *>(tile + tile_off(row, 4 + c)) = make_uint4(o[4 * c], o[4 * c + 1], o[4 * c + 2], o[4 * c + 3]);
}

template <typename WF, int BM, int BN, int WM, int WN>
PSN_DEV void prefill_body(const psn_prefill_args &a) {
    static_assert(WM * WN == 4, "four waves");
    static_assert(BN == 64 || BN == 128 || BN == 256, "BN");
    constexpr int NT = 64 * WM * WN;                        /* threads per workgroup */
    constexpr int TM = BM / WM / 32, TN = BN / WN / 32;     /* 32x32 MFMA tiles per wave */
    constexpr int KCH = NT / BN;                            /* 256-wide K chunks held in registers per round */
    constexpr int XBYTES = BM * 128, WBYTES = BN * 128;
    extern __shared__ uint4 psn_smem[];
    char *smem = reinterpret_cast<char *>(psn_smem);
    char *xs[2] = {smem, smem + XBYTES};
    char *ws[2] = {smem + 2 * XBYTES, smem + 2 * XBYTES + WBYTES};

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;
    const int M = a.M, N = a.N, K = a.K, C = K >> 8;

    /* XCD-aware tile choice: workgroups b, b+8, b+16, ... share an XCD; give them the M tiles of one
     * N tile in a row so that a weight panel is fetched into a single L2 */
    const int mt = (M + BM - 1) / BM, nt = (N + BN - 1) / BN;
    const int S = a.ksplit;
    const int xcd = blockIdx.x & 7, local = blockIdx.x >> 3;
    const int per_xcd_n = (nt + 7) >> 3;
    const int tile_m = local % mt, split = (local / mt) % S, tn_local = local / (mt * S);
    const int tile_n = xcd + 8 * tn_local;
    if (tn_local >= per_xcd_n || tile_n >= nt) return;            /* whole workgroup leaves together */
    const int m0 = tile_m * BM, n0 = tile_n * BN;

    float16_t acc[TM][TN];
    UNROLL for (int i = 0; i < TM; ++i) UNROLL for (int j = 0; j < TN; ++j) UNROLL for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    const int wrow = tid % BN, wsel = tid / BN;                  /* weight row and which chunk of the round */
    const uint8_t *wbase = a.W + (int64_t)min(n0 + wrow, N - 1) * a.row_bytes;
    u32 w[WF::DW], wnext[WF::DW];

    auto stage_x = [&](char *tile, int k0) {
        /* slot s = 16-byte word s of the tile in LDS order: row s/8, position s%8 holds chunk (s%8)^(row&7) */
        UNROLL for (int i = 0; i < BM * 8 / NT; ++i) {
            const int s = i * NT + tid, row = s >> 3, chunk = (s & 7) ^ (row & 7);
            const uint16_t *src = a.X + (int64_t)min(m0 + row, M - 1) * K + k0 + chunk * 8;
            __builtin_amdgcn_global_load_lds((const void *)src, (__attribute__((address_space(3))) void *)(tile + (i * NT + __builtin_amdgcn_readfirstlane(wave) * 64) * 16), 16, 0, 0);
        }
    };
    auto compute = [&](const char *xt, const char *wt) {
        UNROLL for (int kk = 0; kk < 4; ++kk) {
            half8_t af[TM], bf[TN];
            const int chunk = 2 * kk + (lane >> 5);
            UNROLL for (int i = 0; i < TM; ++i)
                af[i] = *reinterpret_cast<const half8_t *>(xt + tile_off(wm * (BM / WM) + 32 * i + (lane & 31), chunk));
            UNROLL for (int j = 0; j < TN; ++j)
                bf[j] = *reinterpret_cast<const half8_t *>(wt + tile_off(wn * (BN / WN) + 32 * j + (lane & 31), chunk));
            UNROLL for (int i = 0; i < TM; ++i) UNROLL for (int j = 0; j < TN; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i], bf[j], acc[i][j], 0, 0, 0);
        }
    };

    /* Software pipeline: while the MFMAs of step s run from one LDS buffer, step s+1 is staged into
     * the other (X by direct-to-LDS loads, W dequantized from registers), and the next round's
     * weight chunk is already on its way into a second register set. */
    const int rounds_all = (C + KCH - 1) / KCH, per_split = (rounds_all + S - 1) / S;
    const int r_begin = split * per_split, r_end = min(r_begin + per_split, rounds_all);
    if (r_begin >= r_end) return;                                 /* an empty K range adds nothing */
    auto load_chunk = [&](int chunk, u32 (&dst)[WF::DW]) {
        if (chunk < C) {
            WF::load(wbase + (int64_t)chunk * WF::BYTES, dst);
        } else {
            UNROLL for (int i = 0; i < WF::DW; ++i) dst[i] = 0;    /* scale 0: contributes nothing */
        }
    };
    load_chunk(r_begin * KCH + wsel, w);
    stage_x(xs[0], r_begin * KCH * 256);
    if (wsel == 0) stage_w_row<WF, 0>(w, ws[0], wrow);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    const int k_end = min(K, r_end * KCH * 256);
    for (int r = r_begin; r < r_end; ++r) {
        load_chunk((r + 1) * KCH + wsel, wnext);
        UNROLL for (int sub = 0; sub < 4 * KCH; ++sub) {
            const int k0 = (r * KCH * 4 + sub) * 64;
            if (k0 < k_end) {                                      /* uniform */
                const int cur = sub & 1, nxt = cur ^ 1;            /* 4*KCH is even, so parity restarts every round */
                if (k0 + 64 < k_end) {
                    stage_x(xs[nxt], k0 + 64);
                    if (sub + 1 < 4 * KCH) {
                        if (wsel == (sub + 1) / 4) {
                            switch ((sub + 1) % 4) {
                                case 0: stage_w_row<WF, 0>(w, ws[nxt], wrow); break;
                                case 1: stage_w_row<WF, 1>(w, ws[nxt], wrow); break;
                                case 2: stage_w_row<WF, 2>(w, ws[nxt], wrow); break;
                                default: stage_w_row<WF, 3>(w, ws[nxt], wrow); break;
                            }
                        }
                    } else if (wsel == 0) {
                        stage_w_row<WF, 0>(wnext, ws[nxt], wrow);
                    }
                }
                compute(xs[cur], ws[cur]);
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                __syncthreads();
            }
        }
        UNROLL for (int i = 0; i < WF::DW; ++i) w[i] = wnext[i];
    }

    /* 32x32 accumulator: lane holds column (lane & 31); register r is row 8*(r/4) + 4*(lane/32) + r%4.
     * The wave's tile position is worked out again from the thread index (opaque to the compiler), so
     * that nothing of it has to stay in a register through the K loop. */
    int tid_out = threadIdx.x;
    asm volatile("" : "+v"(tid_out));
    const int wm_out = (tid_out >> 6) / WN, wn_out = (tid_out >> 6) % WN, lane_out = tid_out & 63;
    UNROLL for (int i = 0; i < TM; ++i) UNROLL for (int j = 0; j < TN; ++j) {
        const int col = n0 + wn_out * (BN / WN) + 32 * j + (lane_out & 31);
        UNROLL for (int r = 0; r < 16; ++r) {
            const int row = m0 + wm_out * (BM / WM) + 32 * i + 8 * (r >> 2) + 4 * (lane_out >> 5) + (r & 3);
            if (row < M && col < N) {
                if (S == 1) a.Y[(int64_t)row * N + col] = acc[i][j][r];
                else unsafeAtomicAdd(&a.Y[(int64_t)row * N + col], acc[i][j][r]);
            }
        }
    }
}

/* ---- decode helpers of the producer / consumer variant: 256/BN threads share a weight row, each
 *      turning 64*BN/256 weights of a K step into fp16 ---- */

/* raw quants and fp16 scale bits of GGUF block B of a chunk */
template <int B> PSN_DEV void raw_block(const u32 (&w)[36], u32 (&q)[8], u32 &dbits) {       /* Q4_0: q[0..3] used */
    constexpr int base = 9 * (B >> 1);
    if constexpr ((B & 1) == 0) {
        dbits = w[base] & 0xffffu;
        UNROLL for (int i = 0; i < 4; ++i) q[i] = align2(w[base + i + 1], w[base + i]);
    } else {
        dbits = w[base + 4] >> 16;
        UNROLL for (int i = 0; i < 4; ++i) q[i] = w[base + 5 + i];
    }
    UNROLL for (int i = 4; i < 8; ++i) q[i] = 0;
}
template <int B> PSN_DEV void raw_block(const u32 (&w)[68], u32 (&q)[8], u32 &dbits) {       /* Q8_0 */
    constexpr int base = 17 * (B >> 1);
    if constexpr ((B & 1) == 0) {
        dbits = w[base] & 0xffffu;
        UNROLL for (int i = 0; i < 8; ++i) q[i] = align2(w[base + i + 1], w[base + i]);
    } else {
        dbits = w[base + 8] >> 16;
        UNROLL for (int i = 0; i < 8; ++i) q[i] = w[base + 9 + i];
    }
}
/* 16 weights (half H of a block given raw) -> 8 dwords of fp16 */
template <typename WF> PSN_DEV void deq16(const u32 (&q)[8], u32 dbits, int H, u32 (&o)[8]) {
    const half2_t d2 = bits_h2(dbits | (dbits << 16));
    if constexpr (WF::DW == 36) {
        const half2_t bias = bits_h2(0x64086408u);
        UNROLL for (int i = 0; i < 4; ++i) bytes_to_h4(q[i] >> (4 * H), 0x640f640fu, bias, d2, o[2 * i], o[2 * i + 1]);
    } else {
        const half2_t bias = bits_h2(0x64806480u);
        UNROLL for (int i = 0; i < 4; ++i) bytes_to_h4((H ? q[4 + i] : q[i]) ^ 0x80808080u, 0x64ff64ffu, bias, d2, o[2 * i], o[2 * i + 1]);
    }
}
/* the part of K step SUB (blocks 2*SUB, 2*SUB+1 of the chunk) that thread part `q` of P owns -> LDS */
template <typename WF, int SUB, int P>
PSN_DEV void stage_part(const u32 (&w)[WF::DW], char *tile, int row, int part) {
    if constexpr (WF::KQ) {
        /* K-quants: one producer thread per weight row (128 x 256 tile), both blocks of the step */
        static_assert(P == 1, "the K-quants have the 128 x 256 producer / consumer kernel only");
        /* (the scheduler is kept from interleaving the four halves: it would hold all 64 results at once) */
        u32 o[8];
        WF::template deq_half<2 * SUB, 0>(w, o);
        *reinterpret_cast<uint4 *>(tile + tile_off(row, 0)) = make_uint4(o[0], o[1], o[2], o[3]);
        *reinterpret_cast<uint4 *>(tile + tile_off(row, 1)) = make_uint4(o[4], o[5], o[6], o[7]);
        __builtin_amdgcn_sched_barrier(0);
        WF::template deq_half<2 * SUB, 1>(w, o);
        *reinterpret_cast<uint4 *>(tile + tile_off(row, 2)) = make_uint4(o[0], o[1], o[2], o[3]);
        *reinterpret_cast<uint4 *>(tile + tile_off(row, 3)) = make_uint4(o[4], o[5], o[6], o[7]);
        __builtin_amdgcn_sched_barrier(0);
        WF::template deq_half<2 * SUB + 1, 0>(w, o);
        *reinterpret_cast<uint4 *>(tile + tile_off(row, 4)) = make_uint4(o[0], o[1], o[2], o[3]);
        *reinterpret_cast<uint4 *>(tile + tile_off(row, 5)) = make_uint4(o[4], o[5], o[6], o[7]);
        __builtin_amdgcn_sched_barrier(0);
        WF::template deq_half<2 * SUB + 1, 1>(w, o);
        *reinterpret_cast<uint4 *>(tile + tile_off(row, 6)) = make_uint4(o[0], o[1], o[2], o[3]);
        *reinterpret_cast<uint4 *>(tile + tile_off(row, 7)) = make_uint4(o[4], o[5], o[6], o[7]);
        __builtin_amdgcn_sched_barrier(0);
        return;
    } else {
    u32 qa[8], qb[8], da, db;
    raw_block<2 * SUB>(w, qa, da);
    raw_block<2 * SUB + 1>(w, qb, db);
    if constexpr (P == 1) {
        UNROLL for (int h = 0; h < 2; ++h) {
            u32 o[8];
            deq16<WF>(qa, da, h, o);
            *reinterpret_cast<uint4 *>(tile + tile_off(row, 2 * h)) = make_uint4(o[0], o[1], o[2], o[3]);
            *reinterpret_cast<uint4 *>(tile + tile_off(row, 2 * h + 1)) = make_uint4(o[4], o[5], o[6], o[7]);
            deq16<WF>(qb, db, h, o);
            *reinterpret_cast<uint4 *>(tile + tile_off(row, 4 + 2 * h)) = make_uint4(o[0], o[1], o[2], o[3]);
            *reinterpret_cast<uint4 *>(tile + tile_off(row, 4 + 2 * h + 1)) = make_uint4(o[4], o[5], o[6], o[7]);
        }
    } else {
        const bool second = P == 2 ? part == 1 : part >= 2;        /* which of the two blocks */
        u32 q[8];
        UNROLL for (int i = 0; i < 8; ++i) q[i] = second ? qb[i] : qa[i];
        const u32 d = second ? db : da;
        if constexpr (P == 2) {
            UNROLL for (int h = 0; h < 2; ++h) {
                u32 o[8];
                deq16<WF>(q, d, h, o);
                *reinterpret_cast<uint4 *>(tile + tile_off(row, 4 * part + 2 * h)) = make_uint4(o[0], o[1], o[2], o[3]);
                *reinterpret_cast<uint4 *>(tile + tile_off(row, 4 * part + 2 * h + 1)) = make_uint4(o[4], o[5], o[6], o[7]);
            }
        } else {
            u32 o[8];
            deq16<WF>(q, d, part & 1, o);
            *reinterpret_cast<uint4 *>(tile + tile_off(row, 2 * part)) = make_uint4(o[0], o[1], o[2], o[3]);
            *reinterpret_cast<uint4 *>(tile + tile_off(row, 2 * part + 1)) = make_uint4(o[4], o[5], o[6], o[7]);
        }
    }
    }
}

/* ---- producer / consumer variant ----------------------------------------------------------------
 * Measured on MI355X: a wave's own VALU work does not overlap its MFMAs (decode-only and MFMA-only
 * runs of the kernels above add up to the full run), so the weight decode has to come from OTHER
 * waves of the same SIMD.  512 threads: waves 0-3 only multiply (each a quarter of the BM x BN tile),
 * waves 4-7 only stage -- X three K steps ahead by direct-to-LDS loads into four per-stage arrays,
 * W one step ahead decoded from registers into two arrays.  One raw barrier per K step; producers
 * wait only for the X stage that is due. */
template <typename WF, int BM, int BN>
PSN_DEV void prefill_body_ws(const psn_prefill_args &a) {
    constexpr int NP = 256;                                 /* producer threads */
    constexpr int P = NP / BN;                              /* producer threads per weight row */
    constexpr int WM = 2, WN = 2;
    constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
    constexpr int NX = BM * 8 / NP;
    constexpr int NW = WF::DW / 4;
    static_assert(P >= 1 && NX >= 1, "tile");
    __shared__ uint4 xs0[BM * 8], xs1[BM * 8], xs2[BM * 8], xs3[BM * 8];
    __shared__ uint4 ws0[BN * 8], ws1[BN * 8];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const bool producer = wave >= 4;                        /* wave-uniform */
    const int M = a.M, N = a.N, K = a.K, C = K >> 8;
    const int mt = (M + BM - 1) / BM, nt = (N + BN - 1) / BN;
    const int S = a.ksplit;
    const int xcd = blockIdx.x & 7, local = blockIdx.x >> 3;
    const int per_xcd_n = (nt + 7) >> 3;
    const int tile_m = local % mt, split = (local / mt) % S, tn_local = local / (mt * S);
    const int tile_n = xcd + 8 * tn_local;
    if (tn_local >= per_xcd_n || tile_n >= nt) return;
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int per_split = (C + S - 1) / S;
    const int c_begin = split * per_split, c_end = min(c_begin + per_split, C);
    if (c_begin >= c_end) return;
    const int k_last = c_end * 256 - 64;

    if (producer) {
        const int ptid = tid - 256;
        const int pwave = __builtin_amdgcn_readfirstlane(wave) - 4;   /* scalar: it addresses the LDS side of the DMA */
        const int wrow = ptid % BN, part = ptid / BN;
        const uint8_t *wbase = a.W + (int64_t)min(n0 + wrow, N - 1) * a.row_bytes;
        u32 w[WF::DW], wnext[WF::DW];
        auto stage_x = [&](uint4 *tile, int k0) {
            k0 = min(k0, k_last);
            UNROLL for (int i = 0; i < NX; ++i) {
                const int s_ = i * NP + ptid, row = s_ >> 3, chunk = (s_ & 7) ^ (row & 7);
                const uint16_t *src = a.X + (int64_t)min(m0 + row, M - 1) * K + k0 + chunk * 8;
                __builtin_amdgcn_global_load_lds((const void *)src, (__attribute__((address_space(3))) void *)(tile + i * NP + pwave * 64), 16, 0, 0);
            }
        };
        WF::load(wbase + (int64_t)c_begin * WF::BYTES, w);
        const int k_begin = c_begin * 256;
        stage_x(xs0, k_begin);
        stage_x(xs1, k_begin + 64);
        stage_x(xs2, k_begin + 128);
        stage_part<WF, 0, P>(w, reinterpret_cast<char *>(ws0), wrow, part);
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
#define PSN_WS_PRODUCE(SUB, NSUB, wsrc, xp, wq, KEEP)                                                 \
        {                                                                                             \
            stage_x(xp, (c * 4 + SUB + 3) * 64);                                               \
            stage_part<WF, NSUB, P>(wsrc, reinterpret_cast<char *>(wq), wrow, part);                  \
            asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(KEEP) : "memory");            \
        }
        for (int c = c_begin; c < c_end; ++c) {
            WF::load(wbase + (int64_t)min(c + 1, C - 1) * WF::BYTES, wnext);
            PSN_WS_PRODUCE(0, 1, w, xs3, ws1, 2 * NX + NW)
            PSN_WS_PRODUCE(1, 2, w, xs0, ws0, 2 * NX + NW)
            PSN_WS_PRODUCE(2, 3, w, xs1, ws1, 2 * NX)
            PSN_WS_PRODUCE(3, 0, wnext, xs2, ws0, 2 * NX)
            UNROLL for (int i = 0; i < WF::DW; ++i) w[i] = wnext[i];
        }
#undef PSN_WS_PRODUCE
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        return;
    }

    /* consumers */
    const int wm = wave / WN, wn = wave % WN;
    float16_t acc[TM][TN];
    UNROLL for (int i = 0; i < TM; ++i) UNROLL for (int j = 0; j < TN; ++j) UNROLL for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
    auto load_frags = [&](const uint4 *xt, const uint4 *wt, int kk, half8_t (&af)[TM], half8_t (&bf)[TN]) {
        const int chunk = 2 * kk + (lane >> 5);
        UNROLL for (int i = 0; i < TM; ++i)
            af[i] = *reinterpret_cast<const half8_t *>(reinterpret_cast<const char *>(xt) + tile_off(wm * (BM / WM) + 32 * i + (lane & 31), chunk));
        UNROLL for (int j = 0; j < TN; ++j)
            bf[j] = *reinterpret_cast<const half8_t *>(reinterpret_cast<const char *>(wt) + tile_off(wn * (BN / WN) + 32 * j + (lane & 31), chunk));
    };
    auto mfmas = [&](const half8_t (&af)[TM], const half8_t (&bf)[TN]) {
        UNROLL for (int i = 0; i < TM; ++i) UNROLL for (int j = 0; j < TN; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i], bf[j], acc[i][j], 0, 0, 0);
    };
    asm volatile("s_barrier" ::: "memory");                  /* the prologue stages are in place */
#define PSN_WS_CONSUME(xc, wc)                                                                        \
    {                                                                                                 \
        half8_t af0[TM], bf0[TN], af1[TM], bf1[TN];                                                   \
        load_frags(xc, wc, 0, af0, bf0);                                                              \
        load_frags(xc, wc, 1, af1, bf1);                                                              \
        mfmas(af0, bf0);                                                                              \
        load_frags(xc, wc, 2, af0, bf0);                                                              \
        mfmas(af1, bf1);                                                                              \
        load_frags(xc, wc, 3, af1, bf1);                                                              \
        mfmas(af0, bf0);                                                                              \
        mfmas(af1, bf1);                                                                              \
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");                               \
    }
    for (int c = c_begin; c < c_end; ++c) {
        PSN_WS_CONSUME(xs0, ws0)
        PSN_WS_CONSUME(xs1, ws1)
        PSN_WS_CONSUME(xs2, ws0)
        PSN_WS_CONSUME(xs3, ws1)
    }
#undef PSN_WS_CONSUME
    UNROLL for (int i = 0; i < TM; ++i) UNROLL for (int j = 0; j < TN; ++j) {
        const int col = n0 + wn * (BN / WN) + 32 * j + (lane & 31);
        UNROLL for (int r = 0; r < 16; ++r) {
            const int row = m0 + wm * (BM / WM) + 32 * i + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
            if (row < M && col < N) {
                if (S == 1) a.Y[(int64_t)row * N + col] = acc[i][j][r];
                else unsafeAtomicAdd(&a.Y[(int64_t)row * N + col], acc[i][j][r]);
            }
        }
    }
}

/* ---- skinny variant (M <= 64) ---------------------------------------------------------------------
 * With at most 64 activation rows the matmul is a weight stream (HBM-bound), and a workgroup's 64-wide K
 * step carries so little arithmetic (a 64 x 64 tile: 16 MFMAs) that the step time of the kernels above
 * is their per-step chain of barrier, decode and memory latency.  This kernel has no per-step
 * synchronization at all:
 *   - everything arrives by direct-to-LDS loads into rings of dynamic LDS, a whole 256-wide chunk of K
 *     at a time: X (64 rows x 256 k, four swizzled 64-k tiles) and the raw GGUF bytes of 64 weight rows
 *     exactly as they sit in memory.  X comes out of the L2 caches (every workgroup walks all of it) and
 *     needs two chunks in flight; the weight bytes come from HBM and need as many bytes in flight as LDS
 *     can hold.  Loads of one wave complete in issue order, so a wave can only wait for "all but the
 *     youngest n" of its own loads: waves 0..3 issue the X loads and waves 4..7 the weight loads, each
 *     ring with its own depth;
 *   - eight waves multiply; a chunk is eight GGUF blocks and wave w owns block w (two k16 slices) of
 *     every chunk, for the whole 64 x 64 tile.  A wave decodes the weights its own MFMA operands need
 *     straight from the raw ring (16 bytes + the fp16 scale per lane and block; for Q4_0 the same eight
 *     bytes carry both slices), so there is no fp16 weight tile, no decode stage and no producer wave;
 *   - the two waves of a SIMD (w and w+4) run in opposite phases -- waves 0..3 decode a block and then
 *     multiply it, waves 4..7 first multiply the block they decoded before -- so that one wave's decode
 *     (VALU) runs under the other's MFMAs although a barrier lines them up once per chunk;
 *   - one workgroup barrier per CHUNK (every wave waits for its own share of the next chunk's loads first);
 *   - the eight partial tiles are summed through LDS at the end, in a fixed order.
 * Loads past the end of the K range re-read its last chunk into ring slots nothing reads any more, so
 * every iteration issues the same number of loads and the outstanding-load count is a constant. */
template <typename WF> struct SkinnyRings {
    static constexpr int XR = 3;                                /* X chunks in the ring */
    /* DATA: the 16-byte words that hold a row's chunk.  Q6_K's 210-byte super-blocks start on 2-byte boundaries: what is
     * loaded is the window of fourteen aligned words that holds the super-block (rows must be whole 16-byte words, K a
     * multiple of 2048; chunk c then starts (210 c) mod 16 bytes into its window, the same for every row).
     * LROW: bytes between rows in LDS.  A wave reads the same 32-bit field of 32 different rows at a time; rows lie whole
     * 16-byte words apart, so those reads can reach only eight of the 32 banks (a four-way conflict) -- unless the rows
     * are ROTated against each other: row n is fetched from 4 rho(n) bytes before its chunk, rho(n) = (n >> RSH) & 3 (one
     * more word per row takes the bytes pushed out at the end; the bytes in front belong to the chunk or the row before).
     * With 304 (Q8_0) or 240 (Q6_K) bytes between rows all 32 rows then hit different banks.  Q4_K / Q5_K read whole
     * aligned words instead; Q4_0 stays unrotated (measured: with 160 bytes between rows its conflicts halve and the
     * kernel gets 10 % slower -- the fetches that no longer start on 16-byte words and the extra word cost more than
     * its few 32-bit reads per chunk). */
    static constexpr int DATA = (WF::BYTES % 16 == 0 ? WF::BYTES : WF::BYTES + 14 + 15) / 16;
    static constexpr bool ROT = DATA == 17 || DATA == 14;
    static constexpr int LROW = !ROT ? WF::BYTES : DATA == 17 ? 304 : 240;
    static constexpr int RSH = 3;
    static constexpr int RS = LROW <= 160 ? 6 : LROW == 176 ? 5 : LROW == 240 ? 4 : 3;   /* raw weight chunks in the ring: what 160 KB hold beside X */
    static constexpr int XBYTES = 4 * 64 * 128, RBYTES = 64 * LROW;
    static constexpr int BYTES = XR * XBYTES + RS * RBYTES;
};

/* LOADER 0: waves 0..3 (X loads; decode, then multiply); 1: wave 4 (weight loads, one more than the others;
 * multiply the block before, then decode); 2: waves 5..7.  EVEN: the wave's block index is even -- the
 * block starts on a dword (scale in the low half of its first dword, quants two bytes in: aligned dwords
 * are read and shifted; LDS reads that straddle dwords are very slow); an odd block starts two bytes
 * later (scale in the high half of the dword before, quants aligned).  Q4_K / Q5_K: the chunk is the row's
 * super-block and the wave's "block" its sub-block `wave` -- even ones sit in the low nibbles, odd ones in the
 * high nibbles of the same 32 bytes; sub-blocks 0..3 (LOADER 0) and 4..7 unpack their 6-bit scale and min
 * from different bytes of the 12-byte field; every LDS read is an aligned dword.  Q6_K: sub-block `wave` again
 * (LOADER 0: the super-block's first half; EVEN: the first 32 of a 64-byte group of ql); its fields start on
 * 2-byte boundaries, so three aligned dwords are read around each eight bytes and shifted with v_alignbyte. */
template <typename WF, int LOADER, bool EVEN>
PSN_DEV void prefill_skinny_loop(const psn_prefill_args &a, int wave, int lane, int n0, int c_begin, int nq, int rot, bool rotate_rows,
                                 u32 xs_base, u32 raw_base, __attribute__((address_space(3))) char *lds_ptr, u32 lds0, float16_t (&acc)[2][2]) {
    typedef SkinnyRings<WF> R;
    constexpr bool KQ = WF::KQ;                             /* Q4_K / Q5_K: the chunk is one super-block per row, wave w owns its sub-block w */
    constexpr bool Q4 = !KQ && WF::DW == 36;
    constexpr bool Q5K = KQ && WF::DW == 44;
    constexpr bool Q6K = KQ && WF::DW == 53;
    constexpr int XR = R::XR, RS = R::RS, XBYTES = R::XBYTES, RBYTES = R::RBYTES, LROW = R::LROW;
    constexpr int RINSTR = RBYTES / 1024;                   /* wave-wide load instructions per raw chunk: 9, 10, 11, 15 or 19 */
    constexpr int CX = 8;                                   /* X loads per X wave and chunk (32 KB over 4 waves) */
    /* raw loads per weight wave and chunk: wave 4 takes the one load that does not divide over four waves; when
     * three or two are left over (Q5_K, Q6_K) every wave issues the same number and the last waves repeat the chunk's
     * last load */
    constexpr bool EVEN_SHARE = RINSTR % 4 != 1;
    constexpr int CR = EVEN_SHARE ? (RINSTR + 3) / 4 : RINSTR / 4 + (LOADER == 1 ? 1 : 0);
    constexpr int DEPTH = LOADER == 0 ? XR : RS, PER = LOADER == 0 ? CX : CR;
    constexpr int BB = WF::BYTES / 8;                       /* Q4_0 / Q8_0: bytes of a GGUF block: 18 or 34 */
    constexpr int NP = Q4 ? 1 : 2;                          /* raw register sets per block: Q4_0 keeps both slices in the same bytes */
    static_assert(LROW % 16 == 0 && RBYTES % 1024 == 0, "whole 16-byte words per row, whole load instructions per chunk");
    const int M = a.M, N = a.N, K = a.K;
    auto chunk_of = [&](int q) { const int r = min(q, nq - 1) + rot; return c_begin + (r >= nq ? r - nq : r); };
    auto issue = [&](int q) {
        const int c = chunk_of(q);
        if constexpr (LOADER == 0) {
            const int k0 = c * 256;
            __attribute__((address_space(3))) char *dst = lds_ptr + (xs_base - lds0) + (q % XR) * XBYTES;
            UNROLL for (int u = 0; u < CX; ++u) {
                /* 16-byte word s_ of the stage in LDS order: step s_/512, row (s_%512)/8, position s_%8 holds chunk pos^(row&7) */
                const int i = wave * CX + u, s_ = i * 64 + lane, step = s_ >> 9, row = (s_ >> 3) & 63, chunk = (s_ & 7) ^ (row & 7);
                const uint16_t *src = a.X + (int64_t)min(row, M - 1) * K + k0 + step * 64 + chunk * 8;
                __builtin_amdgcn_global_load_lds((const void *)src, (__attribute__((address_space(3))) void *)(dst + i * 1024), 16, 0, 0);
            }
        } else {
            __attribute__((address_space(3))) char *dst = lds_ptr + (raw_base - lds0) + (q % RS) * RBYTES;
            UNROLL for (int u = 0; u < CR; ++u) {
                const int i = min((wave - 4) + 4 * u, RINSTR - 1);   /* instruction index (the last waves repeat the chunk's last load when the count does not divide) */
                const int word = i * 64 + lane, row = word / (LROW / 16);
                const int rho = R::ROT && rotate_rows ? ((row & 31) >> R::RSH) & 3 : 0;
                /* words past the row's data (and past the one that takes the rotated-out bytes) repeat its last one */
                const int wd = min(word % (LROW / 16), R::DATA - 1 + (rho > 0));
                const int64_t coff = Q6K ? (int64_t)((c * WF::BYTES) & ~15) : (int64_t)c * WF::BYTES;
                const uint8_t *src = a.W + (int64_t)min(n0 + row, N - 1) * a.row_bytes + coff + wd * 16 - 4 * rho;
                __builtin_amdgcn_global_load_lds((const void *)src, (__attribute__((address_space(3))) void *)(dst + i * 1024), 16, 0, 0);
            }
        }
    };
    /* this wave: block `wave` of the chunk = k16 slices 2*(wave&1) and 2*(wave&1)+1 of 64-k step wave/2.  Per-lane
     * LDS offsets inside a ring slot: the two X fragments (rows 32.. sit 4096 bytes on), the row's block
     * (rows 32.. sit 32 rows on) with and without the lane's quant offset 8h. */
    const int h = lane >> 5;
    u32 xlane[2];
    UNROLL for (int sl = 0; sl < 2; ++sl) xlane[sl] = (u32)((wave >> 1) * 8192 + tile_off(lane & 31, 2 * (2 * (wave & 1) + sl) + h));
    /* K-quants: the row's super-block; its quants of sub-block `wave` (bytes 32 (wave / 2) .. + 31 of the nibble
     * array, this lane's eight at 8h and 16 + 8h); Q5_K: the fifth bits of the same elements (qh, bit `wave`) */
    /* Q6_K, sub-block `wave` = half wave / 4, quarter t = wave % 4 of the super-block: low bits in ql[64 half + 32 (t & 1)
     * + l] (high nibble for t >= 2), bits 4..5 in qh[32 half + l] >> 2 t, int8 scales[8 half + 2 t + l / 16], d at 208 */
    const u32 rho_lane = R::ROT && rotate_rows ? (u32)(((lane & 31) >> R::RSH) & 3) : 0u;
    const u32 rlane = (KQ ? (u32)((lane & 31) * LROW) : (u32)((lane & 31) * LROW + wave * BB)) + 4u * rho_lane;
    const u32 qlane = Q6K ? rlane + (u32)(64 * (LOADER != 0) + 32 * !EVEN + 8 * h)
                    : KQ  ? rlane + (u32)((Q5K ? 48 : 16) + 32 * (wave >> 1) + 8 * h) : rlane + 8u * (u32)h;
    const u32 hlane = Q6K ? rlane + (u32)(128 + 32 * (LOADER != 0) + 8 * h) : rlane + (u32)(16 + 8 * h);
    constexpr int ROW32 = 32 * LROW;

    /* Q4_K / Q5_K: kh[j] = d | dmin << 16 and the three scale dwords, kv[j][0..1] = quants of slice 0, 1 (two dwords each),
     * kv[j][2..3] = qh likewise; Q6_K, kq[j]: 0..5 = the aligned dwords around ql (three per slice), 6..11 = around qh,
     * 12 = the two scales, 13 = d */
    struct unit { u32x4 xf[2][2]; u32 raw[KQ ? 1 : NP][2][3], wd[2], kq[2][Q6K ? 14 : 1]; u32x4 kh[2]; u32x2 kv[2][4]; };
    /* `o`: Q6_K only, where in its 16-byte-aligned window this chunk's super-block starts (even, wave-uniform) */
    auto fetch = [&](u32 xst, u32 rst, unit &t, u32 o) {
        const u32 xa0 = xst + xlane[0], xa1 = xst + xlane[1], rw = rst + rlane, rq = rst + qlane;
        t.xf[0][0] = lds_read128<0>(xa0);
        t.xf[0][1] = lds_read128<4096>(xa0);
        t.xf[1][0] = lds_read128<0>(xa1);
        t.xf[1][1] = lds_read128<4096>(xa1);
        if constexpr (Q6K) {
            /* every field starts o bytes into the record; o mod 4 is 0 or 2: aligned dwords are read and shifted in decode */
            const u32 ob = o & ~3u, ql = rq + ob, qh = rst + hlane + ob;
            const u32 sc = rw + (u32)(192 + 8 * (LOADER != 0)) + 2u * (u32)(wave & 3) + o, dd = rw + 208u + o;
            t.kq[0][0] = lds_read32o<0>(ql);
            t.kq[0][1] = lds_read32o<4>(ql);
            t.kq[0][2] = lds_read32o<8>(ql);
            t.kq[0][3] = lds_read32o<16>(ql);
            t.kq[0][4] = lds_read32o<20>(ql);
            t.kq[0][5] = lds_read32o<24>(ql);
            t.kq[1][0] = lds_read32o<ROW32>(ql);
            t.kq[1][1] = lds_read32o<ROW32 + 4>(ql);
            t.kq[1][2] = lds_read32o<ROW32 + 8>(ql);
            t.kq[1][3] = lds_read32o<ROW32 + 16>(ql);
            t.kq[1][4] = lds_read32o<ROW32 + 20>(ql);
            t.kq[1][5] = lds_read32o<ROW32 + 24>(ql);
            t.kq[0][6] = lds_read32o<0>(qh);
            t.kq[0][7] = lds_read32o<4>(qh);
            t.kq[0][8] = lds_read32o<8>(qh);
            t.kq[0][9] = lds_read32o<16>(qh);
            t.kq[0][10] = lds_read32o<20>(qh);
            t.kq[0][11] = lds_read32o<24>(qh);
            t.kq[1][6] = lds_read32o<ROW32>(qh);
            t.kq[1][7] = lds_read32o<ROW32 + 4>(qh);
            t.kq[1][8] = lds_read32o<ROW32 + 8>(qh);
            t.kq[1][9] = lds_read32o<ROW32 + 16>(qh);
            t.kq[1][10] = lds_read32o<ROW32 + 20>(qh);
            t.kq[1][11] = lds_read32o<ROW32 + 24>(qh);
            t.kq[0][12] = lds_read_u16(sc);
            t.kq[1][12] = lds_read_u16(sc + (u32)ROW32);
            t.kq[0][13] = lds_read_u16(dd);
            t.kq[1][13] = lds_read_u16(dd + (u32)ROW32);
        } else if constexpr (KQ) {
            /* a 32-bit read of 32 rows hits each LDS bank four times (rows are whole 16-byte words apart) and takes as long
             * as a conflict-free 128-bit one: the header word (d, dmin, scales) is read whole, the quants 64 bits at a time */
            const u32 rh = rst + hlane;
            t.kh[0] = lds_read128<0>(rw);
            t.kh[1] = lds_read128<ROW32>(rw);
            t.kv[0][0] = lds_read64o<0>(rq);
            t.kv[0][1] = lds_read64o<16>(rq);
            t.kv[1][0] = lds_read64o<ROW32>(rq);
            t.kv[1][1] = lds_read64o<ROW32 + 16>(rq);
            if constexpr (Q5K) {
                t.kv[0][2] = lds_read64o<0>(rh);
                t.kv[0][3] = lds_read64o<16>(rh);
                t.kv[1][2] = lds_read64o<ROW32>(rh);
                t.kv[1][3] = lds_read64o<ROW32 + 16>(rh);
            }
        } else if constexpr (EVEN) {
            t.wd[0] = lds_read32o<0>(rw);                                    /* scale | first two quant bytes */
            t.wd[1] = lds_read32o<ROW32>(rw);
            UNROLL for (int p = 0; p < NP; ++p) {
                t.raw[p][0][0] = p ? lds_read32o<16>(rq) : lds_read32o<0>(rq);
                t.raw[p][0][1] = p ? lds_read32o<20>(rq) : lds_read32o<4>(rq);
                t.raw[p][0][2] = p ? lds_read32o<24>(rq) : lds_read32o<8>(rq);
                t.raw[p][1][0] = p ? lds_read32o<ROW32 + 16>(rq) : lds_read32o<ROW32>(rq);
                t.raw[p][1][1] = p ? lds_read32o<ROW32 + 20>(rq) : lds_read32o<ROW32 + 4>(rq);
                t.raw[p][1][2] = p ? lds_read32o<ROW32 + 24>(rq) : lds_read32o<ROW32 + 8>(rq);
            }
        } else {
            t.wd[0] = lds_read32(rw - 2u);                                   /* last two bytes of the block before | scale */
            t.wd[1] = lds_read32(rw + (u32)(ROW32 - 2));
            UNROLL for (int p = 0; p < NP; ++p) {
                t.raw[p][0][0] = p ? lds_read32o<18>(rq) : lds_read32o<2>(rq);
                t.raw[p][0][1] = p ? lds_read32o<22>(rq) : lds_read32o<6>(rq);
                t.raw[p][0][2] = 0;
                t.raw[p][1][0] = p ? lds_read32o<ROW32 + 18>(rq) : lds_read32o<ROW32 + 2>(rq);
                t.raw[p][1][1] = p ? lds_read32o<ROW32 + 22>(rq) : lds_read32o<ROW32 + 6>(rq);
                t.raw[p][1][2] = 0;
            }
        }
    };
    auto arrived = [&](unit &t) {
        tie(t.xf[0]);
        tie(t.xf[1]);
        if constexpr (Q6K) {
            UNROLL for (int j = 0; j < 2; ++j) UNROLL for (int i = 0; i < 14; ++i) tie1(t.kq[j][i]);
        } else if constexpr (KQ) {
            tie(t.kh);
            UNROLL for (int j = 0; j < 2; ++j) UNROLL for (int i = 0; i < (Q5K ? 4 : 2); ++i) asm volatile("" : "+v"(t.kv[j][i]));
        } else UNROLL for (int j = 0; j < 2; ++j) {
            tie1(t.wd[j]);
            UNROLL for (int p = 0; p < NP; ++p) { tie1(t.raw[p][j][0]); tie1(t.raw[p][j][1]); if (EVEN) tie1(t.raw[p][j][2]); }
        }
    };
    /* MFMA operands of the block's two slices, column blocks j = 0, 1 */
    auto decode = [&](const unit &t, u32x4 (&wf)[2][2], u32 o) {
        if constexpr (Q6K) {
            const u32 sh = o & 2u;                          /* byte shift of every field against its aligned dwords */
            const int tq = wave & 3;
            UNROLL for (int j = 0; j < 2; ++j) {
                const float d = h2f_lo(t.kq[j][13]);
                UNROLL for (int sl = 0; sl < 2; ++sl) {
                    const float ds = __fmul_rn(d, (float)(int)(int8_t)((t.kq[j][12] >> (8 * sl)) & 0xffu)), dm = ds * 32.f;
                    u32 o4[4];
                    UNROLL for (int e = 0; e < 2; ++e) {
                        const u32 lo = __builtin_amdgcn_alignbyte(t.kq[j][3 * sl + e + 1], t.kq[j][3 * sl + e], sh);
                        const u32 hi = __builtin_amdgcn_alignbyte(t.kq[j][6 + 3 * sl + e + 1], t.kq[j][6 + 3 * sl + e], sh);
                        const u32 q = ((lo >> (4 * (tq >> 1))) & 0x0f0f0f0fu) | (((hi >> (2 * tq)) & 0x03030303u) << 4);
                        pf_affine4(q, ds, dm, o4[2 * e], o4[2 * e + 1]);
                    }
                    wf[sl][j] = (u32x4){o4[0], o4[1], o4[2], o4[3]};
                }
            }
        } else if constexpr (KQ) {
            const int sh = 8 * (wave & 3);                  /* this sub-block's byte of the scale dwords */
            UNROLL for (int j = 0; j < 2; ++j) {
                u32 sc, mn;
                if constexpr (LOADER == 0) {
                    sc = (t.kh[j][1] >> sh) & 63u;
                    mn = (t.kh[j][2] >> sh) & 63u;
                } else {
                    sc = ((t.kh[j][3] >> sh) & 0xfu) | (((t.kh[j][1] >> sh) >> 2) & 0x30u);
                    mn = ((t.kh[j][3] >> (sh + 4)) & 0xfu) | (((t.kh[j][2] >> sh) >> 2) & 0x30u);
                }
                const float d1 = __fmul_rn(h2f_lo(t.kh[j][0]), (float)sc), m1 = __fmul_rn(h2f_hi(t.kh[j][0]), (float)mn);
                UNROLL for (int sl = 0; sl < 2; ++sl) {
                    u32 o[4];
                    UNROLL for (int e = 0; e < 2; ++e) {
                        u32 q = (EVEN ? t.kv[j][sl][e] : t.kv[j][sl][e] >> 4) & 0x0f0f0f0fu;
                        if constexpr (Q5K) q |= ((t.kv[j][2 + sl][e] >> wave) & 0x01010101u) << 4;
                        pf_affine4(q, d1, m1, o[2 * e], o[2 * e + 1]);
                    }
                    wf[sl][j] = (u32x4){o[0], o[1], o[2], o[3]};
                }
            }
        } else UNROLL for (int j = 0; j < 2; ++j) {
            const half2_t w2 = bits_h2(t.wd[j]);
            const half2_t d2 = EVEN ? __builtin_shufflevector(w2, w2, 0, 0) : __builtin_shufflevector(w2, w2, 1, 1);
            u32 q[NP][2];
            UNROLL for (int p = 0; p < NP; ++p) {
                q[p][0] = EVEN ? align2(t.raw[p][j][1], t.raw[p][j][0]) : t.raw[p][j][0];
                q[p][1] = EVEN ? align2(t.raw[p][j][2], t.raw[p][j][1]) : t.raw[p][j][1];
            }
            UNROLL for (int sl = 0; sl < 2; ++sl) {
                u32 o[4];
                if constexpr (Q4) {
                    bytes_to_h4((sl ? q[0][0] >> 4 : q[0][0]) & 0x0f0f0f0fu, 0xffffffffu, bits_h2(0x64086408u), d2, o[0], o[1]);
                    bytes_to_h4((sl ? q[0][1] >> 4 : q[0][1]) & 0x0f0f0f0fu, 0xffffffffu, bits_h2(0x64086408u), d2, o[2], o[3]);
                } else {
                    bytes_to_h4(q[Q4 ? 0 : sl][0] ^ 0x80808080u, 0xffffffffu, bits_h2(0x64806480u), d2, o[0], o[1]);
                    bytes_to_h4(q[Q4 ? 0 : sl][1] ^ 0x80808080u, 0xffffffffu, bits_h2(0x64806480u), d2, o[2], o[3]);
                }
                wf[sl][j] = (u32x4){o[0], o[1], o[2], o[3]};
            }
        }
    };
    auto multiply = [&](const u32x4 (&xf)[2][2], const u32x4 (&wf)[2][2]) {
        UNROLL for (int sl = 0; sl < 2; ++sl) UNROLL for (int i = 0; i < 2; ++i) UNROLL for (int j = 0; j < 2; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, xf[sl][i]), __builtin_bit_cast(half8_t, wf[sl][j]), acc[i][j], 0, 0, 0);
    };

    for (int q = 0; q < DEPTH - 1; ++q) issue(q);
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"((DEPTH - 2) * PER) : "memory");   /* my share of chunk 0 has landed */
    lds_barrier();
    u32x4 xp[2][2], wp[2][2];                               /* LOADER != 0: the block decoded last */
    UNROLL for (int sl = 0; sl < 2; ++sl) UNROLL for (int i = 0; i < 2; ++i) xp[sl][i] = wp[sl][i] = (u32x4){0, 0, 0, 0};
    for (int q = 0; q < nq; ++q) {
        issue(q + DEPTH - 1);
        unit t;
        const u32 o = Q6K ? (u32)((chunk_of(q) * WF::BYTES) & 15) : 0u;
        fetch(xs_base + (u32)((q % XR) * XBYTES), raw_base + (u32)((q % RS) * RBYTES), t, o);
        if constexpr (LOADER == 0) {
            u32x4 wf[2][2];
            lds_wait();
            arrived(t);
            decode(t, wf, o);
            __builtin_amdgcn_sched_barrier(0);
            multiply(t.xf, wf);
        } else {
            multiply(xp, wp);
            __builtin_amdgcn_sched_barrier(0);
            lds_wait();
            arrived(t);
            decode(t, wp, o);
            UNROLL for (int sl = 0; sl < 2; ++sl) UNROLL for (int i = 0; i < 2; ++i) xp[sl][i] = t.xf[sl][i];
        }
        /* my share of chunk q+1: everything but the loads of the youngest DEPTH-2 iterations */
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"((DEPTH - 2) * PER) : "memory");
        lds_barrier();
    }
    if constexpr (LOADER != 0) multiply(xp, wp);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");        /* nothing lands in the rings any more ... */
    lds_barrier();                                          /* ... for any wave: they can hold the partial tiles */
}

template <typename WF>
PSN_DEV void prefill_skinny_body(const psn_prefill_args &a) {
    typedef SkinnyRings<WF> R;
    constexpr int BN = 64;
    extern __shared__ uint4 psn_smem[];
    typedef __attribute__((address_space(3))) char lds_char;
    lds_char *const lds_ptr = (lds_char *)psn_smem;
    const u32 lds0 = (u32)(uintptr_t)lds_ptr;
    const u32 xs_base = lds0, raw_base = xs_base + R::XR * R::XBYTES;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int M = a.M, N = a.N, C = a.K >> 8;
    const int nt = (N + BN - 1) / BN, S = a.ksplit;
    const int tile_n = blockIdx.x % nt, split = blockIdx.x / nt;
    const int per_split = (C + S - 1) / S;
    const int c_begin = split * per_split, c_end = min(c_begin + per_split, C);
    if (c_begin >= c_end) return;                           /* whole workgroup leaves together */
    const int n0 = tile_n * BN, nq = c_end - c_begin;
    /* Every workgroup walks the same X, so workgroups that started together would ask the same cache
     * lines of the same L2 channel at the same moment: each one starts its (cyclic) walk over the K
     * range at a different chunk.  The summation order of an output element depends only on its tile. */
    const int rot = (int)((blockIdx.x * 5u) % (unsigned)nq);

    float16_t acc[2][2];
    UNROLL for (int i = 0; i < 2; ++i) UNROLL for (int j = 0; j < 2; ++j) UNROLL for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
    /* the last tile's rows stay unrotated: the word that takes a rotated row's last bytes reaches up to twelve bytes
     * past the row, which for the matrix's last row is past the buffer */
    const bool rotate_rows = tile_n != nt - 1;
#define PSN_SKINNY_LOOP(LOADER, EVEN) prefill_skinny_loop<WF, LOADER, EVEN>(a, wave, lane, n0, c_begin, nq, rot, rotate_rows, xs_base, raw_base, lds_ptr, lds0, acc)
    if (wave < 4) {
        if ((wave & 1) == 0) PSN_SKINNY_LOOP(0, true);
        else PSN_SKINNY_LOOP(0, false);
    } else if (wave == 4) {
        PSN_SKINNY_LOOP(1, true);
    } else if ((wave & 1) == 0) {
        PSN_SKINNY_LOOP(2, true);
    } else {
        PSN_SKINNY_LOOP(2, false);
    }
#undef PSN_SKINNY_LOOP

    /* partial tiles of the eight waves -> LDS (16 KB each, lane-contiguous); then wave w sums registers
     * 8*(w/4) .. +8 of tile w%4 over the eight waves, always in the order 0 .. 7 */
    {
        const u32 base = lds0 + (u32)(wave * 16384 + lane * 4);
        UNROLL for (int i = 0; i < 2; ++i) UNROLL for (int j = 0; j < 2; ++j) UNROLL for (int r = 0; r < 16; ++r)
            lds_write32(base + (u32)(((i * 2 + j) * 16 + r) * 256), __float_as_uint(acc[i][j][r]));
    }
    lds_barrier();
    {
        const int t = wave & 3, i = t >> 1, j = t & 1, r0 = 8 * (wave >> 2);
        u32 v[8][8];
        UNROLL for (int w = 0; w < 8; ++w) UNROLL for (int r = 0; r < 8; ++r)
            v[w][r] = lds_read32(lds0 + (u32)(w * 16384 + (t * 16 + r0 + r) * 256 + lane * 4));
        lds_wait();
        UNROLL for (int w = 0; w < 8; ++w) UNROLL for (int r = 0; r < 8; ++r) tie1(v[w][r]);
        const int col = n0 + 32 * j + (lane & 31);
        UNROLL for (int r = 0; r < 8; ++r) {
            float sum = __uint_as_float(v[0][r]);
            UNROLL for (int w = 1; w < 8; ++w) sum += __uint_as_float(v[w][r]);
            const int rr = r0 + r, row = 32 * i + 8 * (rr >> 2) + 4 * (lane >> 5) + (rr & 3);
            if (row < M && col < N) {
                if (S == 1) a.Y[(int64_t)row * N + col] = sum;
                else unsafeAtomicAdd(&a.Y[(int64_t)row * N + col], sum);
            }
        }
    }
}

/* ---- wide variant (large M) --------------------------------------------------------------------------
 * The kernels above move more bytes through LDS per MFMA than the LDS pipe can serve at the MFMA rate
 * (fragment reads of 64 x 128 wave tiles plus the fp16 weight tile the producers write).  This one has
 * four waves, one per SIMD, each holding all 256 rows x 64 columns of the workgroup's tile of Y in 256
 * accumulator registers (a wave decodes only the two weight fragments of its own columns per K slice: no
 * decode is done twice), and no fp16 weight tile at all:
 *   - per 64 of K, X (256 rows, the swizzled tile layout of the other kernels) and the raw GGUF bytes of
 *     the workgroup's 256 weight rows (two blocks per row: 36 or 68 bytes, copied dword by dword) arrive
 *     by direct-to-LDS loads, in rings three stages deep: loads run two stages ahead and nobody spends
 *     VALU time on staging;
 *   - a wave decodes the eight weights per lane its own MFMA operand needs straight from the raw bytes
 *     (aligned dword reads, shifted into place), one 16-wide K slice ahead of the MFMAs that use them, and
 *     the decode instructions are interleaved with those MFMAs (measured on MI355X: an MFMA 32x32x16 keeps
 *     the matrix pipe for 32 cycles but the issue port for about 13, so three to four VALU instructions
 *     per MFMA ride along for free);
 *   - one workgroup barrier per 64 of K; every wave first waits for its own share of the next stage's
 *     loads (loads complete in issue order, so "at most n outstanding" identifies them). */
template <int N> struct pf_int { static constexpr int value = N; };

template <typename WF>
PSN_DEV void prefill_wide_body(const psn_prefill_args &a) {
    constexpr int BM = 256, BN = 256, TM = 8, TN = 2, NS = 3;     /* a wave: all 256 rows x 64 columns */
    constexpr bool Q4 = WF::DW == 36;
    constexpr int BB = WF::BYTES / 8;                       /* bytes of a GGUF block: 18 or 34 */
    constexpr int SB = 2 * BB;                              /* raw bytes per row and stage */
    constexpr int XBYTES = BM * 128, RBYTES = BN * SB;
    constexpr int NX = XBYTES / 1024 / 4;                   /* X loads per wave and stage: 8 */
    constexpr int NR = RBYTES / 4 / 64 / 4;                 /* raw dword loads per wave and stage: 9 or 17 */
    extern __shared__ uint4 psn_smem[];
    typedef __attribute__((address_space(3))) char lds_char;
    lds_char *const lds_ptr = (lds_char *)psn_smem;
    const u32 lds0 = (u32)(uintptr_t)lds_ptr;
    const int tid = threadIdx.x, lane = tid & 63, h = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wn = wave;
    const int M = a.M, N = a.N, K = a.K, C = K >> 8;

    const int mt = (M + BM - 1) / BM, nt = (N + BN - 1) / BN;
    const int S = a.ksplit;
    const int xcd = blockIdx.x & 7, local = blockIdx.x >> 3;
    const int per_xcd_n = (nt + 7) >> 3;
    const int tile_m = local % mt, split = (local / mt) % S, tn_local = local / (mt * S);
    const int tile_n = xcd + 8 * tn_local;
    if (tn_local >= per_xcd_n || tile_n >= nt) return;            /* whole workgroup leaves together */
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int per_split = (C + S - 1) / S;
    const int c_begin = split * per_split, c_end = min(c_begin + per_split, C);
    if (c_begin >= c_end) return;
    const int nsteps = (c_end - c_begin) * 4, g_base = c_begin * 4;

    float16_t acc[TM][TN];
    UNROLL for (int i = 0; i < TM; ++i) UNROLL for (int j = 0; j < TN; ++j) UNROLL for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    /* One stage = NX 16-byte words of X and NR dwords of raw weight bytes per thread, always at the same
     * per-thread byte offsets from a base that moves with the stage (scalar arithmetic only).  Stages past
     * the end of the K range repeat its last one (into ring slots nothing reads any more), so every step
     * issues the same number of loads. */
    u32 xoff_g[NX], woff_g[NR];
    UNROLL for (int u = 0; u < NX; ++u) {
        const int s_ = (wave * NX + u) * 64 + lane, row = s_ >> 3, chunk = (s_ & 7) ^ (row & 7);
        xoff_g[u] = (u32)min(m0 + row, M - 1) * (u32)(K * 2) + (u32)(chunk * 16);
    }
    UNROLL for (int u = 0; u < NR; ++u) {
        const int dw = (u * 4 + wave) * 64 + lane, row = dw / (SB / 4), off = dw % (SB / 4);
        woff_g[u] = (u32)min(n0 + row, N - 1) * (u32)a.row_bytes + (u32)(off * 4);
    }
    auto issue = [&](int g) {
        const int gg = g_base + min(g, nsteps - 1), slot = g % NS;
        const char *xb = reinterpret_cast<const char *>(a.X) + (int64_t)gg * 128;
        const char *wb = reinterpret_cast<const char *>(a.W) + (int64_t)gg * SB;
        lds_char *xd = lds_ptr + slot * XBYTES, *rd = lds_ptr + NS * XBYTES + slot * RBYTES;
        UNROLL for (int u = 0; u < NX; ++u)
            __builtin_amdgcn_global_load_lds((const void *)(xb + xoff_g[u]), (__attribute__((address_space(3))) void *)(xd + (wave * NX + u) * 1024), 16, 0, 0);
        UNROLL for (int u = 0; u < NR; ++u)
            __builtin_amdgcn_global_load_lds((const void *)(wb + woff_g[u]), (__attribute__((address_space(3))) void *)(rd + (u * 4 + wave) * 256), 4, 0, 0);
    };

    /* per-lane LDS offsets: the X fragment of K slice kk (row base + swizzled 16-byte position; the four
     * 32-row blocks of the wave's tile are 4096 bytes apart), the raw bytes of weight row block j */
    u32 xsw[4], rrow[TN];
    UNROLL for (int kk = 0; kk < 4; ++kk) xsw[kk] = (u32)((lane & 31) * 128) + ((((u32)(2 * kk + h)) ^ (u32)(lane & 7)) << 4);
    UNROLL for (int j = 0; j < TN; ++j) rrow[j] = (u32)((wn * 64 + 32 * j + (lane & 31)) * SB);
    const u32 hq = 8u * (u32)h;

    /* Raw unit U: Q4_0 -- block U of the stage (its 8 quant bytes 8h.. carry both nibble planes, K slices
     * 2U and 2U+1); Q8_0 -- K slice U (bytes 16*(U%2) + 8h.. of block U/2).  Blocks start on even bytes,
     * not on dwords, and LDS reads that straddle dwords are slow: a stage's first block starts on a dword
     * (scale in the low half, quants two bytes in: three dwords to shift), the second two bytes later. */
    auto read_unit = [&](u32 rst, auto uc, u32 (&raw)[TN][3], u32 (&wd)[TN]) {
        constexpr int U = decltype(uc)::value;
        constexpr int blk = Q4 ? U : U >> 1, qo = Q4 ? 0 : 16 * (U & 1);
        UNROLL for (int j = 0; j < TN; ++j) {
            const u32 rb = rst + rrow[j];
            if constexpr (blk == 0) {
                wd[j] = lds_read32o<0>(rb);
                raw[j][0] = lds_read32o<qo>(rb + hq);
                raw[j][1] = lds_read32o<qo + 4>(rb + hq);
                raw[j][2] = lds_read32o<qo + 8>(rb + hq);
            } else {
                wd[j] = lds_read32o<BB - 2>(rb);
                raw[j][0] = lds_read32o<BB + 2 + qo>(rb + hq);
                raw[j][1] = lds_read32o<BB + 6 + qo>(rb + hq);
                raw[j][2] = 0;
            }
        }
    };
    auto tie_unit = [&](u32 (&raw)[TN][3], u32 (&wd)[TN]) {
        UNROLL for (int j = 0; j < TN; ++j) { tie1(wd[j]); tie1(raw[j][0]); tie1(raw[j][1]); tie1(raw[j][2]); }
    };
    auto read_a = [&](u32 xst, int kk, u32x4 (&af)[TM]) {
        const u32 ab = xst + xsw[kk];
        af[0] = lds_read128<0>(ab);
        af[1] = lds_read128<4096>(ab);
        af[2] = lds_read128<8192>(ab);
        af[3] = lds_read128<12288>(ab);
        af[4] = lds_read128<16384>(ab);
        af[5] = lds_read128<20480>(ab);
        af[6] = lds_read128<24576>(ab);
        af[7] = lds_read128<28672>(ab);
    };
    /* One K slice: the 16 MFMAs of slice `cur` (fragments af, bf), every second one followed by four VALU
     * instructions of the decode of the NEXT slice's operand (K slice kn, out of its raw unit, into bn)
     * -- a quarter of a fragment: perm, and, subtract the bias, multiply by the scale -- with the
     * scheduler told not to move anything across the groups.  DEC false: the step's last slice, nothing left to decode. */
    auto slice = [&](auto kc, auto decc, const u32x4 (&af)[TM], const u32x4 (&bf)[TN], const u32 (&raw)[TN][3], const u32 (&wd)[TN], u32x4 (&bn)[TN]) {
        constexpr int kn = decltype(kc)::value;
        constexpr bool DEC = decltype(decc)::value != 0;
        UNROLL for (int j = 0; j < TN; ++j) {
            u32 q[2] = {0, 0};
            half2_t d2 = bits_h2(0);
            if constexpr (DEC) {
                u32 d;
                if constexpr ((kn & 2) == 0) {
                    q[0] = align2(raw[j][1], raw[j][0]);
                    q[1] = align2(raw[j][2], raw[j][1]);
                    d = wd[j] & 0xffffu;
                } else {
                    q[0] = raw[j][0];
                    q[1] = raw[j][1];
                    d = wd[j] >> 16;
                }
                d2 = bits_h2(d | (d << 16));
                if constexpr (Q4) {
                    if constexpr ((kn & 1) != 0) { q[0] >>= 4; q[1] >>= 4; }
                } else {
                    q[0] ^= 0x80808080u;
                    q[1] ^= 0x80808080u;
                }
            }
            u32 o[4];
            UNROLL for (int t = 0; t < 4; ++t) {
                acc[2 * t][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, af[2 * t]), __builtin_bit_cast(half8_t, bf[j]), acc[2 * t][j], 0, 0, 0);
                if constexpr (DEC) {
                    const u32 x = __builtin_amdgcn_perm(0x64646464u, q[t >> 1], (t & 1) ? 0x04030402u : 0x04010400u) & (Q4 ? 0x640f640fu : 0x64ff64ffu);
                    o[t] = h2_bits((bits_h2(x) - bits_h2(Q4 ? 0x64086408u : 0x64806480u)) * d2);
                }
                __builtin_amdgcn_sched_barrier(0);
                acc[2 * t + 1][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, af[2 * t + 1]), __builtin_bit_cast(half8_t, bf[j]), acc[2 * t + 1][j], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
            }
            if constexpr (DEC) bn[j] = (u32x4){o[0], o[1], o[2], o[3]};
        }
    };
    /* The step's last slice multiplies out of registers only, so it runs AFTER the step's barrier, while the
     * first reads of the next stage are on their way: eight MFMAs, then the wait for those reads, then the
     * other eight, each followed by a quarter of the decode of the next step's first operand (raw -> bn). */
    auto slice_last = [&](const u32x4 (&af)[TM], const u32x4 (&bf)[TN], const u32 (&raw)[TN][3], const u32 (&wd)[TN], u32x4 (&bn)[TN], auto &&arrive) {
        UNROLL for (int j = 0; j < TN; ++j) UNROLL for (int i = 0; i < 4; ++i) {
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, af[i]), __builtin_bit_cast(half8_t, bf[j]), acc[i][j], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
        arrive();
        UNROLL for (int j = 0; j < TN; ++j) {
            u32 q[2] = {align2(raw[j][1], raw[j][0]), align2(raw[j][2], raw[j][1])};
            const u32 d = wd[j] & 0xffffu;
            const half2_t d2 = bits_h2(d | (d << 16));
            if constexpr (!Q4) {
                q[0] ^= 0x80808080u;
                q[1] ^= 0x80808080u;
            }
            u32 o[4];
            UNROLL for (int t = 0; t < 4; ++t) {
                acc[4 + t][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, af[4 + t]), __builtin_bit_cast(half8_t, bf[j]), acc[4 + t][j], 0, 0, 0);
                const u32 x = __builtin_amdgcn_perm(0x64646464u, q[t >> 1], (t & 1) ? 0x04030402u : 0x04010400u) & (Q4 ? 0x640f640fu : 0x64ff64ffu);
                o[t] = h2_bits((bits_h2(x) - bits_h2(Q4 ? 0x64086408u : 0x64806480u)) * d2);
                __builtin_amdgcn_sched_barrier(0);
            }
            bn[j] = (u32x4){o[0], o[1], o[2], o[3]};
        }
    };

    /* Steady state at the top of step g: stage g's first raw unit(s) and first two X fragments sit in
     * registers, the operand of its first slice is decoded; stages g+1 and g+2 are on their way. */
    constexpr int RU = Q4 ? 2 : 3;                            /* raw register sets */
    u32x4 af[4][TM], bf[2][TN];
    u32 raw[RU][TN][3], wd[RU][TN];
    issue(0);
    issue(1);
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NX + NR) : "memory");       /* my share of stage 0 */
    lds_barrier();
    issue(2);
    {
        const u32 xst = lds0, rst = lds0 + (u32)(NS * XBYTES);
        read_unit(rst, pf_int<0>(), raw[0], wd[0]);
        if constexpr (!Q4) read_unit(rst, pf_int<1>(), raw[1], wd[1]);
        read_a(xst, 0, af[0]);
        read_a(xst, 1, af[1]);
        lds_wait();
        tie_unit(raw[0], wd[0]);
        if constexpr (!Q4) tie_unit(raw[1], wd[1]);
        tie(af[0]);
        tie(af[1]);
        UNROLL for (int j = 0; j < TN; ++j) {
            const u32 q0 = align2(raw[0][j][1], raw[0][j][0]), q1 = align2(raw[0][j][2], raw[0][j][1]), d = wd[0][j] & 0xffffu;
            const half2_t d2 = bits_h2(d | (d << 16));
            u32 o[4];
            if constexpr (Q4) {
                bytes_to_h4(q0, 0x640f640fu, bits_h2(0x64086408u), d2, o[0], o[1]);
                bytes_to_h4(q1, 0x640f640fu, bits_h2(0x64086408u), d2, o[2], o[3]);
            } else {
                bytes_to_h4(q0 ^ 0x80808080u, 0x64ff64ffu, bits_h2(0x64806480u), d2, o[0], o[1]);
                bytes_to_h4(q1 ^ 0x80808080u, 0x64ff64ffu, bits_h2(0x64806480u), d2, o[2], o[3]);
            }
            bf[0][j] = (u32x4){o[0], o[1], o[2], o[3]};
        }
    }
    for (int g = 0; g < nsteps; ++g) {
        const int slot = g % NS, nslot = (g + 1) % NS;
        const u32 xst = lds0 + (u32)(slot * XBYTES), rst = lds0 + (u32)(NS * XBYTES + slot * RBYTES);
        const u32 xsn = lds0 + (u32)(nslot * XBYTES), rsn = lds0 + (u32)(NS * XBYTES + nslot * RBYTES);
        if constexpr (Q4) {
            /* slice 0 multiplies, slice 1 (the other nibble plane of block 0) is decoded; block 1 and X of slice 2 arrive */
            read_unit(rst, pf_int<1>(), raw[1], wd[1]);
            read_a(xst, 2, af[2]);
            slice(pf_int<1>(), pf_int<1>(), af[0], bf[0], raw[0], wd[0], bf[1]);
            lds_wait();
            tie_unit(raw[1], wd[1]);
            tie(af[2]);
            read_a(xst, 3, af[3]);
            slice(pf_int<2>(), pf_int<1>(), af[1], bf[1], raw[1], wd[1], bf[0]);
            lds_wait();
            tie(af[3]);
            slice(pf_int<3>(), pf_int<1>(), af[2], bf[0], raw[1], wd[1], bf[1]);
        } else {
            read_unit(rst, pf_int<2>(), raw[2], wd[2]);
            read_a(xst, 2, af[2]);
            slice(pf_int<1>(), pf_int<1>(), af[0], bf[0], raw[1], wd[1], bf[1]);
            lds_wait();
            tie_unit(raw[2], wd[2]);
            tie(af[2]);
            read_unit(rst, pf_int<3>(), raw[1], wd[1]);
            read_a(xst, 3, af[3]);
            slice(pf_int<2>(), pf_int<1>(), af[1], bf[1], raw[2], wd[2], bf[0]);
            lds_wait();
            tie_unit(raw[1], wd[1]);
            tie(af[3]);
            slice(pf_int<3>(), pf_int<1>(), af[2], bf[0], raw[1], wd[1], bf[1]);
        }
        /* my share of stage g+1 (stage g+2 may still be on its way); then nobody reads stage g any more */
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NX + NR) : "memory");
        lds_barrier();
        issue(g + 3);
        read_unit(rsn, pf_int<0>(), raw[0], wd[0]);
        if constexpr (!Q4) read_unit(rsn, pf_int<1>(), raw[1], wd[1]);
        read_a(xsn, 0, af[0]);
        read_a(xsn, 1, af[1]);
        slice_last(af[3], bf[1], raw[0], wd[0], bf[0], [&]() {
            lds_wait();
            tie_unit(raw[0], wd[0]);
            if constexpr (!Q4) tie_unit(raw[1], wd[1]);
            tie(af[0]);
            tie(af[1]);
        });
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

    int tid_out = threadIdx.x;
    asm volatile("" : "+v"(tid_out));
    const int wn_o = tid_out >> 6, lane_o = tid_out & 63;
    const bool whole = m0 + BM <= M && n0 + BN <= N;              /* uniform: no element of the tile needs a bounds check */
    UNROLL for (int i = 0; i < TM; ++i) UNROLL for (int j = 0; j < TN; ++j) {
        const int col = n0 + wn_o * 64 + 32 * j + (lane_o & 31);
        float *yc = a.Y + (int64_t)(m0 + 32 * i + 4 * (lane_o >> 5)) * N + col;
        UNROLL for (int r = 0; r < 16; ++r) {
            const int dr = 8 * (r >> 2) + (r & 3);
            if (whole || (m0 + 32 * i + 4 * (lane_o >> 5) + dr < M && col < N)) {
                if (S == 1) yc[(int64_t)dr * N] = acc[i][j][r];
                else unsafeAtomicAdd(&yc[(int64_t)dr * N], acc[i][j][r]);
            }
        }
    }
}

/* ------------------------------------------------------------------------------------------
 * Dense family: dequantize once, multiply as plain fp16.
 *
 * A workgroup of any other family dequantizes its weight tile again for every M tile that needs it; from
 * a few thousand rows of X on (and from 2048 for the K-quants, whose dequantization is fp32 arithmetic per
 * weight) it is cheaper to turn the whole matrix into fp16 once per call and run a matmul with no decode
 * in its loop.  psn_prefill_<fmt>_unpack writes h(deq(W)) -- the same fp16 values every other family
 * feeds the MFMA -- in the order the multiply kernel consumes them: fragment (32-row block nb, 16-wide K
 * slice ks) is 1 KB, lane (h = lane >> 5, n = lane & 31) holding W[32 nb + n][16 ks + 8 h .. + 7], i.e.
 * exactly one B operand of v_mfma_f32_32x32x16_f16.  psn_prefill_dense_f16 (256 x 256 tile, four waves,
 * each all 256 rows x 64 columns as in the wide kernel) and psn_prefill_dense_f16_m128 (128 x 256 tile: half the
 * rows and accumulators per wave, twice the workgroups -- shapes whose 256-row tiles leave compute units idle or
 * end on a mostly empty round) then fetch their weight fragments with plain
 * 16-byte loads straight into registers, four 32-wide K stages ahead, so that LDS carries only X: a
 * stage of X is 256 (128) rows of 64 bytes, the four 16-byte pieces of a row stored at piece ^ ((row >> 2) & 3)
 * (conflict-free fragment reads), filled by direct-to-LDS loads into a ring of four slots; one barrier
 * per stage, placed between the stage's two K slices so that both batches of fragment reads hide under
 * sixteen MFMAs.
 * ------------------------------------------------------------------------------------------ */
template <typename WF>
PSN_DEV void prefill_unpack_body(const psn_unpack_args &a) {
    const int C = a.K >> 8, KF = a.K >> 4;
    const int rb = (int)(blockIdx.x / (unsigned)C), chunk = (int)(blockIdx.x % (unsigned)C);
    const int row = rb * 256 + (int)threadIdx.x;
    if (row >= a.N) return;                                   /* rows of the last 256-row panel past N stay unwritten: their columns are never stored */
    u32 w[WF::DW];
    WF::load(a.W + (int64_t)row * a.row_bytes + (int64_t)chunk * WF::BYTES, w);
    uint4 *frag = reinterpret_cast<uint4 *>(a.out) + ((int64_t)(row >> 5) * KF + chunk * 16) * 64 + (row & 31);
    auto put = [&](auto bc) {
        constexpr int B = decltype(bc)::value;
        u32 o[16];
        WF::template deq_block<B>(w, o);
        UNROLL for (int i = 0; i < 4; ++i)                    /* elements 8 i .. 8 i + 7 of the sub-block: K slice 2 B + (i >> 1), half i & 1 */
            frag[(2 * B + (i >> 1)) * 64 + (i & 1) * 32] = make_uint4(o[4 * i], o[4 * i + 1], o[4 * i + 2], o[4 * i + 3]);
    };
    put(pf_int<0>()); put(pf_int<1>()); put(pf_int<2>()); put(pf_int<3>());
    put(pf_int<4>()); put(pf_int<5>()); put(pf_int<6>()); put(pf_int<7>());
}

template <int TM> PSN_DEV void prefill_dense_body(const psn_prefill_args &a) {
    static_assert(TM == 4 || TM == 8, "128 or 256 rows of X per workgroup");
    constexpr int BM = 32 * TM, BN = 256, TN = 2, NS = 4;
    constexpr int KS = 32;                                   /* k per stage */
    constexpr int XB = BM * KS * 2;                          /* bytes of X per stage: 8 or 16 KB */
    constexpr int XL = XB / 4096;                            /* X loads per wave and stage: 2 or 4 */
    constexpr int NL = XL + 2 * TN;                          /* loads per wave and stage: those of X and 4 of W */
    extern __shared__ uint4 psn_smem[];
    typedef __attribute__((address_space(3))) char lds_char;
    lds_char *const lds_ptr = (lds_char *)psn_smem;
    const u32 lds0 = (u32)(uintptr_t)lds_ptr;
    const int tid = threadIdx.x, lane = tid & 63, h = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int M = a.M, N = a.N, K = a.K, C = K >> 8;
    const int mt = (M + BM - 1) / BM, nt = (N + BN - 1) / BN;
    const int S = a.ksplit;
    const int xcd = blockIdx.x & 7, local = blockIdx.x >> 3;
    const int per_xcd_n = (nt + 7) >> 3;
    const int tile_m = local % mt, split = (local / mt) % S, tn_local = local / (mt * S);
    const int tile_n = xcd + 8 * tn_local;
    if (tn_local >= per_xcd_n || tile_n >= nt) return;            /* whole workgroup leaves together */
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int per_split = (C + S - 1) / S;
    const int c_begin = split * per_split, c_end = min(c_begin + per_split, C);
    if (c_begin >= c_end) return;
    const int nsteps = (c_end - c_begin) * (256 / KS), g_base = c_begin * (256 / KS);   /* a multiple of NS */

    float16_t acc[TM][TN];
    UNROLL for (int i = 0; i < TM; ++i) UNROLL for (int j = 0; j < TN; ++j) UNROLL for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    /* X: load instruction u of wave w fills LDS bytes [(XL w + u) * 1024, + 1024) of the stage's slot; the
     * lane picks the global piece that belongs at its LDS position.  Stages past the end of the K range
     * repeat its last one (into slots nothing reads any more), so every stage issues the same loads. */
    u32 xoff_g[XL];
    UNROLL for (int u = 0; u < XL; ++u) {
        const int s_ = (wave * XL + u) * 64 + lane, row = s_ >> 2, piece = (s_ & 3) ^ ((row >> 2) & 3);
        xoff_g[u] = (u32)min(m0 + row, M - 1) * (u32)(K * 2) + (u32)(piece * 16);
    }
    const int KF = K >> 4;                                   /* fragments per 32-row block */
    const char *wfrag = reinterpret_cast<const char *>(a.W) + ((int64_t)((n0 >> 5) + wave * 2) * KF) * 1024 + lane * 16;
    const int64_t wjump = (int64_t)KF * 1024;                /* the wave's second 32-row block */
    u32x4 bq[NS][2][TN];
    auto issue_x = [&](int g) {
        const int gg = g_base + min(g, nsteps - 1), slot = g % NS;
        const char *xb = reinterpret_cast<const char *>(a.X) + (int64_t)gg * (KS * 2);
        lds_char *xd = lds_ptr + slot * XB;
        UNROLL for (int u = 0; u < XL; ++u)
            __builtin_amdgcn_global_load_lds((const void *)(xb + xoff_g[u]), (__attribute__((address_space(3))) void *)(xd + (wave * XL + u) * 1024), 16, 0, 0);
    };
    auto issue_b = [&](int g, u32x4 (&dst)[2][TN]) {
        const int gg = g_base + min(g, nsteps - 1);
        const char *p = wfrag + (int64_t)gg * 2048;
        UNROLL for (int kk = 0; kk < 2; ++kk) UNROLL for (int j = 0; j < TN; ++j) dst[kk][j] = global_read128(p + kk * 1024 + j * wjump);
    };
    u32 fsw[2];                                              /* per-lane offset of the fragment of K slice kk inside a 32-row block of X */
    UNROLL for (int kk = 0; kk < 2; ++kk) fsw[kk] = (u32)((lane & 31) * 64) + ((((u32)(2 * kk + h)) ^ (u32)((lane >> 2) & 3)) << 4);
    auto read_a = [&](u32 st, int kk, u32x4 (&af)[TM]) {
        const u32 ab = st + fsw[kk];
        af[0] = lds_read128<0>(ab);
        af[1] = lds_read128<2048>(ab);
        af[2] = lds_read128<4096>(ab);
        af[3] = lds_read128<6144>(ab);
        if constexpr (TM == 8) {
            af[4] = lds_read128<8192>(ab);
            af[5] = lds_read128<10240>(ab);
            af[6] = lds_read128<12288>(ab);
            af[7] = lds_read128<14336>(ab);
        }
    };
    auto mfmas = [&](const u32x4 (&af)[TM], const u32x4 (&bf)[TN]) {
        UNROLL for (int j = 0; j < TN; ++j) UNROLL for (int i = 0; i < TM; ++i)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, af[i]), __builtin_bit_cast(half8_t, bf[j]), acc[i][j], 0, 0, 0);
    };
    u32x4 a0[TM], a1[TM];
    UNROLL for (int s = 0; s < NS; ++s) { issue_x(s); issue_b(s, bq[s]); }
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"((NS - 1) * NL) : "memory");        /* my share of stage 0 */
    lds_barrier();
    read_a(lds0, 0, a0);
    lds_wait();
    tie(a0);
    for (int g = 0; g < nsteps; g += NS) {
        UNROLL for (int s = 0; s < NS; ++s) {
            const u32 st = lds0 + (u32)(s * XB), sn = lds0 + (u32)(((s + 1) % NS) * XB);
            read_a(st, 1, a1);
            mfmas(a0, bq[s][0]);
            /* stage g + s + 1 has landed (the two after it may still be on their way); my reads of this stage are done */
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"((NS - 2) * NL) : "memory");
            lds_barrier();
            tie(a1);
            tie(bq[s][1]);
            issue_x(g + s + NS);                             /* into this stage's slot: nobody reads it any more */
            read_a(sn, 0, a0);
            mfmas(a1, bq[s][1]);
            issue_b(g + s + NS, bq[s]);                      /* both of the stage's fragment sets have been multiplied */
            lds_wait();
            tie(a0);
            tie(bq[(s + 1) % NS][0]);
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

    int tid_out = threadIdx.x;
    asm volatile("" : "+v"(tid_out));
    const int wn_o = tid_out >> 6, lane_o = tid_out & 63;
    const bool whole = m0 + BM <= M && n0 + BN <= N;              /* uniform: no element of the tile needs a bounds check */
    UNROLL for (int i = 0; i < TM; ++i) UNROLL for (int j = 0; j < TN; ++j) {
        const int col = n0 + wn_o * 64 + 32 * j + (lane_o & 31);
        float *yc = a.Y + (int64_t)(m0 + 32 * i + 4 * (lane_o >> 5)) * N + col;
        UNROLL for (int r = 0; r < 16; ++r) {
            const int dr = 8 * (r >> 2) + (r & 3);
            if (whole || (m0 + 32 * i + 4 * (lane_o >> 5) + dr < M && col < N)) {
                if (S == 1) yc[(int64_t)dr * N] = acc[i][j][r];
                else unsafeAtomicAdd(&yc[(int64_t)dr * N], acc[i][j][r]);
            }
        }
    }
}

#define PSN_PREFILL_KERNEL_WIDE(fmt, WF)                                                                     \
    extern "C" __global__ void __launch_bounds__(256) psn_prefill_##fmt##_wide(const psn_prefill_args a) {   \
        prefill_wide_body<WF>(a);                                                                            \
    }

#define PSN_PREFILL_KERNEL_SKINNY(fmt, WF)                                                                   \
    extern "C" __global__ void __launch_bounds__(512) psn_prefill_##fmt##_skinny(const psn_prefill_args a) { \
        prefill_skinny_body<WF>(a);                                                                          \
    }

#define PSN_PREFILL_KERNEL(fmt, WF, BM, BN, WM, WN)                                                          \
    extern "C" __global__ void __launch_bounds__(256) psn_prefill_##fmt##_m##BM##_n##BN(const psn_prefill_args a) { \
        prefill_body<WF, BM, BN, WM, WN>(a);                                                                 \
    }


#define PSN_PREFILL_KERNEL_WS(fmt, WF, BM, BN)                                                               \
    extern "C" __global__ void __launch_bounds__(512) psn_prefill_##fmt##_m##BM##_n##BN##_ws(const psn_prefill_args a) { \
        prefill_body_ws<WF, BM, BN>(a);                                                                      \
    }


#define PSN_PREFILL_FAMILY_WS(fmt, WF)           \
    PSN_PREFILL_KERNEL_WS(fmt, WF, 64, 64)       \
    PSN_PREFILL_KERNEL_WS(fmt, WF, 64, 128)      \
    PSN_PREFILL_KERNEL_WS(fmt, WF, 128, 128)     \
    PSN_PREFILL_KERNEL_WS(fmt, WF, 128, 256)
#define PSN_PREFILL_FAMILY_BASE(fmt, WF)         \
    PSN_PREFILL_KERNEL(fmt, WF, 64, 64, 2, 2)    \
    PSN_PREFILL_KERNEL(fmt, WF, 64, 128, 2, 2)   \
    PSN_PREFILL_KERNEL(fmt, WF, 128, 128, 2, 2)  \
    PSN_PREFILL_KERNEL(fmt, WF, 128, 256, 2, 2)  \
    PSN_PREFILL_KERNEL(fmt, WF, 256, 128, 2, 2)  \
    PSN_PREFILL_KERNEL(fmt, WF, 256, 256, 2, 2)

/* The build compiles this file once per (format, kernel family) -- -DPSN_BUILD_ONLY -DPSN_BUILD_PF=<n>
 * -DPSN_BUILD_PF_Q4_0 or _Q8_0 -- so that the code objects build in parallel; without PSN_BUILD_ONLY
 * everything lands in one.  Family numbers: 0 skinny + fill, 1 ws (producer / consumer), 2 wide, 4 base (four waves),
 * 5 dense (unpack kernels of all formats + the fp16 multiply). */

#if !defined(PSN_BUILD_ONLY) || PSN_BUILD_PF == 0
/* zero fill with plain vector stores (graph-safe stand-in for a memset node) */
extern "C" __global__ void __launch_bounds__(256) psn_fill_zero(const psn_fill_args a) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    uint4 *p = reinterpret_cast<uint4 *>(a.p);
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < a.n16; i += stride) p[i] = make_uint4(0, 0, 0, 0);
}
PSN_PREFILL_KERNEL_SKINNY(q4_0, PfQ4_0)
PSN_PREFILL_KERNEL_SKINNY(q8_0, PfQ8_0)
PSN_PREFILL_KERNEL_SKINNY(q4_K, PfQ4_K)
PSN_PREFILL_KERNEL_SKINNY(q5_K, PfQ5_K)
PSN_PREFILL_KERNEL_SKINNY(q6_K, PfQ6_K)
#endif
#if !defined(PSN_BUILD_ONLY) || PSN_BUILD_PF == 2
PSN_PREFILL_KERNEL_WIDE(q4_0, PfQ4_0)
PSN_PREFILL_KERNEL_WIDE(q8_0, PfQ8_0)
#endif
#if !defined(PSN_BUILD_ONLY) || defined(PSN_BUILD_PF_Q4_0)
#if !defined(PSN_BUILD_ONLY) || PSN_BUILD_PF == 1
PSN_PREFILL_FAMILY_WS(q4_0, PfQ4_0)
#endif
#if !defined(PSN_BUILD_ONLY) || PSN_BUILD_PF == 4
PSN_PREFILL_FAMILY_BASE(q4_0, PfQ4_0)
#endif
#endif
#if !defined(PSN_BUILD_ONLY) || defined(PSN_BUILD_PF_Q8_0)
#if !defined(PSN_BUILD_ONLY) || PSN_BUILD_PF == 1
PSN_PREFILL_FAMILY_WS(q8_0, PfQ8_0)
#endif
#if !defined(PSN_BUILD_ONLY) || PSN_BUILD_PF == 4
PSN_PREFILL_FAMILY_BASE(q8_0, PfQ8_0)
#endif
#endif
#if !defined(PSN_BUILD_ONLY) || PSN_BUILD_PF == 5
extern "C" __global__ void __launch_bounds__(256) psn_prefill_dense_f16(const psn_prefill_args a) { prefill_dense_body<8>(a); }
extern "C" __global__ void __launch_bounds__(256) psn_prefill_dense_f16_m128(const psn_prefill_args a) { prefill_dense_body<4>(a); }
#define PSN_PREFILL_KERNEL_UNPACK(fmt, WF) \
    extern "C" __global__ void __launch_bounds__(256) psn_prefill_##fmt##_unpack(const psn_unpack_args a) { prefill_unpack_body<WF>(a); }
PSN_PREFILL_KERNEL_UNPACK(q4_0, PfQ4_0)
PSN_PREFILL_KERNEL_UNPACK(q8_0, PfQ8_0)
PSN_PREFILL_KERNEL_UNPACK(q4_K, PfQ4_K)
PSN_PREFILL_KERNEL_UNPACK(q5_K, PfQ5_K)
PSN_PREFILL_KERNEL_UNPACK(q6_K, PfQ6_K)
#endif
/* K-quants: the four-wave family, and for Q4_K / Q5_K the 128 x 256 producer / consumer kernel
 * (-DPSN_BUILD_PF=4 -DPSN_BUILD_PF_Q4_K / _Q5_K / _Q6_K) */
#if !defined(PSN_BUILD_ONLY) || (defined(PSN_BUILD_PF_Q4_K) && PSN_BUILD_PF == 4)
PSN_PREFILL_FAMILY_BASE(q4_K, PfQ4_K)
PSN_PREFILL_KERNEL_WS(q4_K, PfQ4_K, 128, 256)
#endif
#if !defined(PSN_BUILD_ONLY) || (defined(PSN_BUILD_PF_Q5_K) && PSN_BUILD_PF == 4)
PSN_PREFILL_FAMILY_BASE(q5_K, PfQ5_K)
PSN_PREFILL_KERNEL_WS(q5_K, PfQ5_K, 128, 256)
#endif
#if !defined(PSN_BUILD_ONLY) || (defined(PSN_BUILD_PF_Q6_K) && PSN_BUILD_PF == 4)
PSN_PREFILL_FAMILY_BASE(q6_K, PfQ6_K)
#endif
