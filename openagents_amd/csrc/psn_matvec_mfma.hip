/*
 * psn_matvec_mfma.hip -- small-batch (2..8 columns) decode matvec for the K-quant formats whose
 * sub-blocks carry integer scales (Q4_K, Q5_K), scheme Q8 (Q8_K activations).
 *
 * At batch 1 a lane multiplies one 256-weight chunk against the one activation vector with
 * v_dot4_i32_i8.  With several columns the integer dot products are a skinny matrix product, and
 * v_mfma_i32_16x16x32_i8 does one 32-element sub-block of 16 matrix rows against up to 16 columns in
 * a single instruction: A = the columns' int8 activations (m = column), B = the rows' unpacked
 * quants (n = row), D[m][n] = the sub-block's integer dot product -- bit for bit what the dot4 path
 * computes.  A lane then holds four columns of ONE matrix row (n = lane & 15), so the row's 6-bit
 * sub-block scales are unpacked once per lane and applied with v_mad_i32_i24; the min term
 * sum_j mn[j] * bsum[j] is two more MFMAs over the eight sub-blocks (bsums split into a 6-bit low
 * part and a signed high part so that both fit int8).  The cost per weight does not depend on the
 * batch, so the launch stays a weight stream.
 *
 * Work unit: 16 rows x SL chunks (a "slice", SL <= 8).  A workgroup of 8 (or 4) waves holds
 * waves/KS row tiles at a time, the KS waves of a tile each own one K slice of it and never change
 * slice: their columns' activations (256 int8 per chunk and column, fetched 256 contiguous bytes at a
 * time and regrouped into MFMA operands through LDS) are read once per wave.  Partial sums of the KS
 * waves meet in LDS.
 *
 * The weights arrive by 16-byte direct-to-LDS loads, one buffer per wave, requested one chunk ahead of
 * the arithmetic (a compute unit's memory path accepts a bounded number of bytes and stalls the issuing
 * wave, so a wave that requests its whole unit up front multiplies nothing meanwhile).  A load
 * instruction fetches four consecutive 16-byte words (64 contiguous bytes) of each of the 16 rows; word t
 * of row r lands at
 *     (t >> 2) * 1024 + (4 r + ((t ^ (r >> 2)) & 3)) * 16
 * so that the 16 rows of one word sit in 16 different 16-byte columns of the LDS banks (the reads
 * below are conflict-free) while the four lanes of a row still fetch one contiguous 64 bytes.
 * Every wait is placed by hand (see psn_device.h).
 */
#include "psn_args.h"
#include "psn_device.h"

#define UNROLL _Pragma("unroll")

typedef int v4i __attribute__((ext_vector_type(4)));
typedef unsigned long long u64;

template <int OFF> PSN_DEV u64 lds_read64(u32 addr) {
    u64 v;
    asm volatile("ds_read_b64 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF) : "memory");
    return v;
}
PSN_DEV u64 global_read64(const void *p) {
    u64 v;
    asm volatile("global_load_dwordx2 %0, %1, off" : "=v"(v) : "v"(p) : "memory");
    return v;
}
PSN_DEV u32 global_read32(const void *p) {
    u32 v;
    asm volatile("global_load_dword %0, %1, off" : "=v"(v) : "v"(p) : "memory");
    return v;
}
PSN_DEV void lds_write64(u32 addr, u64 v) { asm volatile("ds_write_b64 %0, %1" ::"v"(addr), "v"(v) : "memory"); }
PSN_DEV void tie64(u64 &v) { asm volatile("" : "+v"(v)); }
PSN_DEV u64 pack64(u32 lo, u32 hi) { return ((u64)hi << 32) | lo; }
PSN_DEV v4i mfma_i8(u64 a, u64 b) {
    return __builtin_amdgcn_mfma_i32_16x16x32_i8((long)a, (long)b, (v4i)(0), 0, 0, 0);
}

/* Q4_K: 9 words per super-block: word 0 = d | dmin | 12 scale bytes, words 1..8 = nibbles.
 * Q5_K: 11 words: word 0 the same, words 1..2 = qh, words 3..10 = nibbles. */
struct MfQ4_K { static constexpr int WORDS = 9, NIB0 = 1; static constexpr bool HIGH = false; };
struct MfQ5_K { static constexpr int WORDS = 11, NIB0 = 3; static constexpr bool HIGH = true; };

PSN_DEV void kq_scales(u32 s0, u32 s1, u32 s2, u32 (&sc)[2], u32 (&mn)[2]) {
    sc[0] = s0 & 0x3f3f3f3fu;
    mn[0] = s1 & 0x3f3f3f3fu;
    sc[1] = (s2 & 0x0f0f0f0fu) | ((s0 >> 2) & 0x30303030u);
    mn[1] = ((s2 >> 4) & 0x0f0f0f0fu) | ((s1 >> 2) & 0x30303030u);
}

/* per-lane read addresses into the wave's buffer: index k = (word index of the access) & 3 */
struct LaneOffs {
    u32 hdr[4];   /* 16-byte read of word t (t & 3 == k) of row n */
    u32 w[4];     /* 8-byte read: word t + (kq >> 1), half kq & 1 */
};

template <typename F, int CI>
PSN_DEV void mf_chunk(const LaneOffs &o, u32 xs_addr, u32 dx_addr, const u64 (&x)[8], bool first_quarter, float (&acc)[4]) {
    constexpr int T0 = F::WORDS * (CI & 3);                 /* first word of the chunk in the wave's buffer, a ring of four chunks */
    const u32x4 hdr = lds_read128<(T0 >> 2) * 1024>(o.hdr[T0 & 3]);
    u64 wq[4];
    constexpr int TA = T0 + F::NIB0, TB = TA + 2, TC = TA + 4, TD = TA + 6;
    wq[0] = lds_read64<(TA >> 2) * 1024>(o.w[TA & 3]);
    wq[1] = lds_read64<(TB >> 2) * 1024>(o.w[TB & 3]);
    wq[2] = lds_read64<(TC >> 2) * 1024>(o.w[TC & 3]);
    wq[3] = lds_read64<(TD >> 2) * 1024>(o.w[TD & 3]);
    u64 qh = 0;
    if constexpr (F::HIGH) {
        constexpr int TH = T0 + 1;
        qh = lds_read64<(TH >> 2) * 1024>(o.w[TH & 3]);
    }
    u32x4 xsv = lds_read128<CI * 128>(xs_addr);             /* the column's eight sub-block sums, low and high parts */
    u32x4 dxv = lds_read128<CI * 32>(dx_addr);              /* activation scales of this lane's four columns */
    lds_wait();
    u32x4 h = hdr;
    asm volatile("" : "+v"(h), "+v"(xsv), "+v"(dxv));
    UNROLL for (int g = 0; g < 4; ++g) tie64(wq[g]);
    if constexpr (F::HIGH) tie64(qh);

    u32 sc[2], mn[2];
    kq_scales(h.y, h.z, h.w, sc, mn);
    /* min term: only the lanes of the first k quarter carry B values (k = sub-block index 0..7) */
    const u64 bm = first_quarter ? pack64(mn[0], mn[1]) : 0ull;
    const v4i mlo = mfma_i8(pack64(xsv.x, xsv.y), bm);
    const v4i mhi = mfma_i8(pack64(xsv.z, xsv.w), bm);
    int isum[4] = {0, 0, 0, 0};
    UNROLL for (int g = 0; g < 4; ++g) {
        const u32 w0 = (u32)wq[g], w1 = (u32)(wq[g] >> 32);
        u32 l0 = w0 & 0x0f0f0f0fu, l1 = w1 & 0x0f0f0f0fu;
        u32 h0 = (w0 >> 4) & 0x0f0f0f0fu, h1 = (w1 >> 4) & 0x0f0f0f0fu;
        if constexpr (F::HIGH) {
            /* bit j of qh byte l is the fifth bit of element l of sub-block j */
            const u32 q0 = (u32)qh, q1 = (u32)(qh >> 32);
            l0 |= ((q0 >> (2 * g)) & 0x01010101u) << 4;
            l1 |= ((q1 >> (2 * g)) & 0x01010101u) << 4;
            h0 |= ((q0 >> (2 * g + 1)) & 0x01010101u) << 4;
            h1 |= ((q1 >> (2 * g + 1)) & 0x01010101u) << 4;
        }
        const v4i dl = mfma_i8(x[2 * g], pack64(l0, l1));
        const v4i dh = mfma_i8(x[2 * g + 1], pack64(h0, h1));
        const int s0 = (int)((sc[g >> 1] >> (16 * (g & 1))) & 0xffu), s1 = (int)((sc[g >> 1] >> (16 * (g & 1) + 8)) & 0xffu);
        UNROLL for (int i = 0; i < 4; ++i) { isum[i] += __mul24(s0, dl[i]); isum[i] += __mul24(s1, dh[i]); }
    }
    const float d = h2f_lo(h.x), dm = h2f_hi(h.x);
    UNROLL for (int i = 0; i < 4; ++i) {
        const int msum = mlo[i] + (mhi[i] << 6);
        const float dx = __uint_as_float(dxv[i]);
        acc[i] += (d * dx) * (float)isum[i] - (dm * dx) * (float)msum;
    }
}

/* SLMAX: chunks per slice the instantiation is unrolled for.  PERSIST: the regrouped activations of the
 * whole slice stay in registers so that a wave can walk any number of units (SLMAX 4: 64 registers);
 * without it they are regrouped chunk by chunk into the same 16 registers, and a wave handles exactly one
 * unit (the host launches enough workgroups). */
template <typename F, int SLMAX, bool PERSIST>
PSN_DEV void mv_mfma(const psn_matvec_args &a) {
#define PSN_XI(CI) (PERSIST ? ((CI) < SLMAX ? (CI) : 0) : 0)
    extern __shared__ uint4 psn_smem[];
    typedef __attribute__((address_space(3))) char lds_char;
    lds_char *const lds_ptr = (lds_char *)psn_smem;
    const u32 lds0 = (u32)(uintptr_t)lds_ptr;
    const int lane = threadIdx.x & 63, n = lane & 15, kq = lane >> 4;
    const int wpb = a.threads >> 6;
    const int wib = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int K = a.K, C = K >> 8, KS = a.kslices, SL = C / KS, TPW = wpb / KS;
    const int ks = wib % KS, tl = wib / KS;
    const int c0 = ks * SL;                                  /* first chunk of this wave's K slice */
    const int nw = SL * F::WORDS;                            /* 16-byte words per row of a slice */
    const int ntiles = a.N >> 4;
    const int rb = (int)a.row_bytes;
    const int batch = a.batch;
    const int NI = (nw + 3) >> 2;                            /* load instructions (1 KB each) per unit */

    /* LDS: sub-block sums [C][8 columns][16 B], activation scales [C][8] floats (every wave fills in and
     * reads only its own chunks), 1 KB per wave (regrouping of the activations, later the partial sums
     * [4][64] floats), then one buffer per wave: a ring of four chunks (4 x WORDS words = WORDS load
     * instructions of 1 KB; load instruction i of a unit lands in slot i % WORDS) */
    const u32 xs_tab = lds0, dx_tab = xs_tab + (u32)C * 128u, red = dx_tab + (u32)C * 32u;
    const u32 buf_off = (u32)C * 160u + (u32)wpb * 1024u + (u32)wib * (u32)(F::WORDS << 10);
    const u32 buf = lds0 + buf_off;

    /* The matrices sharing the launch: lane i (< 4) of these registers holds matrix i's base addresses, first
     * row and row count (v_readlane with the matrix index picks one: no block of scalar registers is tied up
     * for the whole kernel, and no indexed read of the kernel arguments).  Row ends past the last matrix
     * equal the total, so they never compare below a row. */
    const int E0 = a.row_end[0], E1 = a.row_end[1], E2 = a.row_end[2];
    u32 seg_w_lo, seg_w_hi, seg_y_lo, seg_y_hi, seg_first, seg_rows;
    {
        const int li = lane & 3;
        /* (the empty asm keeps the compiler from turning the selects into an indexed load from a private
         * copy of the arguments) */
        const uint8_t *W0 = a.W[0], *W1 = a.W[1], *W2 = a.W[2], *W3 = a.W[3];
        float *Y0 = a.y[0], *Y1 = a.y[1], *Y2 = a.y[2], *Y3 = a.y[3];
        int E3 = a.row_end[3];
        asm volatile("" : "+s"(W0), "+s"(W1), "+s"(W2), "+s"(W3), "+s"(Y0), "+s"(Y1), "+s"(Y2), "+s"(Y3), "+s"(E3));
        const uint8_t *wv = li == 0 ? W0 : li == 1 ? W1 : li == 2 ? W2 : W3;
        float *yv = li == 0 ? Y0 : li == 1 ? Y1 : li == 2 ? Y2 : Y3;
        const int fv = li == 0 ? 0 : li == 1 ? E0 : li == 2 ? E1 : E2;
        const int ev = li == 0 ? E0 : li == 1 ? E1 : li == 2 ? E2 : E3;
        seg_w_lo = (u32)(uintptr_t)wv; seg_w_hi = (u32)((uintptr_t)wv >> 32);
        seg_y_lo = (u32)(uintptr_t)yv; seg_y_hi = (u32)((uintptr_t)yv >> 32);
        seg_first = (u32)fv; seg_rows = (u32)(ev - fv);
    }
    /* a tile never straddles two matrices (every matrix holds a multiple of 16 rows) */
    auto tile_base = [&](int tile, const uint8_t *&w, float *&y, int &nrows) {
        const int row0 = tile << 4;
        const int si = (row0 >= E0) + (row0 >= E1) + (row0 >= E2);
        const u64 wb = pack64(__builtin_amdgcn_readlane(seg_w_lo, si), __builtin_amdgcn_readlane(seg_w_hi, si));
        const u64 yb = pack64(__builtin_amdgcn_readlane(seg_y_lo, si), __builtin_amdgcn_readlane(seg_y_hi, si));
        const int first = __builtin_amdgcn_readlane(seg_first, si);
        nrows = __builtin_amdgcn_readlane(seg_rows, si);
        w = (const uint8_t *)(uintptr_t)wb + (int64_t)(row0 - first) * rb;
        y = (float *)(uintptr_t)yb + (row0 - first);
    };

    /* ---- what a wave requests, in this order: its table inputs, then chunk by chunk the activations
     *      (first unit only) and the weight words up to the chunk's end.  A compute unit keeps a bounded
     *      number of bytes in flight and an issuing wave stalls until its request is accepted, so loads
     *      are requested LA chunks ahead of the arithmetic instead of all at once: while some waves sit
     *      in a load instruction the others multiply. ---- */

    /* table inputs: entry e = lane covers (column e & 7, chunk e >> 3) of this wave's slice */
    const int te_m = lane & 7, te_c = lane >> 3;
    const bool te_live = te_c < SL && te_m < batch;
    u32x4 tb0 = (u32x4)(0u), tb1 = (u32x4)(0u);
    u32 tbd = 0;
    if (te_live) {
        const int16_t *p = reinterpret_cast<const int16_t *>(a.xs) + ((int64_t)te_m * C + c0 + te_c) * 16;
        tb0 = global_read128(p);
        tb1 = global_read128(p + 8);
        tbd = global_read32(a.xd + te_m * C + c0 + te_c);
    }

    /* activations: one instruction covers 256 contiguous bytes (a chunk) of each of four columns */
    constexpr int LA = 1;                                    /* chunks requested ahead of the one being multiplied (measured:
                                                              * 0 is 20 % slower, 2 and 3 are 3-8 % slower than 1) */
    u32x4 xt[LA + 1][2];                                     /* chunks CI .. CI + LA are in flight: slot CI % (LA + 1) */
    const int xcol = lane >> 4;                              /* + 4 i */
    const int8_t *xp = a.xqs + (int64_t)xcol * K + (int64_t)c0 * 256 + (lane & 15) * 16;
    const int nx = batch > 4 ? 2 : 1;
    /* weights: lane p fetches row p >> 2; in instruction i it owns word 4 i + ((p & 3) ^ (row >> 2)) */
    const int lrow = lane >> 2, lword = (lane & 3) ^ (lrow >> 2);
    const int64_t lane_goff = (int64_t)lrow * rb + (int64_t)c0 * (F::WORDS * 16);
    const uint8_t *wsrc_lane = nullptr;                      /* current unit's tile + lane_goff */
    auto issue_w = [&](int i0, int i1) {                     /* load instructions i0 .. i1 of the current unit */
        int slot = i0 % F::WORDS;
        int t = lword + 4 * i0;
        for (int i = i0; i <= i1; ++i) {
            lds_char *dst = lds_ptr + buf_off + (slot << 10);
            __builtin_amdgcn_global_load_lds((const void *)(wsrc_lane + min(t, nw - 1) * 16), (__attribute__((address_space(3))) void *)dst, 16, 0, 0);
            t += 4;
            slot = slot + 1 == F::WORDS ? 0 : slot + 1;
        }
    };
    bool first_unit = true;
#define PSN_MF_ISSUE(CI)                                                                                     \
    if (CI < SL) {                                                                                           \
        if (first_unit) {                                                                                    \
            UNROLL for (int i = 0; i < 2; ++i) {                                                             \
                xt[(CI) % (LA + 1)][i] = (u32x4)(0u);                                                                     \
                if (4 * i < batch) {                                                                         \
                    if (xcol + 4 * i < batch) xt[(CI) % (LA + 1)][i] = global_read128(xp + (int64_t)(4 * i) * K + CI * 256); \
                }                                                                                            \
            }                                                                                                \
        }                                                                                                    \
        issue_w(CI == 0 ? 0 : ((F::WORDS * CI - 1) >> 2) + 1, min((F::WORDS * CI + F::WORDS - 1) >> 2, NI - 1)); \
    }

    const int tiles_per_round = a.blocks * TPW;
    const int iters = PERSIST ? (ntiles + tiles_per_round - 1) / tiles_per_round : 1;
    int tile = blockIdx.x * TPW + tl;
    const uint8_t *wtile;
    float *ydst;
    int nrows = 0;
    if (tile < ntiles) {
        tile_base(tile, wtile, ydst, nrows);
        wsrc_lane = wtile + lane_goff;
        if (LA > 0) { PSN_MF_ISSUE(0) }
        if (LA > 1) { PSN_MF_ISSUE(1) }
        if (LA > 2) { PSN_MF_ISSUE(2) }
    }

    /* ---- this wave's table entries: the eight sub-block sums of (column, chunk) as (low 6 bits, signed
     *      rest) bytes, and the activation scale ---- */
    /* the last load instruction of the unit that chunk j needs */
    auto w_last = [&](int j) { return min((F::WORDS * j + F::WORDS - 1) >> 2, NI - 1); };
    {
        const int g = min(LA, SL);                           /* chunks requested so far */
        wait_vmcnt(tile < ntiles ? g * nx + w_last(g - 1) + 1 : 0);
    }
    asm volatile("" : "+v"(tb0), "+v"(tb1), "+v"(tbd));
    if (te_c < SL) {
        u32 lo[2] = {0, 0}, hi[2] = {0, 0};
        UNROLL for (int j = 0; j < 8; ++j) {
            const u32 v = j < 4 ? tb0[j] : tb1[j - 4];
            const int s16 = (int)(int16_t)(v & 0xffffu) + ((int)v >> 16);
            lo[j >> 2] |= (u32)(s16 & 63) << (8 * (j & 3));
            hi[j >> 2] |= (u32)((s16 >> 6) & 0xff) << (8 * (j & 3));
        }
        u32x4 e;
        e.x = lo[0]; e.y = lo[1]; e.z = hi[0]; e.w = hi[1];
        const u32 item = (u32)((c0 + te_c) * 8 + te_m);
        lds_write128(xs_tab + item * 16u, e);
        lds_write32(dx_tab + item * 4u, tbd);
    }

    /* Regrouping of a chunk's activations: lane (m = lane & 15, kq = lane >> 4) needs bytes 8 kq .. 8 kq + 7
     * of every sub-block of column m.  Four columns pass through the wave's own 1 KB at a time: the 8-byte
     * piece (column cq, sub-block sb, quarter kq) sits at
     *     cq * 256 + (((sb >> 1) ^ cq) & 3) * 64 + kq * 16 + (sb & 1) * 8,
     * so a lane picks up two sub-blocks per 16-byte read and the lanes of one read touch every bank
     * once.  One wave's LDS operations execute in order: no waits in between. */
    u64 x[PERSIST ? SLMAX : 1][8];
    UNROLL for (int c = 0; c < (PERSIST ? SLMAX : 1); ++c) UNROLL for (int sb = 0; sb < 8; ++sb) x[c][sb] = 0ull;
    const u32 scratch = red + (u32)wib * 1024u;
    u32 rg_wr, rg_rd;
    {
        const u32 cq_w = (u32)(lane >> 4), w = (u32)(lane & 15), sb_w = w >> 1;
        rg_wr = scratch + cq_w * 256u + ((((sb_w >> 1) ^ cq_w) & 3u) << 6) + (w & 1u) * 32u + (sb_w & 1u) * 8u;
        rg_rd = scratch + (u32)(n & 3) * 256u + (u32)kq * 16u;
    }
    const u32 cq_r = (u32)(n & 3);
#define PSN_MF_REGROUP(CI)                                                                                   \
    UNROLL for (int i = 0; i < 2; ++i) {                                                                     \
        if (4 * i < batch) {                                                                                 \
            asm volatile("" : "+v"(xt[(CI) % (LA + 1)][i]));                                                              \
            lds_write64(rg_wr, pack64(xt[(CI) % (LA + 1)][i].x, xt[(CI) % (LA + 1)][i].y));                                            \
            lds_write64(rg_wr + 16u, pack64(xt[(CI) % (LA + 1)][i].z, xt[(CI) % (LA + 1)][i].w));                                      \
            if ((n >> 2) == i) {                                                                             \
                UNROLL for (u32 q = 0; q < 4; ++q) {                                                         \
                    const u32x4 v = lds_read128<0>(rg_rd + (((q ^ cq_r) & 3u) << 6));                        \
                    x[PSN_XI(CI)][2 * q] = pack64(v.x, v.y);                                                         \
                    x[PSN_XI(CI)][2 * q + 1] = pack64(v.z, v.w);                                                     \
                }                                                                                            \
            }                                                                                                \
        }                                                                                                    \
    }                                                                                                        \
    lds_wait();                                                                                              \
    UNROLL for (int sb = 0; sb < 8; ++sb) tie64(x[PSN_XI(CI)][sb]);

    LaneOffs o;
    {
        const u32 rx = (u32)(n >> 2), hh = (u32)(kq >> 1), half = (u32)(kq & 1);
        const u32 base = buf + (u32)n * 64u;
        UNROLL for (u32 k = 0; k < 4; ++k) {
            o.hdr[k] = base + (((k ^ rx) & 3u) << 4);
            const u32 t = k + hh;
            o.w[k] = base + (t >> 2) * 1024u + ((((t & 3u) ^ rx) & 3u) << 4) + half * 8u;
        }
    }
    const u32 xs_addr = xs_tab + (u32)c0 * 128u + (u32)(n & 7) * 16u;
    const u32 dx_addr = dx_tab + (u32)c0 * 32u + (u32)(kq & 1) * 16u;   /* columns past 7 do not exist: their lanes re-read 0..7 */
    const u32 red_w = red + (u32)wib * 1024u + (u32)lane * 4u;
    const bool first_quarter = kq == 0;

    for (int it = 0; it < iters; ++it) {
        float acc[4] = {0.f, 0.f, 0.f, 0.f};
        const bool live = tile < ntiles;
        if (live) {
            /* chunk CI: request chunk CI + LA, wait until CI's own requests have landed (everything
             * requested later may stay in flight), regroup its activations (first unit), multiply */
#define PSN_MF_CHUNK(CI)                                                                   \
            if (CI < SLMAX && CI < SL) {                                                   \
                if (CI + LA < SLMAX) { PSN_MF_ISSUE((CI + LA < 8 ? CI + LA : 7)) }         \
                {                                                                          \
                    const int g = min(CI + LA + 1, SL);  /* chunks requested so far */     \
                    wait_vmcnt((g - CI - 1) * (first_unit ? nx : 0) + w_last(g - 1) - w_last(CI)); \
                }                                                                          \
                if (first_unit) { PSN_MF_REGROUP(CI) }                                     \
                mf_chunk<F, CI>(o, xs_addr, dx_addr, x[PSN_XI(CI)], first_quarter, acc);   \
            }
            PSN_MF_CHUNK(0) PSN_MF_CHUNK(1) PSN_MF_CHUNK(2) PSN_MF_CHUNK(3)
            PSN_MF_CHUNK(4) PSN_MF_CHUNK(5) PSN_MF_CHUNK(6) PSN_MF_CHUNK(7)
#undef PSN_MF_CHUNK
            first_unit = false;
        }
        float *const ycur = ydst;
        const int ncur = nrows;
        /* the buffer is free: the next unit's first chunks are requested while the partial sums are folded */
        tile += tiles_per_round;
        if (live && tile < ntiles) {
            tile_base(tile, wtile, ydst, nrows);
            wsrc_lane = wtile + lane_goff;
            if (LA > 0) { PSN_MF_ISSUE(0) }
            if (LA > 1) { PSN_MF_ISSUE(1) }
            if (LA > 2) { PSN_MF_ISSUE(2) }
        }
        if (KS > 1) {
            UNROLL for (int i = 0; i < 4; ++i) lds_write32(red_w + (u32)i * 256u, __float_as_uint(acc[i]));
            lds_barrier();
            if (ks == 0) {
                for (int s = 1; s < KS; ++s) {
                    u32 v[4];
                    UNROLL for (int i = 0; i < 4; ++i) v[i] = lds_read32(red_w + (u32)s * 1024u + (u32)i * 256u);
                    lds_wait();
                    UNROLL for (int i = 0; i < 4; ++i) { tie1(v[i]); acc[i] += __uint_as_float(v[i]); }
                }
            }
        }
        if (live && ks == 0) {
            UNROLL for (int i = 0; i < 4; ++i) {
                const int col = 4 * kq + i;
                if (col < batch) ycur[(int64_t)col * ncur + n] = acc[i];
            }
        }
        if (KS > 1) lds_barrier();
    }
#undef PSN_MF_ISSUE
#undef PSN_MF_REGROUP
#undef PSN_XI
}

/* psn_mvm_<fmt>_q8_p4: slices of at most four chunks, any number of units per wave;
 * psn_mvm_<fmt>_q8_t8: slices of at most eight chunks, one unit per wave */
extern "C" __global__ void __launch_bounds__(512) psn_mvm_q4_K_q8_p4(const psn_matvec_args a) { mv_mfma<MfQ4_K, 4, true>(a); }
extern "C" __global__ void __launch_bounds__(512) psn_mvm_q4_K_q8_t8(const psn_matvec_args a) { mv_mfma<MfQ4_K, 8, false>(a); }
extern "C" __global__ void __launch_bounds__(512) psn_mvm_q5_K_q8_p4(const psn_matvec_args a) { mv_mfma<MfQ5_K, 4, true>(a); }
extern "C" __global__ void __launch_bounds__(512) psn_mvm_q5_K_q8_t8(const psn_matvec_args a) { mv_mfma<MfQ5_K, 8, false>(a); }
