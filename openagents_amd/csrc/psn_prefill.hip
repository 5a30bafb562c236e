/*
 * psn_prefill.hip -- gfx950 quantized prefill matmul  Y[m][n] = sum_k h(deq(W)[n][k]) * X[m][k]
 * for GGUF Q4_0 / Q8_0 weights, fp16 activations, fp32 accumulation on v_mfma_f32_32x32x16_f16.
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

#ifndef PSN_ABLATE
#define PSN_ABLATE 0   /* development builds: 1 skips the weight decode, 2 the X loads, 4 the MFMAs of the K loop */
#endif

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

/* 64 dequantized fp16 (blocks 2P and 2P+1 of the chunk) into one swizzled tile row */
template <typename WF, int P>
PSN_DEV void stage_w_row(const u32 (&w)[WF::DW], char *tile, int row) {
    u32 o[32];
    u32 (&o0)[16] = *reinterpret_cast<u32 (*)[16]>(&o[0]);
    u32 (&o1)[16] = *reinterpret_cast<u32 (*)[16]>(&o[16]);
    WF::template deq_block<2 * P>(w, o0);
    WF::template deq_block<2 * P + 1>(w, o1);
    UNROLL for (int c = 0; c < 8; ++c)
        *reinterpret_cast<uint4 *>(tile + tile_off(row, c)) = make_uint4(o[4 * c], o[4 * c + 1], o[4 * c + 2], o[4 * c + 3]);
}

template <typename WF, int BM, int BN, int WM, int WN>
PSN_DEV void prefill_body(const psn_prefill_args &a) {
    static_assert(WM * WN == 4 || WM * WN == 8, "four or eight waves");
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
            __builtin_amdgcn_global_load_lds((const void *)src, (__attribute__((address_space(3))) void *)(tile + (i * NT + wave * 64) * 16), 16, 0, 0);
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

    /* 32x32 accumulator: lane holds column (lane & 31); register r is row 8*(r/4) + 4*(lane/32) + r%4 */
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

/* ---- interleaved variant ------------------------------------------------------------------
 * Same tiles and LDS layout, but arranged so that one basic block holds a whole K step:
 *  - all 256 threads dequantize in every step (256/BN threads share a weight row, each turning
 *    64*BN/256 weights of it into fp16), so there is no divergent branch around the dequantization;
 *  - the operand fragments of k16 slice kk+1 are read while the MFMAs of slice kk are issued;
 *  - scheduling barriers ask the compiler to issue, per MFMA, a share of the dequantization VALU
 *    work and of the LDS traffic, so the matrix pipeline is fed while the vector ALUs decode. */

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

/* X tiles: four LDS stages filled three K steps ahead by direct-to-LDS loads; W tiles: two stages
 * filled one step ahead from registers.  Every stage is its own __shared__ array so that alias
 * analysis can tell the compiler that a W write or a fragment read never touches the stage a
 * pending X load is landing in -- otherwise it waits for all outstanding loads in mid-step. */
template <typename WF, int BM, int BN, int WM, int WN>
PSN_DEV void prefill_body_il(const psn_prefill_args &a) {
    static_assert(WM * WN == 4, "four waves");
    constexpr int NT = 256;
    constexpr int P = NT / BN;                              /* threads per weight row */
    constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
    constexpr int NX = BM * 8 / NT;                         /* direct-to-LDS instructions per X stage */
    constexpr int NW = WF::DW / 4;                          /* global loads per weight chunk */
    __shared__ uint4 xs0[BM * 8], xs1[BM * 8], xs2[BM * 8], xs3[BM * 8];
    __shared__ uint4 ws0[BN * 8], ws1[BN * 8];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;
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
    const int k_last = c_end * 256 - 64;                    /* last K step of this range; later prefetches re-read it */

    float16_t acc[TM][TN];
    UNROLL for (int i = 0; i < TM; ++i) UNROLL for (int j = 0; j < TN; ++j) UNROLL for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
    const int wrow = tid % BN, part = tid / BN;
    const uint8_t *wbase = a.W + (int64_t)min(n0 + wrow, N - 1) * a.row_bytes;
    u32 w[WF::DW], wnext[WF::DW];

    auto stage_x = [&](uint4 *tile, int k0) {
        k0 = min(k0, k_last);
        UNROLL for (int i = 0; i < NX; ++i) {
            const int s = i * NT + tid, row = s >> 3, chunk = (s & 7) ^ (row & 7);
            const uint16_t *src = a.X + (int64_t)min(m0 + row, M - 1) * K + k0 + chunk * 8;
            __builtin_amdgcn_global_load_lds((const void *)src, (__attribute__((address_space(3))) void *)(tile + i * NT + wave * 64), 16, 0, 0);
        }
    };
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

    /* prologue: weight chunk, X stages for the first three steps, W stage for the first */
    WF::load(wbase + (int64_t)c_begin * WF::BYTES, w);
    const int k_begin = c_begin * 256;
    stage_x(xs0, k_begin);
    stage_x(xs1, k_begin + 64);
    stage_x(xs2, k_begin + 128);
    stage_part<WF, 0, P>(w, reinterpret_cast<char *>(ws0), wrow, part);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();

    /* one K step: X stage `xc` and W stage `wc` are current; X for step +3 goes to `xp`, W for step +1
     * to `wq` (from `wsrc`, blocks 2*NSUB and 2*NSUB+1).  KEEP = loads that may stay in flight past the
     * barrier: the X stages of steps +2 and +3, plus the next weight chunk when it was requested after
     * the X stage of step +1. */
#define PSN_PF_STEP(SUB, NSUB, wsrc, xc, xp, wc, wq, KEEP)                                            \
    {                                                                                                 \
        if (!(PSN_ABLATE & 2)) stage_x(xp, (c * 4 + SUB + 3) * 64);                                   \
        half8_t af0[TM], bf0[TN], af1[TM], bf1[TN];                                                   \
        if (!(PSN_ABLATE & 4)) {                                                                      \
            load_frags(xc, wc, 0, af0, bf0);                                                          \
            load_frags(xc, wc, 1, af1, bf1);                                                          \
            mfmas(af0, bf0);                                                                          \
            load_frags(xc, wc, 2, af0, bf0);                                                          \
            mfmas(af1, bf1);                                                                          \
            load_frags(xc, wc, 3, af1, bf1);                                                          \
            mfmas(af0, bf0);                                                                          \
        }                                                                                             \
        if (!(PSN_ABLATE & 1)) stage_part<WF, NSUB, P>(wsrc, reinterpret_cast<char *>(wq), wrow, part); \
        if (!(PSN_ABLATE & 4)) mfmas(af1, bf1);                                                       \
        UNROLL for (int i_ = 0; i_ < 4 * TM * TN; ++i_) {                                             \
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                                        \
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);                                        \
            __builtin_amdgcn_sched_group_barrier(0x002, 6, 0);                                        \
            __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);                                        \
        }                                                                                             \
        /* raw barrier: __syncthreads() would first drain every outstanding load, prefetches included */ \
        asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(KEEP) : "memory");            \
    }

    for (int c = c_begin; c < c_end; ++c) {
        WF::load(wbase + (int64_t)min(c + 1, C - 1) * WF::BYTES, wnext);
        PSN_PF_STEP(0, 1, w, xs0, xs3, ws0, ws1, 2 * NX + NW)
        PSN_PF_STEP(1, 2, w, xs1, xs0, ws1, ws0, 2 * NX + NW)
        PSN_PF_STEP(2, 3, w, xs2, xs1, ws0, ws1, 2 * NX)
        PSN_PF_STEP(3, 0, wnext, xs3, xs2, ws1, ws0, 2 * NX)
        UNROLL for (int i = 0; i < WF::DW; ++i) w[i] = wnext[i];
    }
#undef PSN_PF_STEP
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

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
        const int ptid = tid - 256, pwave = wave - 4;
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
            if (!(PSN_ABLATE & 2)) stage_x(xp, (c * 4 + SUB + 3) * 64);                               \
            if (!(PSN_ABLATE & 1)) stage_part<WF, NSUB, P>(wsrc, reinterpret_cast<char *>(wq), wrow, part); \
            asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"((PSN_ABLATE & 2) ? 0 : KEEP) : "memory"); \
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
        if (!(PSN_ABLATE & 4)) {                                                                      \
            load_frags(xc, wc, 0, af0, bf0);                                                          \
            load_frags(xc, wc, 1, af1, bf1);                                                          \
            mfmas(af0, bf0);                                                                          \
            load_frags(xc, wc, 2, af0, bf0);                                                          \
            mfmas(af1, bf1);                                                                          \
            load_frags(xc, wc, 3, af1, bf1);                                                          \
            mfmas(af0, bf0);                                                                          \
            mfmas(af1, bf1);                                                                          \
        }                                                                                             \
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

/* ---- register-prefetch variant ----------------------------------------------------------------
 * As above, but the X tile travels global -> registers -> LDS: the loads of step s+3 are issued while
 * step s multiplies (two register sets, each load has two full steps to land), and the tile of step
 * s+1 is written to LDS from registers next to the decoded weights.  Ordinary register loads let the
 * compiler count outstanding loads exactly, so nothing drains the queue in mid-loop; two LDS stages
 * per operand suffice. */
template <typename WF, int BM, int BN, int WM, int WN>
PSN_DEV void prefill_body_rp(const psn_prefill_args &a) {
    static_assert(WM * WN == 4, "four waves");
    constexpr int NT = 256;
    constexpr int P = NT / BN;
    constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
    constexpr int NX = BM * 8 / NT;                         /* 16-byte words of X per thread and step */
    __shared__ uint4 xs0[BM * 8], xs1[BM * 8];
    __shared__ uint4 ws0[BN * 8], ws1[BN * 8];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;
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

    float16_t acc[TM][TN];
    UNROLL for (int i = 0; i < TM; ++i) UNROLL for (int j = 0; j < TN; ++j) UNROLL for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
    const int wrow = tid % BN, part = tid / BN;
    const uint8_t *wbase = a.W + (int64_t)min(n0 + wrow, N - 1) * a.row_bytes;
    u32 w[WF::DW], wnext[WF::DW];

    /* this thread's NX words of an X tile: word s = i*NT + tid -> row s/8, chunk (s%8)^(row&7) lands at s */
    const uint16_t *xsrc[NX];
    UNROLL for (int i = 0; i < NX; ++i) {
        const int s_ = i * NT + tid, row = s_ >> 3, chunk = (s_ & 7) ^ (row & 7);
        xsrc[i] = a.X + (int64_t)min(m0 + row, M - 1) * K + chunk * 8;
    }
    auto load_x = [&](uint4 (&r)[NX], int k0) {
        k0 = min(k0, k_last);
        UNROLL for (int i = 0; i < NX; ++i) r[i] = *reinterpret_cast<const uint4 *>(xsrc[i] + k0);
    };
    auto store_x = [&](uint4 *tile, const uint4 (&r)[NX]) {
        UNROLL for (int i = 0; i < NX; ++i) tile[i * NT + tid] = r[i];
    };
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

    /* prologue: step 0 into LDS, steps 1 and 2 into the two register sets */
    uint4 xa[NX], xb[NX];
    const int k_begin = c_begin * 256;
    WF::load(wbase + (int64_t)c_begin * WF::BYTES, w);
    load_x(xa, k_begin);
    store_x(xs0, xa);
    load_x(xb, k_begin + 64);                               /* X(1) */
    load_x(xa, k_begin + 128);                              /* X(2) */
    stage_part<WF, 0, P>(w, reinterpret_cast<char *>(ws0), wrow, part);
    __syncthreads();

    /* step SUB of chunk c: multiply from (xc, wc); X(step+1) goes from `xr` to LDS stage xq and `xr` is
     * refilled with X(step+3); W(step+1) is decoded from `wsrc` (blocks 2*NSUB, 2*NSUB+1) into wq */
#define PSN_RP_STEP(SUB, NSUB, wsrc, xc, xq, wc, wq, xr)                                               \
    {                                                                                                 \
        half8_t af0[TM], bf0[TN], af1[TM], bf1[TN];                                                   \
        load_frags(xc, wc, 0, af0, bf0);                                                              \
        load_frags(xc, wc, 1, af1, bf1);                                                              \
        store_x(xq, xr);                                                                              \
        load_x(xr, (c * 4 + SUB + 3) * 64);                                                           \
        mfmas(af0, bf0);                                                                              \
        load_frags(xc, wc, 2, af0, bf0);                                                              \
        mfmas(af1, bf1);                                                                              \
        load_frags(xc, wc, 3, af1, bf1);                                                              \
        mfmas(af0, bf0);                                                                              \
        stage_part<WF, NSUB, P>(wsrc, reinterpret_cast<char *>(wq), wrow, part);                      \
        mfmas(af1, bf1);                                                                              \
        UNROLL for (int i_ = 0; i_ < 4 * TM * TN; ++i_) {                                             \
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                                        \
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);                                        \
            __builtin_amdgcn_sched_group_barrier(0x002, 6, 0);                                        \
            __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);                                        \
        }                                                                                             \
        __builtin_amdgcn_s_waitcnt(0xC07F);                 /* lgkmcnt(0): this wave's LDS writes are done */ \
        __builtin_amdgcn_s_barrier();                                                                 \
    }

    for (int c = c_begin; c < c_end; ++c) {
        WF::load(wbase + (int64_t)min(c + 1, C - 1) * WF::BYTES, wnext);
        PSN_RP_STEP(0, 1, w, xs0, xs1, ws0, ws1, xb)
        PSN_RP_STEP(1, 2, w, xs1, xs0, ws1, ws0, xa)
        PSN_RP_STEP(2, 3, w, xs0, xs1, ws0, ws1, xb)
        PSN_RP_STEP(3, 0, wnext, xs1, xs0, ws1, ws0, xa)
        UNROLL for (int i = 0; i < WF::DW; ++i) w[i] = wnext[i];
    }
#undef PSN_RP_STEP

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

/* zero fill with plain vector stores (graph-safe stand-in for a memset node) */
extern "C" __global__ void __launch_bounds__(256) psn_fill_zero(const psn_fill_args a) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    uint4 *p = reinterpret_cast<uint4 *>(a.p);
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < a.n16; i += stride) p[i] = make_uint4(0, 0, 0, 0);
}

#define PSN_PREFILL_KERNEL(fmt, WF, BM, BN, WM, WN)                                                          \
    extern "C" __global__ void __launch_bounds__(256) psn_prefill_##fmt##_m##BM##_n##BN(const psn_prefill_args a) { \
        prefill_body<WF, BM, BN, WM, WN>(a);                                                                 \
    }
/* eight-wave variants (512 threads, two waves per SIMD: one can multiply while the other stages) */
#define PSN_PREFILL_KERNEL8(fmt, WF, BM, BN, WM, WN)                                                         \
    extern "C" __global__ void __launch_bounds__(512) psn_prefill_##fmt##_m##BM##_n##BN##_w8(const psn_prefill_args a) { \
        prefill_body<WF, BM, BN, WM, WN>(a);                                                                 \
    }

#define PSN_PREFILL_KERNEL_IL(fmt, WF, BM, BN, WM, WN)                                                       \
    extern "C" __global__ void __launch_bounds__(256) psn_prefill_##fmt##_m##BM##_n##BN##_il(const psn_prefill_args a) { \
        prefill_body_il<WF, BM, BN, WM, WN>(a);                                                              \
    }

#define PSN_PREFILL_KERNEL_WS(fmt, WF, BM, BN)                                                               \
    extern "C" __global__ void __launch_bounds__(512) psn_prefill_##fmt##_m##BM##_n##BN##_ws(const psn_prefill_args a) { \
        prefill_body_ws<WF, BM, BN>(a);                                                                      \
    }

#define PSN_PREFILL_KERNEL_RP(fmt, WF, BM, BN, WM, WN)                                                       \
    extern "C" __global__ void __launch_bounds__(256) psn_prefill_##fmt##_m##BM##_n##BN##_rp(const psn_prefill_args a) { \
        prefill_body_rp<WF, BM, BN, WM, WN>(a);                                                              \
    }

#define PSN_PREFILL_ALL(fmt, WF)               \
    PSN_PREFILL_KERNEL_WS(fmt, WF, 128, 128)     \
    PSN_PREFILL_KERNEL_WS(fmt, WF, 128, 256)     \
    PSN_PREFILL_KERNEL_RP(fmt, WF, 128, 128, 2, 2) \
    PSN_PREFILL_KERNEL_RP(fmt, WF, 128, 256, 2, 2) \
    PSN_PREFILL_KERNEL_RP(fmt, WF, 256, 128, 2, 2) \
    PSN_PREFILL_KERNEL_RP(fmt, WF, 256, 256, 2, 2) \
    PSN_PREFILL_KERNEL_IL(fmt, WF, 64, 128, 2, 2)  \
    PSN_PREFILL_KERNEL_IL(fmt, WF, 128, 128, 2, 2) \
    PSN_PREFILL_KERNEL_IL(fmt, WF, 128, 256, 2, 2) \
    PSN_PREFILL_KERNEL(fmt, WF, 64, 64, 2, 2)    \
    PSN_PREFILL_KERNEL(fmt, WF, 64, 128, 2, 2)   \
    PSN_PREFILL_KERNEL(fmt, WF, 128, 128, 2, 2)  \
    PSN_PREFILL_KERNEL(fmt, WF, 128, 256, 2, 2)  \
    PSN_PREFILL_KERNEL(fmt, WF, 256, 128, 2, 2)  \
    PSN_PREFILL_KERNEL(fmt, WF, 256, 256, 2, 2)  \
    PSN_PREFILL_KERNEL8(fmt, WF, 128, 128, 2, 4) \
    PSN_PREFILL_KERNEL8(fmt, WF, 256, 128, 4, 2) \
    PSN_PREFILL_KERNEL8(fmt, WF, 128, 256, 2, 4) \
    PSN_PREFILL_KERNEL8(fmt, WF, 256, 256, 2, 4)

PSN_PREFILL_ALL(q4_0, PfQ4_0)
PSN_PREFILL_ALL(q8_0, PfQ8_0)
