/*
 * psn_matvec.hip -- gfx950 decode kernels: activation quantizers and the batch-1..8 quantized
 * matvec y[b][n] = sum_k deq(W)[n][k] * x[b][k] over GGUF Q4_0 / Q8_0 / Q4_K / Q6_K rows.
 * One launch can serve up to four matrices that share x (q/k/v, gate/up): their rows are walked
 * as one concatenated row space ("segments").
 *
 * The matvec is an HBM stream, so everything is organised around 128-bit loads of the raw GGUF
 * bytes.  Blocks are 18 / 34 / 144 / 210 bytes, which is not a multiple of 16, but 256 weights
 * always are a whole number of 16-byte words for Q4_0 (144 B), Q8_0 (272 B) and Q4_K (144 B), so a
 * lane owns one 256-weight "chunk" of a row: it fetches it with 9 or 17 aligned dwordx4 loads and
 * re-aligns the 2-byte-shifted halves in registers with v_alignbyte.  Q6_K (210 B) is fetched with
 * 2-byte-aligned dwordx4 loads, which gfx950 serves in unaligned access mode.
 *
 * Work split: G lanes share a row (G = 8..64), a wave therefore holds 64/G rows at a time and R
 * such row sets are in flight per lane to keep enough bytes outstanding; partial sums are folded
 * with DPP / ds_swizzle (psn_device.h).  Weights held in registers are re-used for every batch
 * column.  Scheme Q8 multiplies int8 x int8 with v_dot4_i32_i8 and applies the fp16 block scales in
 * fp32; scheme F32 dequantizes to fp32 and uses fp32 FMA.
 */
#include "psn_args.h"
#include "psn_device.h"

#define UNROLL _Pragma("unroll")

/* ------------------------------------------------------------------------------------------
 * Activation quantizers (bit-exact restatements of the Q8_0 / Q8_K row quantizers).  The same
 * math runs as stand-alone kernels and inside the matvec's staging step.
 * ------------------------------------------------------------------------------------------ */

#if !defined(PSN_BUILD_ONLY) || defined(PSN_BUILD_QUANT)
extern "C" __global__ void __launch_bounds__(256) psn_quantize_q8_0(const psn_quantize_args a) {
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;   /* one float4 each */
    const int64_t total4 = (int64_t)a.K * a.batch / 4;
    const bool live = t < total4;
    const float4 v = live ? reinterpret_cast<const float4 *>(a.x)[t] : make_float4(0.f, 0.f, 0.f, 0.f);
    u32 packed;
    float d;
    int s;
    q8_0_quant4(v, packed, d, s);
    if (!live) return;
    reinterpret_cast<u32 *>(a.qs)[t] = packed;
    if ((threadIdx.x & 7) == 0) {
        a.d[t >> 3] = d;
        reinterpret_cast<int *>(a.s)[t >> 3] = s;
    }
}

extern "C" __global__ void __launch_bounds__(256) psn_quantize_q8_K(const psn_quantize_args a) {
    const int lane = threadIdx.x & 63;
    const int64_t sb = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;   /* super-block index */
    const int64_t nsb = (int64_t)a.K * a.batch / 256;
    if (sb >= nsb) return;                                                        /* whole wave leaves together */
    const float4 v = reinterpret_cast<const float4 *>(a.x)[sb * 64 + lane];
    u32 packed;
    float d;
    int s16;
    q8_K_quant_wave(v, lane, packed, d, s16);
    reinterpret_cast<u32 *>(a.qs)[sb * 64 + lane] = packed;
    if ((lane & 3) == 0) reinterpret_cast<int16_t *>(a.s)[sb * 16 + (lane >> 2)] = (int16_t)s16;
    if (lane == 0) a.d[sb] = d;
}
#endif

/* ------------------------------------------------------------------------------------------
 * Shared scaffolding of the chunk-per-lane matvec kernels.
 * ------------------------------------------------------------------------------------------ */

template <int G, int R>
struct RowMap {
    static constexpr int S = 64 / G;          /* rows a wave holds side by side */
    static constexpr int ROWS = S * R;        /* rows a wave retires per pass */
    int lane, slot, j, wave, nwaves;
    PSN_DEV RowMap(const psn_matvec_args &a) {
        lane = threadIdx.x & 63;
        slot = lane / G;
        j = lane % G;
        const int wpb = a.threads >> 6;
        wave = blockIdx.x * wpb + (threadIdx.x >> 6);
        nwaves = a.blocks * wpb;
    }
};

/* The per-matrix base pointers and row boundaries of a launch, pinned in scalar registers (plain
 * locals of the kernel body, declared by this macro).  Lanes pick theirs with compares and selects;
 * the empty asm keeps the compiler from folding the selects back into an indexed (vector-memory)
 * load from a private copy of the kernel arguments, which would put memory round trips in front of
 * the first weight load.  Unused segments repeat the last one (row_end == N), so no count check is
 * needed.  seg_row_ptr(row): start of that row's blocks; seg_out_ptr(row, nrows): where its
 * batch-column-0 output goes and how many rows its matrix has. */
#define PSN_DECLARE_SEGMENTS(a)                                                                             \
    const uint8_t *sgW0 = (a).W[0], *sgW1 = (a).W[1], *sgW2 = (a).W[2], *sgW3 = (a).W[3];                   \
    float *sgY0 = (a).y[0], *sgY1 = (a).y[1], *sgY2 = (a).y[2], *sgY3 = (a).y[3];                           \
    int sgE0 = (a).row_end[0], sgE1 = (a).row_end[1], sgE2 = (a).row_end[2], sgE3 = (a).row_end[3];         \
    asm volatile("" : "+s"(sgW0), "+s"(sgW1), "+s"(sgW2), "+s"(sgW3), "+s"(sgY0), "+s"(sgY1), "+s"(sgY2),   \
                 "+s"(sgY3), "+s"(sgE0), "+s"(sgE1), "+s"(sgE2), "+s"(sgE3));                               \
    const int64_t sg_row_bytes = (a).row_bytes
#define seg_row_ptr(row) seg_row_ptr_fn((row), sg_row_bytes, sgW0, sgW1, sgW2, sgW3, sgE0, sgE1, sgE2)
#define seg_out_ptr(row, nrows) seg_out_ptr_fn((row), (nrows), sgY0, sgY1, sgY2, sgY3, sgE0, sgE1, sgE2, sgE3)

PSN_DEV const uint8_t *seg_row_ptr_fn(int row, int64_t row_bytes, const uint8_t *w0, const uint8_t *w1, const uint8_t *w2,
                                      const uint8_t *w3, int e0, int e1, int e2) {
    const uint8_t *w = w0;
    int first = 0;
    if (row >= e0) { w = w1; first = e0; }
    if (row >= e1) { w = w2; first = e1; }
    if (row >= e2) { w = w3; first = e2; }
    return w + (int64_t)(row - first) * row_bytes;
}
PSN_DEV float *seg_out_ptr_fn(int row, int &rows_of_matrix, float *y0, float *y1, float *y2, float *y3, int e0, int e1, int e2, int e3) {
    float *y = y0;
    int first = 0, end = e0;
    if (row >= e0) { y = y1; first = e0; end = e1; }
    if (row >= e1) { y = y2; first = e1; end = e2; }
    if (row >= e2) { y = y3; first = e2; end = e3; }
    rows_of_matrix = end - first;
    return y + (row - first);
}

/* folds the G-lane partial sums of R row sets x NB batch columns and stores them */
#define PSN_STORE_ROWS(m, acc, a, row0)                                                                     \
    UNROLL for (int r_ = 0; r_ < R; ++r_) {                                                                 \
        const int row_ = (row0) + r_ * (m).S + (m).slot;                                                    \
        int nrows_;                                                                                         \
        float *dst_ = seg_out_ptr(min(row_, (a).N - 1), nrows_);                                            \
        UNROLL for (int nb_ = 0; nb_ < NB; ++nb_) {                                                         \
            const float v_ = group_sum<G>((acc)[r_][nb_]);                                                  \
            if ((m).j == 0 && row_ < (a).N && nb_ < (a).batch) dst_[(int64_t)nb_ * nrows_] = v_;            \
        }                                                                                                   \
    }

/* one chunk (index c) of R rows starting at row0 into registers; rows past the end re-read the last one */
#define PSN_LOAD_ROWS(F, m, a, row0, c, w)                                                                  \
    UNROLL for (int r_ = 0; r_ < R; ++r_) {                                                                 \
        const int row_ = min((row0) + r_ * (m).S + (m).slot, (a).N - 1);                                    \
        F::load(seg_row_ptr(row_) + (int64_t)(c) * F::BYTES, (w)[r_]);                                      \
    }

/* Quantized activations as the kernels see them: either the global three-field layout or a copy
 * staged in LDS.  In LDS every 256-byte chunk of qs is followed by 16 bytes of padding, so lanes
 * that own neighbouring chunks start 68 dwords apart and their 128-bit reads fall into disjoint
 * banks (a 64-dword stride would put all of them on the same ones). */
template <typename ST>
struct ActQ {
    const int8_t *qs;
    const float *d;
    const ST *s;
    int chunk_stride;   /* bytes between consecutive 256-element chunks of qs */
    int col_stride;     /* bytes between batch columns of qs */
    PSN_DEV const uint4 *chunk(int col, int c) const {
        return reinterpret_cast<const uint4 *>(qs + (int64_t)col * col_stride + (int64_t)c * chunk_stride);
    }
};

/* Brings the activations to where the dot products read them, in two halves so that the weight
 * loads of the first chunk can be issued in between: issue() starts the (small) activation loads,
 * finish() waits for them only -- loads return in order, the weights stay in flight -- writes LDS
 * and crosses the workgroup barrier.
 *   XSRC 0: quantized activations stay in global memory (no LDS);
 *   XSRC 1: quantized activations copied into LDS;
 *   XSRC 2: fp32 activations quantized into LDS by the workgroup itself (every workgroup redoes the
 *           tiny quantization instead of a separate launch doing it once).
 * ST = int selects Q8_0 activations (d and s per 32), ST = int16_t Q8_K (d per 256, bsums per 16).
 * Up to SLOTS 16-byte words per thread are held in registers; larger inputs (long K, batch > 1 on
 * small workgroups) take the plain copy loop in finish(). */
template <typename ST, int XSRC, bool REGS = true>
struct Stager {
    static constexpr int SLOTS = 8;
    uint4 t[SLOTS];
    uint4 td, ts;
    int n_qs, n_d, n_s, C, nthreads;
    bool in_regs;

    PSN_DEV void issue(const psn_matvec_args &a, int d_per_col, int s_per_col) {
        C = a.K >> 8;
        nthreads = a.threads;
        n_qs = a.batch * C * 16;                                   /* 16-byte words of int8 */
        n_d = (a.batch * d_per_col * 4 + 15) / 16;                 /* the global fields are padded to 256 B */
        n_s = (a.batch * s_per_col * (int)sizeof(ST) + 15) / 16;
        in_regs = false;
        if constexpr (!REGS) return;                               /* finish() does plain copy loops */
        UNROLL for (int i = 0; i < SLOTS; ++i) t[i] = make_uint4(0, 0, 0, 0);
        td = ts = make_uint4(0, 0, 0, 0);
        if constexpr (XSRC == 1) {
            in_regs = n_qs <= SLOTS * nthreads && n_d <= nthreads && n_s <= nthreads;
            if (in_regs) {
                const uint4 *g_qs = reinterpret_cast<const uint4 *>(a.xqs);
                UNROLL for (int i = 0; i < SLOTS; ++i) {
                    const int idx = threadIdx.x + i * nthreads;
                    if (idx < n_qs) t[i] = g_qs[idx];
                }
                if ((int)threadIdx.x < n_d) td = reinterpret_cast<const uint4 *>(a.xd)[threadIdx.x];
                if ((int)threadIdx.x < n_s) ts = reinterpret_cast<const uint4 *>(a.xs)[threadIdx.x];
            }
        } else if constexpr (XSRC == 2) {
            const float4 *x4 = reinterpret_cast<const float4 *>(a.xf);
            if constexpr (sizeof(ST) == 4) {
                const int total4 = a.batch * C * 64;               /* float4 words: whole waves, whole blocks */
                in_regs = total4 <= SLOTS * nthreads;
                if (in_regs) {
                    UNROLL for (int i = 0; i < SLOTS; ++i) {
                        const int idx = threadIdx.x + i * nthreads;
                        if (idx < total4) { const float4 v = x4[idx]; t[i] = make_uint4(__float_as_uint(v.x), __float_as_uint(v.y), __float_as_uint(v.z), __float_as_uint(v.w)); }
                    }
                }
            } else {
                /* sixteen lanes to a super-block, four blocks to a wave and round: slots 0..3 hold the four quarters
                 * of the lane's block in the first round, slots 4..7 those of the second */
                const int nsb = a.batch * C, wpb = nthreads >> 6, l15 = threadIdx.x & 15;
                in_regs = nsb <= SLOTS * wpb;
                if (in_regs) {
                    UNROLL for (int i = 0; i < SLOTS; ++i) {
                        const int sb = (i >> 2) * (wpb * 4) + (int)(threadIdx.x >> 4);
                        if (sb < nsb) { const float4 v = x4[sb * 64 + (i & 3) * 16 + l15]; t[i] = make_uint4(__float_as_uint(v.x), __float_as_uint(v.y), __float_as_uint(v.z), __float_as_uint(v.w)); }
                    }
                }
            }
        }
    }

    PSN_DEV ActQ<ST> finish(const psn_matvec_args &a) {
        ActQ<ST> x;
        if constexpr (XSRC == 0) {
            x.qs = a.xqs;
            x.d = a.xd;
            x.s = reinterpret_cast<const ST *>(a.xs);
            x.chunk_stride = 256;
            x.col_stride = a.K;
            return x;
        } else {
            extern __shared__ uint4 psn_smem[];
            uint4 *l_qs4 = psn_smem, *l_d4 = l_qs4 + a.batch * C * 17, *l_s4 = l_d4 + n_d;
            if constexpr (XSRC == 1) {
                const uint4 *g_qs = reinterpret_cast<const uint4 *>(a.xqs), *g_d = reinterpret_cast<const uint4 *>(a.xd);
                const uint4 *g_s = reinterpret_cast<const uint4 *>(a.xs);
                if (in_regs) {
                    UNROLL for (int i = 0; i < SLOTS; ++i) {
                        const int idx = threadIdx.x + i * nthreads;
                        if (idx < n_qs) l_qs4[(idx >> 4) * 17 + (idx & 15)] = t[i];
                    }
                    if ((int)threadIdx.x < n_d) l_d4[threadIdx.x] = td;
                    if ((int)threadIdx.x < n_s) l_s4[threadIdx.x] = ts;
                } else {
                    for (int i = threadIdx.x; i < n_qs; i += nthreads) l_qs4[(i >> 4) * 17 + (i & 15)] = g_qs[i];
                    for (int i = threadIdx.x; i < n_d; i += nthreads) l_d4[i] = g_d[i];
                    for (int i = threadIdx.x; i < n_s; i += nthreads) l_s4[i] = g_s[i];
                }
            } else {
                u32 *l_qs = reinterpret_cast<u32 *>(l_qs4);
                float *l_d = reinterpret_cast<float *>(l_d4);
                ST *l_s = reinterpret_cast<ST *>(l_s4);
                const float4 *x4 = reinterpret_cast<const float4 *>(a.xf);
                const int lane = threadIdx.x & 63;
                if constexpr (sizeof(ST) == 4) {
                    const int total4 = a.batch * C * 64;
                    auto one = [&](int i, const float4 v) {
                        u32 packed;
                        float d;
                        int sum;
                        q8_0_quant4(v, packed, d, sum);
                        l_qs[(i >> 6) * 68 + (i & 63)] = packed;      /* chunk index i/64 already runs over batch */
                        if ((lane & 7) == 0) { l_d[i >> 3] = d; l_s[i >> 3] = sum; }
                    };
                    if (in_regs) {
                        UNROLL for (int k = 0; k < SLOTS; ++k) {
                            const int i = threadIdx.x + k * nthreads;
                            if (i < total4) one(i, make_float4(__uint_as_float(t[k].x), __uint_as_float(t[k].y), __uint_as_float(t[k].z), __uint_as_float(t[k].w)));
                        }
                    } else {
                        for (int i = threadIdx.x; i < total4; i += nthreads) one(i, x4[i]);
                    }
                } else {
                    const int nsb = a.batch * C, wpb = nthreads >> 6, l15 = lane & 15;
                    /* the wave's four blocks of one round: sb is this lane's, v its four quarters (zeros past the end) */
                    auto four = [&](int sb, const float4 (&v)[4]) {
                        u32 packed[4];
                        float d;
                        int s16[4];
                        q8_K_quant_row16(v, lane, packed, d, s16);
                        if (sb < nsb) {
                            UNROLL for (int i = 0; i < 4; ++i) {
                                l_qs[sb * 68 + i * 16 + l15] = packed[i];
                                if ((lane & 3) == 0) l_s[sb * 16 + i * 4 + (l15 >> 2)] = (ST)s16[i];
                            }
                            if (l15 == 0) l_d[sb] = d;
                        }
                    };
                    if (in_regs) {
                        UNROLL for (int r = 0; r < SLOTS / 4; ++r) {
                            const int sb = r * (wpb * 4) + (int)(threadIdx.x >> 4);
                            if (__builtin_amdgcn_readfirstlane(sb) < nsb) {       /* wave-uniform: the round's first block exists */
                                float4 v[4];
                                UNROLL for (int i = 0; i < 4; ++i)
                                    v[i] = make_float4(__uint_as_float(t[4 * r + i].x), __uint_as_float(t[4 * r + i].y), __uint_as_float(t[4 * r + i].z), __uint_as_float(t[4 * r + i].w));
                                four(sb, v);
                            }
                        }
                    } else {
                        for (int base = (int)(threadIdx.x >> 6) * 4; base < nsb; base += wpb * 4) {
                            const int sb = base + (lane >> 4);
                            float4 v[4];
                            UNROLL for (int i = 0; i < 4; ++i) v[i] = sb < nsb ? x4[sb * 64 + i * 16 + l15] : make_float4(0.f, 0.f, 0.f, 0.f);
                            four(sb, v);
                        }
                    }
                }
            }
            __syncthreads();
            x.qs = reinterpret_cast<const int8_t *>(l_qs4);
            x.d = reinterpret_cast<const float *>(l_d4);
            x.s = reinterpret_cast<const ST *>(l_s4);
            x.chunk_stride = 272;
            x.col_stride = C * 272;
            return x;
        }
    }
};

/* ------------------------------------------------------------------------------------------
 * Formats.  Each supplies: DW/BYTES (a lane's 256-weight chunk), load() of the chunk's dwords,
 * XR + load_x() (the matching 256 activations with their scales, as registers) and dot()
 * (the chunk's contribution to the row's sum); deq32() serves the F32 scheme.
 *
 * Q4_0: chunk = 8 blocks = 144 B = 36 dwords.  Block b starts at byte 18b: even blocks start on
 * a dword (fp16 d in the low half, quants shifted by two bytes), odd blocks start mid-dword (d in
 * the high half, quants aligned).  sum (q-8)*x = sum q*x - 8*sum x uses the activation block sums
 * so nibbles stay unsigned.
 * ------------------------------------------------------------------------------------------ */

template <int B>
PSN_DEV void q4_0_block(const u32 (&w)[36], float &d, u32 (&lo)[4], u32 (&hi)[4]) {
    constexpr int base = 9 * (B >> 1);
    u32 q[4];
    if constexpr ((B & 1) == 0) {
        d = h2f_lo(w[base]);
        UNROLL for (int i = 0; i < 4; ++i) q[i] = align2(w[base + i + 1], w[base + i]);
    } else {
        d = h2f_hi(w[base + 4]);
        UNROLL for (int i = 0; i < 4; ++i) q[i] = w[base + 5 + i];
    }
    UNROLL for (int i = 0; i < 4; ++i) { lo[i] = q[i] & 0x0f0f0f0fu; hi[i] = (q[i] >> 4) & 0x0f0f0f0fu; }
}

template <int B>
PSN_DEV void q8_0_block(const u32 (&w)[68], float &d, u32 (&q)[8]) {
    constexpr int base = 17 * (B >> 1);
    if constexpr ((B & 1) == 0) {
        d = h2f_lo(w[base]);
        UNROLL for (int i = 0; i < 8; ++i) q[i] = align2(w[base + i + 1], w[base + i]);
    } else {
        d = h2f_hi(w[base + 8]);
        UNROLL for (int i = 0; i < 8; ++i) q[i] = w[base + 9 + i];
    }
}

/* activations of one chunk for the 32-element-block formats: 64 dwords of int8, 8 scales, 8 sums */
PSN_DEV void load_x_q8_0(const ActQ<int> &x, int K, int col, int c, u32 (&xr)[80]) {
    const uint4 *xp = x.chunk(col, c);
    UNROLL for (int i = 0; i < 16; ++i) unpack4(xp[i], &xr[4 * i]);
    const int nblk = K >> 5;
    const uint4 *dp = reinterpret_cast<const uint4 *>(x.d + col * nblk + c * 8);
    const uint4 *sp = reinterpret_cast<const uint4 *>(x.s + col * nblk + c * 8);
    unpack4(dp[0], &xr[64]);
    unpack4(dp[1], &xr[68]);
    unpack4(sp[0], &xr[72]);
    unpack4(sp[1], &xr[76]);
}
/* ... and for the super-block formats: 64 dwords of int8, one scale, 16 int16 group sums */
PSN_DEV void load_x_q8_K(const ActQ<int16_t> &x, int K, int col, int c, u32 (&xr)[73]) {
    const int C = K >> 8;
    const uint4 *xp = x.chunk(col, c);
    UNROLL for (int i = 0; i < 16; ++i) unpack4(xp[i], &xr[4 * i]);
    xr[64] = __float_as_uint(x.d[col * C + c]);
    const uint4 *bp = reinterpret_cast<const uint4 *>(x.s + ((int64_t)col * C + c) * 16);
    unpack4(bp[0], &xr[65]);
    unpack4(bp[1], &xr[69]);
}

struct FmtQ4_0 {
    static constexpr int DW = 36, BYTES = 144, XR = 80;
    typedef int ActSum;
    static PSN_DEV int d_per_col(int K) { return K >> 5; }
    static PSN_DEV int s_per_col(int K) { return K >> 5; }
    static PSN_DEV void load(const uint8_t *p, u32 (&w)[DW]) {
        const uint4 *q = reinterpret_cast<const uint4 *>(p);
        UNROLL for (int i = 0; i < 9; ++i) unpack4(q[i], &w[4 * i]);
    }
    static PSN_DEV void load_x(const ActQ<int> &x, int K, int col, int c, u32 (&xr)[XR]) { load_x_q8_0(x, K, col, c, xr); }
    template <int B>
    static PSN_DEV float block(const u32 (&w)[DW], const u32 (&xr)[XR]) {
        float dw;
        u32 lo[4], hi[4];
        q4_0_block<B>(w, dw, lo, hi);
        int s = 0;
        UNROLL for (int i = 0; i < 4; ++i) s = dot4(lo[i], xr[8 * B + i], s);
        UNROLL for (int i = 0; i < 4; ++i) s = dot4(hi[i], xr[8 * B + 4 + i], s);
        s -= 8 * (int)xr[72 + B];
        return (float)s * dw * __uint_as_float(xr[64 + B]);
    }
    static PSN_DEV float dot(const u32 (&w)[DW], const u32 (&xr)[XR]) {
        float acc = block<0>(w, xr);
        acc += block<1>(w, xr); acc += block<2>(w, xr); acc += block<3>(w, xr);
        acc += block<4>(w, xr); acc += block<5>(w, xr); acc += block<6>(w, xr); acc += block<7>(w, xr);
        return acc;
    }
    /* 32 weights of GGUF block SB of the chunk, fp32, element order (scheme F32) */
    template <int SB>
    static PSN_DEV void deq32(const u32 (&w)[DW], float (&o)[32]) {
        float d;
        u32 lo[4], hi[4];
        q4_0_block<SB>(w, d, lo, hi);
        const float off = -8.f * d;
        UNROLL for (int i = 0; i < 4; ++i) UNROLL for (int b = 0; b < 4; ++b) {
            o[4 * i + b] = __builtin_fmaf((float)((lo[i] >> (8 * b)) & 0xffu), d, off);
            o[16 + 4 * i + b] = __builtin_fmaf((float)((hi[i] >> (8 * b)) & 0xffu), d, off);
        }
    }
};

/* Q8_0: chunk = 8 blocks = 272 B = 68 dwords; block b starts at byte 34b. */
struct FmtQ8_0 {
    static constexpr int DW = 68, BYTES = 272, XR = 80;
    typedef int ActSum;
    static PSN_DEV int d_per_col(int K) { return K >> 5; }
    static PSN_DEV int s_per_col(int K) { return K >> 5; }
    static PSN_DEV void load(const uint8_t *p, u32 (&w)[DW]) {
        const uint4 *q = reinterpret_cast<const uint4 *>(p);
        UNROLL for (int i = 0; i < 17; ++i) unpack4(q[i], &w[4 * i]);
    }
    static PSN_DEV void load_x(const ActQ<int> &x, int K, int col, int c, u32 (&xr)[XR]) { load_x_q8_0(x, K, col, c, xr); }
    template <int B>
    static PSN_DEV float block(const u32 (&w)[DW], const u32 (&xr)[XR]) {
        float dw;
        u32 q[8];
        q8_0_block<B>(w, dw, q);
        int s = 0;
        UNROLL for (int i = 0; i < 8; ++i) s = dot4(q[i], xr[8 * B + i], s);
        return (float)s * (dw * __uint_as_float(xr[64 + B]));
    }
    static PSN_DEV float dot(const u32 (&w)[DW], const u32 (&xr)[XR]) {
        float acc = block<0>(w, xr);
        acc += block<1>(w, xr); acc += block<2>(w, xr); acc += block<3>(w, xr);
        acc += block<4>(w, xr); acc += block<5>(w, xr); acc += block<6>(w, xr); acc += block<7>(w, xr);
        return acc;
    }
    template <int SB>
    static PSN_DEV void deq32(const u32 (&w)[DW], float (&o)[32]) {
        float d;
        u32 q[8];
        q8_0_block<SB>(w, d, q);
        UNROLL for (int i = 0; i < 8; ++i) UNROLL for (int b = 0; b < 4; ++b)
            o[4 * i + b] = (float)(int)(int8_t)((q[i] >> (8 * b)) & 0xffu) * d;
    }
};

/* Q4_K: chunk = one 144-byte super-block: dword 0 = d | dmin<<16, dwords 1..3 = the 12-byte
 * 6-bit scale/min field, dwords 4..35 = 128 nibble bytes (64 weights per 32 bytes: low nibbles
 * then high nibbles). */
PSN_DEV void q4_K_scales(u32 s0, u32 s1, u32 s2, u32 (&sc)[2], u32 (&mn)[2]) {
    sc[0] = s0 & 0x3f3f3f3fu;
    mn[0] = s1 & 0x3f3f3f3fu;
    sc[1] = (s2 & 0x0f0f0f0fu) | ((s0 >> 2) & 0x30303030u);
    mn[1] = ((s2 >> 4) & 0x0f0f0f0fu) | ((s1 >> 2) & 0x30303030u);
}
PSN_DEV int byte_of(const u32 (&v)[2], int i) { return (int)((v[i >> 2] >> (8 * (i & 3))) & 0xffu); }

struct FmtQ4_K {
    static constexpr int DW = 36, BYTES = 144, XR = 73;
    typedef int16_t ActSum;
    static PSN_DEV int d_per_col(int K) { return K >> 8; }
    static PSN_DEV int s_per_col(int K) { return K >> 4; }
    static PSN_DEV void load(const uint8_t *p, u32 (&w)[DW]) {
        const uint4 *q = reinterpret_cast<const uint4 *>(p);
        UNROLL for (int i = 0; i < 9; ++i) unpack4(q[i], &w[4 * i]);
    }
    static PSN_DEV void load_x(const ActQ<int16_t> &x, int K, int col, int c, u32 (&xr)[XR]) { load_x_q8_K(x, K, col, c, xr); }
    static PSN_DEV float dot(const u32 (&w)[DW], const u32 (&xr)[XR]) {
        u32 sc[2], mn[2];
        q4_K_scales(w[1], w[2], w[3], sc, mn);
        int isum = 0, msum = 0;
        /* the eight 32-element sub-block sums of the activation are pairs of 16-element group sums */
        UNROLL for (int i = 0; i < 8; ++i) {
            const u32 b = xr[65 + i];
            msum += byte_of(mn, i) * ((int)(int16_t)(b & 0xffffu) + ((int)b >> 16));
        }
        UNROLL for (int ch = 0; ch < 4; ++ch) {
            int sl = 0, sh = 0;
            UNROLL for (int i = 0; i < 8; ++i) {
                const u32 q = w[4 + 8 * ch + i];
                sl = dot4(q & 0x0f0f0f0fu, xr[16 * ch + i], sl);
                sh = dot4((q >> 4) & 0x0f0f0f0fu, xr[16 * ch + 8 + i], sh);
            }
            isum += byte_of(sc, 2 * ch) * sl + byte_of(sc, 2 * ch + 1) * sh;
        }
        const float dx = __uint_as_float(xr[64]);
        const float d = h2f_lo(w[0]) * dx, dm = h2f_hi(w[0]) * dx;
        return d * (float)isum - dm * (float)msum;
    }
    template <int SB>
    static PSN_DEV void deq32(const u32 (&w)[DW], float (&o)[32]) {
        u32 sc[2], mn[2];
        q4_K_scales(w[1], w[2], w[3], sc, mn);
        const float d = h2f_lo(w[0]) * (float)byte_of(sc, SB);
        const float mv = h2f_hi(w[0]) * (float)byte_of(mn, SB);
        constexpr int ch = SB >> 1, sh = (SB & 1) * 4;
        UNROLL for (int i = 0; i < 8; ++i) UNROLL for (int b = 0; b < 4; ++b)
            o[4 * i + b] = d * (float)((w[4 + 8 * ch + i] >> (8 * b + sh)) & 0xfu) - mv;
    }
};

/* Q5_K: chunk = one 176-byte super-block (11 dwordx4): dword 0 = fp16 d | fp16 dmin, dwords 1..3 =
 * Q4_K's scale/min field, dwords 4..11 = qh (bit j of byte l: fifth bit of element l of sub-block j),
 * dwords 12..43 = the nibble bytes laid out as Q4_K's.  Values 0..31 stay unsigned for the int8 dot. */
struct FmtQ5_K {
    static constexpr int DW = 44, BYTES = 176, XR = 73;
    typedef int16_t ActSum;
    static PSN_DEV int d_per_col(int K) { return K >> 8; }
    static PSN_DEV int s_per_col(int K) { return K >> 4; }
    static PSN_DEV void load(const uint8_t *p, u32 (&w)[DW]) {
        const uint4 *q = reinterpret_cast<const uint4 *>(p);
        UNROLL for (int i = 0; i < 11; ++i) unpack4(q[i], &w[4 * i]);
    }
    static PSN_DEV void load_x(const ActQ<int16_t> &x, int K, int col, int c, u32 (&xr)[XR]) { load_x_q8_K(x, K, col, c, xr); }
    static PSN_DEV float dot(const u32 (&w)[DW], const u32 (&xr)[XR]) {
        u32 sc[2], mn[2];
        q4_K_scales(w[1], w[2], w[3], sc, mn);
        int isum = 0, msum = 0;
        UNROLL for (int i = 0; i < 8; ++i) {
            const u32 b = xr[65 + i];
            msum += byte_of(mn, i) * ((int)(int16_t)(b & 0xffffu) + ((int)b >> 16));
        }
        UNROLL for (int ch = 0; ch < 4; ++ch) {
            int sl = 0, sh = 0;
            UNROLL for (int i = 0; i < 8; ++i) {
                const u32 q = w[12 + 8 * ch + i], h = w[4 + i];
                /* bit 2ch (2ch + 1) of every qh byte moves to bit 4 of the same byte; what a shift drags
                 * in from the neighbouring byte lands on other bits and is masked away */
                const u32 lo = (q & 0x0f0f0f0fu) | (((h >> (2 * ch)) << 4) & 0x10101010u);
                const u32 hi = ((q >> 4) & 0x0f0f0f0fu) | (((h >> (2 * ch + 1)) << 4) & 0x10101010u);
                sl = dot4(lo, xr[16 * ch + i], sl);
                sh = dot4(hi, xr[16 * ch + 8 + i], sh);
            }
            isum += byte_of(sc, 2 * ch) * sl + byte_of(sc, 2 * ch + 1) * sh;
        }
        const float dx = __uint_as_float(xr[64]);
        const float d = h2f_lo(w[0]) * dx, dm = h2f_hi(w[0]) * dx;
        return d * (float)isum - dm * (float)msum;
    }
    template <int SB>
    static PSN_DEV void deq32(const u32 (&w)[DW], float (&o)[32]) {
        u32 sc[2], mn[2];
        q4_K_scales(w[1], w[2], w[3], sc, mn);
        const float d = h2f_lo(w[0]) * (float)byte_of(sc, SB);
        const float mv = h2f_hi(w[0]) * (float)byte_of(mn, SB);
        constexpr int ch = SB >> 1, sh = (SB & 1) * 4;
        UNROLL for (int i = 0; i < 8; ++i) UNROLL for (int b = 0; b < 4; ++b) {
            const u32 v = ((w[12 + 8 * ch + i] >> (8 * b + sh)) & 0xfu) | (((w[4 + i] >> (8 * b + SB)) & 1u) << 4);
            o[4 * i + b] = d * (float)v - mv;
        }
    }
};

/* Q6_K: chunk = one 210-byte super-block at a 2-byte-aligned address: ql[128] | qh[64] |
 * int8 scales[16] | fp16 d.  13 dwordx4 loads cover bytes 0..207.  sum (q-32)*x =
 * sum q*x - 32*bsum per 16-element group keeps the 6-bit values unsigned. */
struct __attribute__((packed, aligned(2))) u4_a2 { u32 x, y, z, w; };

struct FmtQ6_K {
    static constexpr int DW = 53, BYTES = 210, XR = 73;
    typedef int16_t ActSum;
    static PSN_DEV int d_per_col(int K) { return K >> 8; }
    static PSN_DEV int s_per_col(int K) { return K >> 4; }
    static PSN_DEV void load(const uint8_t *p, u32 (&w)[DW]) {
        const u4_a2 *q = reinterpret_cast<const u4_a2 *>(p);
        UNROLL for (int i = 0; i < 13; ++i) {
            const u4_a2 v = q[i];
            w[4 * i] = v.x; w[4 * i + 1] = v.y; w[4 * i + 2] = v.z; w[4 * i + 3] = v.w;
        }
        w[52] = *reinterpret_cast<const unsigned short *>(p + 208);
    }
    static PSN_DEV void load_x(const ActQ<int16_t> &x, int K, int col, int c, u32 (&xr)[XR]) { load_x_q8_K(x, K, col, c, xr); }
    static PSN_DEV float dot(const u32 (&w)[DW], const u32 (&xr)[XR]) {
        int isum = 0;
        UNROLL for (int h = 0; h < 2; ++h) {
            int part[8];
            UNROLL for (int g = 0; g < 8; ++g) part[g] = 0;
            UNROLL for (int i = 0; i < 8; ++i) {      /* dword i holds l = 4i..4i+3 */
                const u32 A = w[16 * h + i], B = w[16 * h + 8 + i], H = w[32 + 8 * h + i];
                const u32 q1 = (A & 0x0f0f0f0fu) | ((H << 4) & 0x30303030u);
                const u32 q2 = (B & 0x0f0f0f0fu) | ((H << 2) & 0x30303030u);
                const u32 q3 = ((A >> 4) & 0x0f0f0f0fu) | (H & 0x30303030u);
                const u32 q4 = ((B >> 4) & 0x0f0f0f0fu) | ((H >> 2) & 0x30303030u);
                const int is = i >> 2;
                part[is + 0] = dot4(q1, xr[32 * h + i], part[is + 0]);
                part[is + 2] = dot4(q2, xr[32 * h + 8 + i], part[is + 2]);
                part[is + 4] = dot4(q3, xr[32 * h + 16 + i], part[is + 4]);
                part[is + 6] = dot4(q4, xr[32 * h + 24 + i], part[is + 6]);
            }
            UNROLL for (int g = 0; g < 8; ++g) {
                const int gi = 8 * h + g;             /* 16-element group of the super-block */
                const u32 sw = w[48 + (gi >> 2)];
                const int scale = (int)(int8_t)((sw >> (8 * (gi & 3))) & 0xffu);
                const u32 bw = xr[65 + (gi >> 1)];
                const int bsum = (gi & 1) ? ((int)bw >> 16) : (int)(int16_t)(bw & 0xffffu);
                isum += scale * (part[g] - 32 * bsum);
            }
        }
        return h2f_lo(w[52]) * __uint_as_float(xr[64]) * (float)isum;
    }
    template <int SB>
    static PSN_DEV void deq32(const u32 (&w)[DW], float (&o)[32]) {
        constexpr int h = SB >> 2, quarter = SB & 3;              /* elements 128h + 32*quarter + l */
        const float d = h2f_lo(w[52]);
        UNROLL for (int i = 0; i < 8; ++i) {
            const u32 L = w[16 * h + 8 * (quarter & 1) + i], H = w[32 + 8 * h + i];
            const u32 nib = (quarter < 2 ? L : (L >> 4)) & 0x0f0f0f0fu;
            const u32 top = ((H >> (2 * quarter)) & 0x03030303u) << 4;
            const u32 q = nib | top;
            const int gi = 8 * h + 2 * quarter + (i >> 2);
            const float ds = d * (float)(int)(int8_t)((w[48 + (gi >> 2)] >> (8 * (gi & 3))) & 0xffu);
            UNROLL for (int b = 0; b < 4; ++b) o[4 * i + b] = ds * (float)((int)((q >> (8 * b)) & 0xffu) - 32);
        }
    }
};

/* ------------------------------------------------------------------------------------------
 * Drivers.
 * ------------------------------------------------------------------------------------------ */

/* Scheme Q8.  A wave walks its work as (row set, chunk iteration) items.  Order of events: the
 * small activation loads are issued, then the first item's weight loads, then the activations are
 * staged (waiting only for their own loads) while the weights are still in flight.  At batch 1 the
 * lane's activation chunk stays in registers for as long as the chunk index does not change. */
template <typename F, int G, int R, int NB, int XSRC>
PSN_DEV void mv_q8(const psn_matvec_args &a) {
    typedef typename F::ActSum ST;
    const RowMap<G, R> m(a);
    PSN_DECLARE_SEGMENTS(a);
    const int K = a.K, C = K >> 8, iters = (C + G - 1) / G, stride = m.nwaves * m.ROWS;
    int row0 = m.wave * m.ROWS, it = 0;
    Stager<ST, XSRC> st;
    st.issue(a, F::d_per_col(K), F::s_per_col(K));
    u32 wa[R][F::DW];
    PSN_LOAD_ROWS(F, m, a, min(row0, a.N - 1), min(m.j, C - 1), wa);
    const ActQ<ST> x = st.finish(a);
    u32 xr[F::XR];
    int xc = -1;
    float acc[R][NB];
    UNROLL for (int r = 0; r < R; ++r) UNROLL for (int nb = 0; nb < NB; ++nb) acc[r][nb] = 0.f;

    auto advance = [&](int &r0, int &i) {
        if (++i == iters) { i = 0; r0 += stride; }
    };
    auto consume = [&](const u32 (&w)[R][F::DW], int r0, int i) {
        const int c = m.j + i * G;
        if (c < C) {
            UNROLL for (int nb = 0; nb < NB; ++nb) {
                const int col = nb < a.batch ? nb : a.batch - 1;
                if (NB > 1 || xc != c) { F::load_x(x, K, col, c, xr); xc = c; }
                UNROLL for (int r = 0; r < R; ++r) acc[r][nb] += F::dot(w[r], xr);
            }
        }
        if (i == iters - 1) {
            PSN_STORE_ROWS(m, acc, a, r0);
            UNROLL for (int r = 0; r < R; ++r) UNROLL for (int nb = 0; nb < NB; ++nb) acc[r][nb] = 0.f;
        }
    };

    bool pre = true;
    while (row0 < a.N) {
        if (!pre) { PSN_LOAD_ROWS(F, m, a, row0, min(m.j + it * G, C - 1), wa); }
        pre = false;
        consume(wa, row0, it);
        advance(row0, it);
    }
}

/* ------------------------------------------------------------------------------------------
 * Scheme Q8, streaming variant (batch 1, rows of at most G chunks).
 *
 * The weights do not pass through registers on their way in: every wave owns a ring of LDS buffers,
 * one pass (the 64/G rows a wave retires together, a contiguous byte range of the matrix) per
 * buffer, filled by 16-byte direct-to-LDS loads (lanes fetch consecutive 16-byte words, so one load
 * instruction covers 1 KB of contiguous row bytes).  A wave first puts all the passes its ring holds
 * in flight, then the workgroup stages the activations (their loads were issued even earlier, and
 * loads return in order), and from then on: wait for the oldest pass only, copy the lane's chunk
 * LDS -> registers, refill that buffer with the pass `ring` steps ahead, multiply.  The memory
 * system therefore always has ring x waves passes queued, independent of the arithmetic.
 *
 * Every wait in this kernel is written by hand.  The compiler's own wait insertion cannot tell the
 * ring buffers (dynamic LDS, run-time offsets) apart and would wait for ALL outstanding loads before
 * any LDS read; so LDS and the activation loads are accessed through inline assembly it does not
 * model, and the vmcnt / lgkmcnt waits are placed explicitly (loads complete in issue order, hence
 * "at most n younger loads outstanding" identifies the pass that has landed).
 * ------------------------------------------------------------------------------------------ */

/* a lane's chunk, LDS -> registers */
template <typename F> PSN_DEV void stream_load_chunk(u32 addr, u32 (&w)[F::DW]);
template <int NW, int I = 0> PSN_DEV void lds_read_seq(u32 addr, u32x4 (&v)[NW]) {
    if constexpr (I < NW) {
        v[I] = lds_read128<16 * I>(addr);                   /* offsets are instruction immediates */
        lds_read_seq<NW, I + 1>(addr, v);
    }
}
template <int NW> PSN_DEV void stream_read_words(u32 addr, u32 *w) {
    u32x4 v[NW];
    lds_read_seq<NW>(addr, v);
    lds_wait();
    tie(v);
    UNROLL for (int i = 0; i < NW; ++i) { w[4 * i] = v[i].x; w[4 * i + 1] = v[i].y; w[4 * i + 2] = v[i].z; w[4 * i + 3] = v[i].w; }
}

/* The staged activations of one chunk, LDS -> registers: 64 dwords of int8 and, for Q8_0 activations, 8
 * scales + 8 block sums, for Q8_K one scale + 16 int16 group sums (same register layout as load_x_*). */
template <typename ST, int XR> PSN_DEV void stream_load_x(u32 qs_addr, u32 d_addr, u32 s_addr, int j, u32 (&xr)[XR]) {
    u32x4 q[16], e[4];
    const u32 qa = qs_addr + (u32)j * 272u;
    lds_read_seq<16>(qa, q);
    u32 dk = 0;
    if constexpr (sizeof(ST) == 4) {
        e[0] = lds_read128<0>(d_addr + (u32)j * 32u);
        e[1] = lds_read128<16>(d_addr + (u32)j * 32u);
        e[2] = lds_read128<0>(s_addr + (u32)j * 32u);
        e[3] = lds_read128<16>(s_addr + (u32)j * 32u);
    } else {
        dk = lds_read32(d_addr + (u32)j * 4u);
        e[0] = lds_read128<0>(s_addr + (u32)j * 32u);
        e[1] = lds_read128<16>(s_addr + (u32)j * 32u);
        e[2] = e[3] = e[0];
    }
    lds_wait();
    tie(q);
    tie(e);
    tie1(dk);
    UNROLL for (int i = 0; i < 16; ++i) { xr[4 * i] = q[i].x; xr[4 * i + 1] = q[i].y; xr[4 * i + 2] = q[i].z; xr[4 * i + 3] = q[i].w; }
    if constexpr (sizeof(ST) == 4) {
        UNROLL for (int i = 0; i < 4; ++i) { xr[64 + 4 * i] = e[i].x; xr[65 + 4 * i] = e[i].y; xr[66 + 4 * i] = e[i].z; xr[67 + 4 * i] = e[i].w; }
    } else {
        xr[64] = dk;
        UNROLL for (int i = 0; i < 2; ++i) { xr[65 + 4 * i] = e[i].x; xr[66 + 4 * i] = e[i].y; xr[67 + 4 * i] = e[i].z; xr[68 + 4 * i] = e[i].w; }
    }
}

/* Activations into LDS for the streaming kernel (layout as in Stager: every 256-byte chunk of int8
 * followed by 16 bytes of padding, then the scales, then the sums).  issue() starts the global loads
 * (at most SLOTS 16-byte words per thread -- the host only picks this kernel when that suffices),
 * finish(pending) waits until at most `pending` younger loads are outstanding, quantizes if the input
 * was fp32 and writes LDS; the caller crosses the workgroup barrier. */
template <typename ST, int XSRC>
struct StreamStager {
    static constexpr int SLOTS = 8;
    static constexpr int NORM_SLOTS = 4;                     /* XSRC 3 holds x, the delta and the norm weights: half the reach */
    u32x4 t[SLOTS];
    u32x4 td, ts;
    u32x4 tdl[XSRC == 3 ? NORM_SLOTS : 1], tw[XSRC == 3 ? NORM_SLOTS : 1];
    int C, nthreads, n_qs, n_d, n_s;

    /* 16-byte word of the fp32 vector that slot i of this thread holds, or -1 */
    PSN_DEV int f32_word(int i) const {
        if constexpr (sizeof(ST) == 4) {
            const int idx = threadIdx.x + i * nthreads;
            return idx < C * 64 ? idx : -1;
        } else {
            const int sb = q8_K_block(i);
            return sb < C ? sb * 64 + (i & 3) * 16 + (int)(threadIdx.x & 15) : -1;
        }
    }
    /* Q8_K: sixteen lanes share a super-block and a wave works on four at a time -- slots 0..3 hold the four
     * quarters of the lane's block in the first round (blocks 0 .. 4 waves - 1 of the vector), slots 4..7 those
     * of the second round */
    PSN_DEV int q8_K_block(int i) const { return (i >> 2) * (nthreads >> 4) + (int)(threadIdx.x >> 4); }

    PSN_DEV void issue(const psn_matvec_args &a, int d_per_col, int s_per_col) {
        C = a.K >> 8;
        nthreads = a.threads;
        n_qs = C * 16;
        n_d = (d_per_col * 4 + 15) / 16;
        n_s = (s_per_col * (int)sizeof(ST) + 15) / 16;
        UNROLL for (int i = 0; i < SLOTS; ++i) t[i] = (u32x4)(0u);
        td = ts = (u32x4)(0u);
        if constexpr (XSRC == 1) {
            const uint4 *g_qs = reinterpret_cast<const uint4 *>(a.xqs);
            UNROLL for (int i = 0; i < SLOTS; ++i) {
                const int idx = threadIdx.x + i * nthreads;
                if (idx < n_qs) t[i] = global_read128(g_qs + idx);
            }
            if ((int)threadIdx.x < n_d) td = global_read128(reinterpret_cast<const uint4 *>(a.xd) + threadIdx.x);
            if ((int)threadIdx.x < n_s) ts = global_read128(reinterpret_cast<const uint4 *>(a.xs) + threadIdx.x);
        } else if constexpr (XSRC == 3) {
            const uint4 *x4 = reinterpret_cast<const uint4 *>(a.xf), *d4 = reinterpret_cast<const uint4 *>(a.x_delta);
            const uint4 *w4 = reinterpret_cast<const uint4 *>(a.norm_w);
            UNROLL for (int i = 0; i < NORM_SLOTS; ++i) {
                tdl[i] = tw[i] = (u32x4)(0u);
                const int idx = f32_word(i);
                if (idx >= 0) {
                    t[i] = global_read128(x4 + idx);
                    if (d4) tdl[i] = global_read128(d4 + idx);
                    tw[i] = global_read128(w4 + idx);
                }
            }
        } else {
            const float4 *x4 = reinterpret_cast<const float4 *>(a.xf);
            if constexpr (sizeof(ST) == 4) {
                const int total4 = C * 64;
                UNROLL for (int i = 0; i < SLOTS; ++i) {
                    const int idx = threadIdx.x + i * nthreads;
                    if (idx < total4) t[i] = global_read128(x4 + idx);
                }
            } else {
                UNROLL for (int i = 0; i < SLOTS; ++i) {
                    const int idx = f32_word(i);
                    if (idx >= 0) t[i] = global_read128(x4 + idx);
                }
            }
        }
    }

    /* XSRC 3: t <- (x + delta) * rsqrt(mean((x + delta)^2) + eps) * weight, in place; workgroup 0 also
     * stores x + delta.  `red` is the LDS address of one float per wave; crosses a workgroup barrier. */
    PSN_DEV void normalize(const psn_matvec_args &a, u32 red) {
        tie(tdl);
        tie(tw);
        float ss = 0.f;
        UNROLL for (int i = 0; i < NORM_SLOTS; ++i) {
            float h[4];
            UNROLL for (int e = 0; e < 4; ++e) {
                h[e] = __uint_as_float(t[i][e]) + __uint_as_float(tdl[i][e]);
                ss += h[e] * h[e];
                t[i][e] = __float_as_uint(h[e]);
            }
            const int idx = f32_word(i);
            if (blockIdx.x == 0 && a.h_out && idx >= 0) reinterpret_cast<float4 *>(a.h_out)[idx] = make_float4(h[0], h[1], h[2], h[3]);
        }
        ss = group_sum<64>(ss);
        const int wpb = nthreads >> 6;
        if ((threadIdx.x & 63) == 0) lds_write32(red + (threadIdx.x >> 6) * 4u, __float_as_uint(ss));
        lds_barrier();
        float total = 0.f;
        for (int w = 0; w < wpb; ++w) {
            u32 v = lds_read32(red + (u32)w * 4u);
            lds_wait();
            tie1(v);
            total += __uint_as_float(v);
        }
        const float scale = 1.0f / sqrtf(total / (float)a.K + a.eps);
        UNROLL for (int i = 0; i < NORM_SLOTS; ++i)
            UNROLL for (int e = 0; e < 4; ++e) t[i][e] = __float_as_uint(__uint_as_float(t[i][e]) * scale * __uint_as_float(tw[i][e]));
    }

    /* base: LDS byte address of the staging area; returns the addresses of the three fields */
    PSN_DEV void finish(const psn_matvec_args &a, int pending, u32 base, u32 &qs_addr, u32 &d_addr, u32 &s_addr) {
        qs_addr = base;
        d_addr = base + (u32)C * 272u;
        s_addr = d_addr + (u32)n_d * 16u;
        wait_vmcnt(pending);
        tie(t);
        asm volatile("" : "+v"(td), "+v"(ts));
        if constexpr (XSRC == 3) normalize(a, s_addr + (u32)n_s * 16u);
        const int lane = threadIdx.x & 63;
        if constexpr (XSRC == 1) {
            UNROLL for (int i = 0; i < SLOTS; ++i) {
                const int idx = threadIdx.x + i * nthreads;
                if (idx < n_qs) lds_write128(qs_addr + (u32)((idx >> 4) * 272 + (idx & 15) * 16), t[i]);
            }
            if ((int)threadIdx.x < n_d) lds_write128(d_addr + threadIdx.x * 16u, td);
            if ((int)threadIdx.x < n_s) lds_write128(s_addr + threadIdx.x * 16u, ts);
        } else if constexpr (sizeof(ST) == 4) {
            const int total4 = C * 64;
            UNROLL for (int k = 0; k < SLOTS; ++k) {
                const int i = threadIdx.x + k * nthreads;
                if (i < total4) {                                  /* whole 8-lane groups: K is a multiple of 256 */
                    u32 packed;
                    float d;
                    int sum;
                    q8_0_quant4(make_float4(__uint_as_float(t[k].x), __uint_as_float(t[k].y), __uint_as_float(t[k].z), __uint_as_float(t[k].w)), packed, d, sum);
                    lds_write32(qs_addr + (u32)((i >> 6) * 272 + (i & 63) * 4), packed);
                    if ((lane & 7) == 0) {
                        lds_write32(d_addr + (u32)(i >> 3) * 4u, __float_as_uint(d));
                        lds_write32(s_addr + (u32)(i >> 3) * 4u, (u32)sum);
                    }
                }
            }
        } else {
            const int l15 = lane & 15;
            UNROLL for (int r = 0; r < SLOTS / 4; ++r) {
                const int sb = q8_K_block(4 * r);
                /* wave-uniform: does the wave's first block of this round exist?  (XSRC 3 holds one round) */
                if ((XSRC != 3 || r == 0) && __builtin_amdgcn_readfirstlane(sb) < C) {
                    float4 v[4];
                    UNROLL for (int i = 0; i < 4; ++i)
                        v[i] = make_float4(__uint_as_float(t[4 * r + i].x), __uint_as_float(t[4 * r + i].y), __uint_as_float(t[4 * r + i].z), __uint_as_float(t[4 * r + i].w));
                    u32 packed[4];
                    float d;
                    int s16[4];
                    q8_K_quant_row16(v, lane, packed, d, s16);
                    if (sb < C) {
                        UNROLL for (int i = 0; i < 4; ++i) {
                            lds_write32(qs_addr + (u32)(sb * 272 + (i * 16 + l15) * 4), packed[i]);
                            if ((lane & 3) == 0) lds_write16(s_addr + (u32)(sb * 16 + i * 4 + (l15 >> 2)) * 2u, (u32)s16[i] & 0xffffu);
                        }
                        if (l15 == 0) lds_write32(d_addr + (u32)sb * 4u, __float_as_uint(d));
                    }
                }
            }
        }
    }
};

/* PAIR (two matrices of equal height, a gate and an up projection): the launch stores silu(W0 x) * (W1 x) into
 * y[0] instead of the two products.  A wave then works in units of two passes -- the same S rows of W0, then of
 * W1 -- keeps the first dot product in a register and stores one value per row. */
template <typename F, int G, int XSRC, int NSEG, bool PAIR = false>
PSN_DEV void mv_q8_stream(const psn_matvec_args &a) {
    static_assert(!PAIR || NSEG == 2, "a pair is two matrices");
    typedef typename F::ActSum ST;
    constexpr int S = 64 / G;                                /* rows per pass; every matrix holds a multiple of S rows */
    extern __shared__ uint4 psn_smem[];
    typedef __attribute__((address_space(3))) char lds_char;
    lds_char *const lds_ptr = (lds_char *)psn_smem;
    const u32 lds0 = (u32)(uintptr_t)lds_ptr;
    const int lane = threadIdx.x & 63, slot = lane / G, j = lane % G;
    const int wpb = a.threads >> 6;
    const int wib = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   /* wave-uniform, and the compiler should know it */
    const int K = a.K, C = K >> 8, N = a.N;
    const int rb = (int)a.row_bytes;                         /* bytes per row; a multiple of 16 */
    const int span = S * rb, nloads = (span + 1023) >> 10;   /* bytes and 1 KB load instructions per pass */
    const int wbuf = nloads << 10;
    const int ring = a.ring;                                 /* passes a wave keeps in flight (LDS buffers per wave) */
    const int npass = N / S;
    const int stride = a.blocks * wpb;
    const int p0 = blockIdx.x * wpb + wib;                   /* this wave's passes: p0, p0 + stride, ... */

    /* The activation loads go out before anything else is computed: they are small, and every load
     * issued later (the weights) completes after them. */
    StreamStager<ST, XSRC> st;
    st.issue(a, F::d_per_col(K), F::s_per_col(K));

    /* where the wave buffers start: right behind the staged activations (same arithmetic as the host) */
    const int n_d = (F::d_per_col(K) * 4 + 15) / 16, n_s = (F::s_per_col(K) * (int)sizeof(ST) + 15) / 16;
    const int stage_bytes = ((C * 272 + (n_d + n_s) * 16 + (XSRC == 3 ? 64 : 0) + 1023) >> 10) << 10;   /* XSRC 3: one float per wave behind the fields */
    const u32 ring_base = lds0 + (u32)stage_bytes + (u32)(wib * ring) * (u32)wbuf;

    /* a pass never straddles two matrices, so its rows are one contiguous range of one of them; the
     * four base pointers are pinned in scalar registers (the empty asm keeps the compiler from turning
     * the selects below back into an indexed load from a private copy of the arguments) */
    const uint8_t *W0 = a.W[0], *W1 = a.W[1], *W2 = a.W[2], *W3 = a.W[3];
    float *Y0 = a.y[0], *Y1 = a.y[1], *Y2 = a.y[2], *Y3 = a.y[3];
    int E0 = a.row_end[0], E1 = a.row_end[1], E2 = a.row_end[2];
    asm volatile("" : "+s"(W0), "+s"(W1), "+s"(W2), "+s"(W3), "+s"(Y0), "+s"(Y1), "+s"(Y2), "+s"(Y3), "+s"(E0), "+s"(E1), "+s"(E2));
    const int nseg = a.nseg;
    auto pass_base = [&](int pass, const uint8_t *&w, float *&y) {
        const int row0 = pass * S;
        const uint8_t *wb = W0;
        float *yb = Y0;
        int first = 0;
        /* with three or four matrices the count is compared at run time: the compiler turns a chain of
         * selects whose length it knows into an indexed load from a private (scratch) copy of the arguments */
        if (NSEG > 1 && row0 >= E0) { wb = W1; yb = Y1; first = E0; }
        if (NSEG > 2 && nseg > 2 && row0 >= E1) { wb = W2; yb = Y2; first = E1; }
        if (NSEG > 2 && nseg > 3 && row0 >= E2) { wb = W3; yb = Y3; first = E2; }
        w = wb + (int64_t)(row0 - first) * rb;
        y = yb + (row0 - first);
    };
    /* one pass into ring buffer `b`: exactly `nloads` load instructions of 1 KB each.  Lanes past the end
     * of the pass re-read its last 16 bytes (into the unused tail of the buffer) instead of being
     * masked off: a masked load costs a branch around every instruction. */
    auto issue = [&](int pass, int b) {
        const uint8_t *w;
        float *y;
        pass_base(pass, w, y);
        lds_char *dst = lds_ptr + (ring_base - lds0) + b * wbuf;
        int off = lane * 16;
        for (int l = 0; l < nloads; ++l) {
            __builtin_amdgcn_global_load_lds((const void *)(w + min(off, span - 16)), (__attribute__((address_space(3))) void *)dst, 16, 0, 0);
            off += 1024;
            dst += 1024;
        }
    };

    if constexpr (PAIR) {
        /* Units: unit u = passes u and nunits + u (rows u S .. of either matrix).  Whole rounds go wave by wave
         * like the passes below; the units of the last, partial round are dealt block by block (unit r of it to
         * block r % blocks, wave r / blocks), so that the compute units, each holding blocks a whole number of
         * compute units apart, end up with equal shares. */
        const int nunits = npass >> 1, full = nunits / stride, rem0 = full * stride;
        const int extra = wib * a.blocks + (int)blockIdx.x;
        const int mine = full + (rem0 + extra < nunits ? 1 : 0);          /* units of this wave */
        auto pass_of = [&](int i) {                                       /* the wave's i-th pass, i < 2 * mine */
            const int k = i >> 1, u = k < full ? p0 + k * stride : rem0 + extra;
            return (i & 1) ? nunits + u : u;
        };
        const int mypasses = 2 * mine;
        int issued = 0;
        for (; issued < ring && issued < mypasses; ++issued) issue(pass_of(issued), issued);
        u32 qs_addr, d_addr, s_addr;
        st.finish(a, issued * nloads, lds0, qs_addr, d_addr, s_addr);
        lds_barrier();
        u32 xr[F::XR];
        UNROLL for (int i = 0; i < F::XR; ++i) xr[i] = 0;
        if (j < C) stream_load_x<ST, F::XR>(qs_addr, d_addr, s_addr, j, xr);
        int b = 0;
        float gate = 0.f;
        for (int i = 0; i < mypasses; ++i) {
            wait_vmcnt((issued - i - 1) * nloads);
            u32 w[F::DW];
            UNROLL for (int q = 0; q < F::DW; ++q) w[q] = 0;
            if (j < C) stream_load_chunk<F>(ring_base + (u32)(b * wbuf + slot * rb + j * F::BYTES), w);
            else lds_wait();
            if (issued < mypasses) {
                issue(pass_of(issued), b);
                ++issued;
            }
            b = b + 1 == ring ? 0 : b + 1;
            float acc = (j < C) ? F::dot(w, xr) : 0.f;
            acc = group_sum<G>(acc);
            if (i & 1) {
                /* the expression of psn_swiglu, so that the fused launch returns its very floats */
                if (j == 0) Y0[(pass_of(i) - nunits) * S + slot] = gate / (1.f + __expf(-gate)) * acc;
            } else {
                gate = acc;
            }
        }
        return;
    }
    /* everything the ring holds goes in flight at once */
    int issued = 0;                                          /* passes issued so far */
    for (; issued < ring && p0 + issued * stride < npass; ++issued) issue(p0 + issued * stride, issued);
    u32 qs_addr, d_addr, s_addr;
    st.finish(a, issued * nloads, lds0, qs_addr, d_addr, s_addr);   /* waits for the activation loads only */
    lds_barrier();
    u32 xr[F::XR];
    UNROLL for (int i = 0; i < F::XR; ++i) xr[i] = 0;
    if (j < C) stream_load_x<ST, F::XR>(qs_addr, d_addr, s_addr, j, xr);
    int b = 0;                                               /* ring buffer of the current pass */
    for (int p = p0, done = 0; p < npass; p += stride, ++done) {
        /* the passes issued after this one (at most ring - 1) may stay in flight */
        wait_vmcnt((issued - done - 1) * nloads);
        u32 w[F::DW];
        UNROLL for (int q = 0; q < F::DW; ++q) w[q] = 0;
        if (j < C) stream_load_chunk<F>(ring_base + (u32)(b * wbuf + slot * rb + j * F::BYTES), w);
        else lds_wait();
        const uint8_t *wsrc;
        float *ydst;
        pass_base(p, wsrc, ydst);
        const int pn = p0 + issued * stride;
        if (pn < npass) {                                    /* this buffer is free again: refill it */
            issue(pn, b);
            ++issued;
        }
        b = b + 1 == ring ? 0 : b + 1;
        float acc = (j < C) ? F::dot(w, xr) : 0.f;
        acc = group_sum<G>(acc);
        if (j == 0) ydst[slot] = acc;
    }
}

template <> PSN_DEV void stream_load_chunk<FmtQ4_0>(u32 addr, u32 (&w)[FmtQ4_0::DW]) { stream_read_words<9>(addr, w); }
template <> PSN_DEV void stream_load_chunk<FmtQ4_K>(u32 addr, u32 (&w)[FmtQ4_K::DW]) { stream_read_words<9>(addr, w); }
template <> PSN_DEV void stream_load_chunk<FmtQ5_K>(u32 addr, u32 (&w)[FmtQ5_K::DW]) { stream_read_words<11>(addr, w); }
template <> PSN_DEV void stream_load_chunk<FmtQ8_0>(u32 addr, u32 (&w)[FmtQ8_0::DW]) { stream_read_words<17>(addr, w); }
/* Q6_K super-blocks are 210 bytes: a lane's chunk starts on an even byte, two bytes past a dword for every other
 * lane.  LDS reads that are not naturally aligned work and stall the LDS pipe (SQ_LDS_UNALIGNED_STALL: two thirds of
 * this kernel's cycles when the chunk was read as thirteen 16-byte words at its own address), so the 53 dwords are
 * read at the aligned address in front of the chunk, two per instruction, and shifted into place. */
template <int I> PSN_DEV void lds_read_pairs(u32 addr, u32x2 (&v)[26]) {
    if constexpr (I < 26) {
        v[I] = lds_read2_b32<2 * I, 2 * I + 1>(addr);
        lds_read_pairs<I + 1>(addr, v);
    }
}
template <> PSN_DEV void stream_load_chunk<FmtQ6_K>(u32 addr, u32 (&w)[FmtQ6_K::DW]) {
    const u32 sh = addr & 2u, a4 = addr - sh;
    u32x2 v[26];
    lds_read_pairs<0>(a4, v);
    u32 last = lds_read32o<208>(a4);
    lds_wait();
    UNROLL for (int i = 0; i < 26; ++i) asm volatile("" : "+v"(v[i]));
    tie1(last);
    UNROLL for (int k = 0; k < 52; ++k) {
        const u32 lo = v[k >> 1][k & 1], hi = k + 1 < 52 ? v[(k + 1) >> 1][(k + 1) & 1] : last;
        w[k] = __builtin_amdgcn_alignbyte(hi, lo, sh);
    }
    w[52] = __builtin_amdgcn_alignbyte(0u, last, sh) & 0xffffu;   /* the fp16 d: bytes 208, 209 of the chunk */
}

/* Scheme F32: weights dequantized to fp32 in registers, fp32 FMA against the fp32 activations.
 * XLDS: the activations are copied into LDS once per workgroup, every 1 KB chunk (256 floats) followed
 * by 16 bytes of padding so that lanes on neighbouring chunks read disjoint banks; a lane then streams
 * its chunk from LDS once per R rows instead of through the vector cache once per row. */
template <typename F, int SB, int R, int NB>
PSN_DEV void f32_step(const u32 (&w)[R][F::DW], const float *xbase, int col_stride, int chunk_off, int batch, float (&acc)[R][NB]) {
    float o[R][32];
    UNROLL for (int r = 0; r < R; ++r) F::template deq32<SB>(w[r], o[r]);
    UNROLL for (int nb = 0; nb < NB; ++nb) {
        const int col = nb < batch ? nb : batch - 1;
        const float4 *xp = reinterpret_cast<const float4 *>(xbase + (int64_t)col * col_stride + chunk_off + SB * 32);
        UNROLL for (int i = 0; i < 8; ++i) {
            const float4 x = xp[i];
            UNROLL for (int r = 0; r < R; ++r) {
                acc[r][nb] = __builtin_fmaf(o[r][4 * i + 0], x.x, acc[r][nb]);
                acc[r][nb] = __builtin_fmaf(o[r][4 * i + 1], x.y, acc[r][nb]);
                acc[r][nb] = __builtin_fmaf(o[r][4 * i + 2], x.z, acc[r][nb]);
                acc[r][nb] = __builtin_fmaf(o[r][4 * i + 3], x.w, acc[r][nb]);
            }
        }
    }
}

template <typename F, int G, int R, int NB, bool XLDS>
PSN_DEV void mv_f32(const psn_matvec_args &a) {
    const RowMap<G, R> m(a);
    PSN_DECLARE_SEGMENTS(a);
    const int K = a.K, C = K >> 8;
    const float *xbase = a.xf;
    int col_stride = K, chunk_stride = 256;
    u32 w[R][F::DW];
    int row0 = m.wave * m.ROWS;
    bool pre = false;
    if constexpr (XLDS) {
        extern __shared__ uint4 psn_smem[];
        /* first chunk's weights on their way before the activations are staged */
        pre = true;
        PSN_LOAD_ROWS(F, m, a, min(row0, a.N - 1), min(m.j, C - 1), w);
        const uint4 *g = reinterpret_cast<const uint4 *>(a.xf);
        const int n16 = a.batch * C * 64;                             /* 16-byte words of fp32 activations */
        for (int i = threadIdx.x; i < n16; i += a.threads) psn_smem[(i >> 6) * 65 + (i & 63)] = g[i];
        __syncthreads();
        xbase = reinterpret_cast<const float *>(psn_smem);
        chunk_stride = 260;
        col_stride = C * 260;
    }
    for (; row0 < a.N; row0 += m.nwaves * m.ROWS) {
        float acc[R][NB];
        UNROLL for (int r = 0; r < R; ++r) UNROLL for (int nb = 0; nb < NB; ++nb) acc[r][nb] = 0.f;
        for (int c = m.j; c < C; c += G) {
            if (!pre) { PSN_LOAD_ROWS(F, m, a, row0, c, w); }
            pre = false;
            const int off = c * chunk_stride;
            f32_step<F, 0>(w, xbase, col_stride, off, a.batch, acc);
            f32_step<F, 1>(w, xbase, col_stride, off, a.batch, acc);
            f32_step<F, 2>(w, xbase, col_stride, off, a.batch, acc);
            f32_step<F, 3>(w, xbase, col_stride, off, a.batch, acc);
            f32_step<F, 4>(w, xbase, col_stride, off, a.batch, acc);
            f32_step<F, 5>(w, xbase, col_stride, off, a.batch, acc);
            f32_step<F, 6>(w, xbase, col_stride, off, a.batch, acc);
            f32_step<F, 7>(w, xbase, col_stride, off, a.batch, acc);
        }
        PSN_STORE_ROWS(m, acc, a, row0);
    }
}

/* ------------------------------------------------------------------------------------------
 * Entry points.  Name = psn_mv_<fmt>_<scheme>_g<G>_r<R>_b<NB>[_lds|_xf]; the host picks one per shape
 * (_lds: quantized activations staged in LDS; _xf: fp32 activations quantized while staging).
 * Workgroups are 256 or 512 threads.
 * ------------------------------------------------------------------------------------------ */

#define PSN_Q8_KERNEL(fmt, F, G, R, NB)                                                                   \
    extern "C" __global__ void __launch_bounds__(512) psn_mv_##fmt##_q8_g##G##_r##R##_b##NB(const psn_matvec_args a) { \
        mv_q8<F, G, R, NB, 0>(a);                                                                         \
    }                                                                                                     \
    extern "C" __global__ void __launch_bounds__(512) psn_mv_##fmt##_q8_g##G##_r##R##_b##NB##_lds(const psn_matvec_args a) { \
        mv_q8<F, G, R, NB, 1>(a);                                                                         \
    }                                                                                                     \
    extern "C" __global__ void __launch_bounds__(512) psn_mv_##fmt##_q8_g##G##_r##R##_b##NB##_xf(const psn_matvec_args a) { \
        mv_q8<F, G, R, NB, 2>(a);                                                                         \
    }

/* streaming kernels: psn_mvs_<fmt>_q8_g<G>_{lds|xf}_s<matrices sharing the launch> */
#define PSN_STREAM_KERNEL(fmt, F, G, NSEG)                                                                \
    extern "C" __global__ void __launch_bounds__(512) psn_mvs_##fmt##_q8_g##G##_lds_s##NSEG(const psn_matvec_args a) { \
        mv_q8_stream<F, G, 1, NSEG>(a);                                                                   \
    }                                                                                                     \
    extern "C" __global__ void __launch_bounds__(512) psn_mvs_##fmt##_q8_g##G##_xf_s##NSEG(const psn_matvec_args a) {  \
        mv_q8_stream<F, G, 2, NSEG>(a);                                                                   \
    }
/* ... and with the residual add + RMSNorm folded into the staging of fp32 activations (_xn) */
#define PSN_STREAM_NORM_KERNEL(fmt, F, G, NSEG)                                                           \
    extern "C" __global__ void __launch_bounds__(512) psn_mvs_##fmt##_q8_g##G##_xn_s##NSEG(const psn_matvec_args a) {  \
        mv_q8_stream<F, G, 3, NSEG>(a);                                                                   \
    }
/* ... and, for a gate | up pair, with SwiGLU applied to the two products (_xnp) */
#define PSN_STREAM_PAIR_KERNEL(fmt, F, G)                                                                 \
    extern "C" __global__ void __launch_bounds__(512) psn_mvs_##fmt##_q8_g##G##_xnp_s2(const psn_matvec_args a) {      \
        mv_q8_stream<F, G, 3, 2, true>(a);                                                                \
    }
#define PSN_STREAM_NORM_G(fmt, F, G) PSN_STREAM_NORM_KERNEL(fmt, F, G, 1) PSN_STREAM_NORM_KERNEL(fmt, F, G, 2) PSN_STREAM_NORM_KERNEL(fmt, F, G, 3) \
    PSN_STREAM_PAIR_KERNEL(fmt, F, G)
#define PSN_STREAM_G(fmt, F, G) PSN_STREAM_KERNEL(fmt, F, G, 1) PSN_STREAM_KERNEL(fmt, F, G, 2) PSN_STREAM_KERNEL(fmt, F, G, 3) PSN_STREAM_KERNEL(fmt, F, G, 4)
#define PSN_STREAM_ALL(fmt, F) PSN_STREAM_G(fmt, F, 8) PSN_STREAM_G(fmt, F, 16) PSN_STREAM_G(fmt, F, 32) PSN_STREAM_G(fmt, F, 64) \
    PSN_STREAM_NORM_G(fmt, F, 8) PSN_STREAM_NORM_G(fmt, F, 16) PSN_STREAM_NORM_G(fmt, F, 32)

#define PSN_F32_KERNEL(fmt, F, G, R, NB)                                                                  \
    extern "C" __global__ void __launch_bounds__(512) psn_mv_##fmt##_f32_g##G##_r##R##_b##NB(const psn_matvec_args a) { \
        mv_f32<F, G, R, NB, false>(a);                                                                    \
    }                                                                                                     \
    extern "C" __global__ void __launch_bounds__(512) psn_mv_##fmt##_f32_g##G##_r##R##_b##NB##_lds(const psn_matvec_args a) { \
        mv_f32<F, G, R, NB, true>(a);                                                                     \
    }

#define PSN_Q8_ALL_G(fmt, F, R, NB) \
    PSN_Q8_KERNEL(fmt, F, 8, R, NB) PSN_Q8_KERNEL(fmt, F, 16, R, NB) PSN_Q8_KERNEL(fmt, F, 32, R, NB) PSN_Q8_KERNEL(fmt, F, 64, R, NB)
#define PSN_Q8_ALL(fmt, F)                                                                 \
    PSN_Q8_ALL_G(fmt, F, 1, 1)                                                             \
    PSN_Q8_ALL_G(fmt, F, 1, 2) PSN_Q8_ALL_G(fmt, F, 1, 4) PSN_Q8_ALL_G(fmt, F, 1, 8)

#define PSN_F32_ALL_G(fmt, F, R, NB) \
    PSN_F32_KERNEL(fmt, F, 8, R, NB) PSN_F32_KERNEL(fmt, F, 16, R, NB) PSN_F32_KERNEL(fmt, F, 32, R, NB) PSN_F32_KERNEL(fmt, F, 64, R, NB)
#define PSN_F32_ALL(fmt, F)                                                               \
    PSN_F32_ALL_G(fmt, F, 1, 1)                                                            \
    PSN_F32_ALL_G(fmt, F, 1, 2) PSN_F32_ALL_G(fmt, F, 1, 4) PSN_F32_ALL_G(fmt, F, 1, 8)

/* The build compiles this file once per format (-DPSN_BUILD_ONLY -DPSN_BUILD_<FMT>) so the four
 * code objects build in parallel; without PSN_BUILD_ONLY everything lands in one. */
#if !defined(PSN_BUILD_ONLY) || defined(PSN_BUILD_Q4_0)
PSN_Q8_ALL(q4_0, FmtQ4_0)
PSN_F32_ALL(q4_0, FmtQ4_0)
PSN_STREAM_ALL(q4_0, FmtQ4_0)
#endif
#if !defined(PSN_BUILD_ONLY) || defined(PSN_BUILD_Q8_0)
PSN_Q8_ALL(q8_0, FmtQ8_0)
PSN_F32_ALL(q8_0, FmtQ8_0)
PSN_STREAM_ALL(q8_0, FmtQ8_0)
#endif
#if !defined(PSN_BUILD_ONLY) || defined(PSN_BUILD_Q4_K)
PSN_Q8_ALL(q4_K, FmtQ4_K)
PSN_F32_ALL(q4_K, FmtQ4_K)
PSN_STREAM_ALL(q4_K, FmtQ4_K)
#endif
#if !defined(PSN_BUILD_ONLY) || defined(PSN_BUILD_Q5_K)
PSN_Q8_ALL(q5_K, FmtQ5_K)
PSN_F32_ALL(q5_K, FmtQ5_K)
PSN_STREAM_ALL(q5_K, FmtQ5_K)
#endif
#if !defined(PSN_BUILD_ONLY) || defined(PSN_BUILD_Q6_K)
PSN_Q8_ALL(q6_K, FmtQ6_K)
PSN_F32_ALL(q6_K, FmtQ6_K)
PSN_STREAM_ALL(q6_K, FmtQ6_K)
#endif
