/*
 * psn_args.h -- kernel argument blocks shared by the host library and the device code.
 * Every kernel takes exactly one of these structs by value, so the host passes a single
 * pointer through hipModuleLaunchKernel and the two sides cannot drift apart.
 */
#ifndef PSN_ARGS_H
#define PSN_ARGS_H

#include <stdint.h>

/* Device layout of quantized activations ("actq"), one region per field, row-major over batch:
 *   Q8_0 activations: int8 qs[B][K]; float d[B][K/32] (the fp16-rounded scale, widened);
 *                     int32 s[B][K/32] (sum of the block's 32 int8)
 *   Q8_K activations: int8 qs[B][K]; float d[B][K/256]; int16 bsums[B][K/16]
 * The three regions live in one allocation at offsets given by psn_actq_layout. */
struct psn_actq_layout {
    int64_t off_qs;   /* always 0 */
    int64_t off_d;
    int64_t off_s;    /* s (Q8_0) or bsums (Q8_K) */
    int64_t bytes;    /* total */
};

struct psn_quantize_args {
    const float *x;   /* [batch][K] */
    int8_t *qs;
    float *d;
    void *s;
    int32_t K;
    int32_t batch;
};

#define PSN_MAX_SEGMENTS 4

/* One launch walks the rows of up to four matrices that share K, the format and x as a single
 * concatenated row space: segment s owns rows [row_end[s-1], row_end[s]). */
struct psn_matvec_args {
    const uint8_t *W[PSN_MAX_SEGMENTS];   /* [N_s][row_bytes] GGUF blocks */
    float *y[PSN_MAX_SEGMENTS];           /* [batch][N_s] */
    int32_t row_end[PSN_MAX_SEGMENTS];    /* cumulative row counts */
    const int8_t *xqs;    /* scheme Q8: activation fields (see above) */
    const float *xd;
    const void *xs;
    const float *xf;      /* scheme F32: [batch][K] */
    int32_t N;            /* total rows = row_end[nseg-1] */
    int32_t K;
    int32_t batch;        /* live batch columns (<= the kernel's compiled NB) */
    int32_t nseg;
    int64_t row_bytes;
    int32_t threads;      /* launch geometry, passed in so that kernels never read the dispatch packet */
    int32_t blocks;
    int32_t ring;         /* streaming kernels: LDS buffers (passes in flight) per wave */
    float eps;            /* the fields below: streaming kernels that normalize while staging (_xn) */
    const float *x_delta; /* [K] added to xf before the norm (may be null) */
    const float *norm_w;  /* [K] RMSNorm weights */
    float *h_out;         /* [K] receives xf + x_delta, written by workgroup 0 (may be null; must not alias xf or x_delta) */
    int32_t kslices;      /* MFMA small-batch kernels: waves sharing a 16-row tile, each owning K / kslices of it */
    int32_t pad0;
};

struct psn_prefill_args {
    const uint8_t *W;     /* [N][row_bytes] GGUF blocks */
    const uint16_t *X;    /* fp16 [M][K] */
    float *Y;             /* [M][N] */
    int32_t M, N, K;
    int32_t ksplit;       /* K is cut into this many ranges; > 1: partial sums are added atomically into a zeroed Y */
    int64_t row_bytes;
};

/* weights -> fp16 fragments for the dense prefill kernel (psn_prefill_<fmt>_unpack) */
struct psn_unpack_args {
    const uint8_t *W;     /* [N][row_bytes] GGUF blocks */
    uint16_t *out;        /* fragment-major fp16: [ceil(N/32)][K/16][64 lanes][8] */
    int32_t N, K;
    int64_t row_bytes;
};

struct psn_fill_args {
    uint32_t *p;          /* 16-byte aligned */
    int64_t n16;          /* number of 16-byte words to zero */
};

struct psn_calib_args {
    const uint8_t *src;   /* 16-byte aligned */
    uint32_t *out;        /* one dword per wave (may be null) */
    int64_t bytes;
    int32_t depth;        /* psn_calib_read_lds: 1 KB LDS slots per wave */
    int32_t every_wg;     /* 1: every workgroup reads the whole range; 0: the workgroups share it */
};

/* psn_selftest_arith: float bit patterns lo .. hi (positive), one mismatch counter per checked identity */
struct psn_selftest_args {
    uint32_t lo, hi;
    unsigned long long *bad;   /* [PSN_SELFTEST_COUNTERS] */
};
#define PSN_SELFTEST_COUNTERS 8

/* decode-step glue kernels (psn_decode.hip) */
/* optional quantized output of an elementwise kernel: the three fields of the activation layout for
 * one row of n elements (qs null = not wanted); act_q8_K selects Q8_K (else Q8_0) */
struct psn_actq_out {
    int8_t *qs;
    float *d;
    void *s;
    int32_t act_q8_K, pad;
};
struct psn_norm_args {
    float *x;             /* [n], updated in place when delta != null */
    const float *delta;   /* optional residual to add first */
    const float *weight;  /* [n] */
    float *y;             /* [n] normalized output (may be null when only the quantized one is wanted) */
    int32_t n;
    float eps;
    struct psn_actq_out qout;
    float *x_out;         /* when set, x + delta goes here and x is left alone */
    int32_t keep_x;       /* nonzero: x + delta is stored nowhere unless x_out is set (x is never written) */
    int32_t pad1;
};
struct psn_rope_args {
    float *q;             /* [n_heads][head_dim], rotated in place */
    float *k;             /* [n_kv_heads][head_dim] */
    const float *v;       /* [n_kv_heads][head_dim] */
    void *k_cache;        /* fp16 [positions][n_kv_heads][head_dim] */
    void *v_cache;
    int32_t n_heads, n_kv_heads, head_dim, pos;
    float theta_base;
    int32_t pad;
};
struct psn_attn_args {
    const float *q;       /* [n_heads][128] */
    const void *k_cache;
    const void *v_cache;
    float *partial;       /* [n_heads][n_splits][130] */
    float *out;           /* [n_heads][128] (may be null when only the quantized one is wanted) */
    int32_t n_heads, n_kv_heads, n_ctx, n_splits;
    float scale;
    int32_t chunks;       /* psn_attn_partial(_rope)_long: 64-position chunks per split (the other kernels: one) */
    struct psn_actq_out qout;
    /* fused rotary + cache append (psn_attn_partial_rope): q and k_new are the raw projections of the
     * token at position n_ctx - 1; the kernel rotates them itself and stores k_new / v_new in the caches */
    const float *k_new;   /* [n_kv_heads][128] */
    const float *v_new;
    void *k_cache_w;
    void *v_cache_w;
    const float *rope_table;   /* [head_dim/2][2]: cos, sin of pos * theta^(-2i/head_dim), from psn_rope_table */
};
struct psn_rope_table_args {
    float *table;
    int32_t head_dim, pos;
    float theta_base;
    int32_t pad;
};
struct psn_swiglu_args {
    const float *gate, *up;
    float *out;           /* may be null when only the quantized output is wanted */
    int32_t n, pad;
    struct psn_actq_out qout;
};

#endif
