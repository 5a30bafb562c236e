/*
 * psn_decode.hip -- the small kernels that sit between the quantized matvecs of a Llama-style
 * decode step: residual add + RMSNorm, rotary embedding + KV-cache append, grouped-query attention
 * over the cache (split over the context, then combined), and SwiGLU.  They exist so that a whole
 * token step can run on the device and the matvec share of it can be measured; none of them is a
 * bandwidth-critical kernel (the KV cache read, 8 MB per layer at context 2048, is the largest).
 */
#include "psn_args.h"
#include "psn_device.h"

#define UNROLL _Pragma("unroll")

/* Quantizes the four consecutive values a thread holds (element index 4*i4 of a row) into the row's
 * activation fields.  Must be reached by whole waves: Q8_K needs the 64 lanes of a wave to hold one
 * 256-element super-block (i4 = 64*sb + lane), Q8_0 needs 8 adjacent lanes per 32-element block. */
PSN_DEV void quantize_out4(const psn_actq_out &q, int i4, float4 v) {
    const int lane = threadIdx.x & 63;
    u32 packed;
    float d;
    if (q.act_q8_K) {
        int s16;
        q8_K_quant_wave(v, lane, packed, d, s16);
        reinterpret_cast<u32 *>(q.qs)[i4] = packed;
        if ((lane & 3) == 0) reinterpret_cast<int16_t *>(q.s)[i4 >> 2] = (int16_t)s16;
        if (lane == 0) q.d[i4 >> 6] = d;
    } else {
        int sum;
        q8_0_quant4(v, packed, d, sum);
        reinterpret_cast<u32 *>(q.qs)[i4] = packed;
        if ((lane & 7) == 0) { q.d[i4 >> 3] = d; reinterpret_cast<int *>(q.s)[i4 >> 3] = sum; }
    }
}

/* sum over a workgroup of up to 1024 threads; every thread gets the result */
PSN_DEV float block_sum(float v, float *scratch) {
    v = group_sum<64>(v);
    const int wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    __syncthreads();                                   /* scratch may still be read from a previous call */
    if ((threadIdx.x & 63) == 0) scratch[wave] = v;
    __syncthreads();
    float t = 0.f;
    for (int i = 0; i < nw; ++i) t += scratch[i];
    return t;
}

/* x += delta (if delta != null);  y = x * rsqrt(mean(x^2) + eps) * weight.   One workgroup, n % 4 == 0.
 * Up to four float4 per thread stay in registers between the two passes and the norm weights are
 * requested before the reduction, so the kernel pays one memory round trip; longer vectors re-read x. */
extern "C" __global__ void __launch_bounds__(1024) psn_add_rmsnorm(const psn_norm_args a) {
    __shared__ float red[16];
    constexpr int KEEP = 4;
    const int n4 = a.n >> 2, nt = blockDim.x;
    const float4 *x4 = reinterpret_cast<const float4 *>(a.x);
    float4 *xo4 = reinterpret_cast<float4 *>(a.x_out ? a.x_out : a.x);      /* where x + delta goes */
    const bool store_sum = a.x_out != nullptr || (a.delta != nullptr && !a.keep_x);
    const float4 *d4 = reinterpret_cast<const float4 *>(a.delta);
    const float4 *w4 = reinterpret_cast<const float4 *>(a.weight);
    float4 *y4 = reinterpret_cast<float4 *>(a.y);
    const bool in_regs = n4 <= KEEP * nt;                          /* uniform */
    float4 v[KEEP], w[KEEP];
    float ss = 0.f;
    if (in_regs) {
        UNROLL for (int k = 0; k < KEEP; ++k) {
            const int i = threadIdx.x + k * nt;
            v[k] = make_float4(0.f, 0.f, 0.f, 0.f);
            w[k] = v[k];
            if (i < n4) {
                v[k] = x4[i];
                w[k] = w4[i];
                if (d4) {
                    const float4 d = d4[i];
                    v[k].x += d.x; v[k].y += d.y; v[k].z += d.z; v[k].w += d.w;
                }
                if (store_sum) xo4[i] = v[k];
            }
            ss += v[k].x * v[k].x + v[k].y * v[k].y + v[k].z * v[k].z + v[k].w * v[k].w;
        }
    } else {
        for (int i = threadIdx.x; i < n4; i += nt) {
            float4 t = x4[i];
            if (d4) {
                const float4 d = d4[i];
                t.x += d.x; t.y += d.y; t.z += d.z; t.w += d.w;
            }
            if (store_sum) xo4[i] = t;
            ss += t.x * t.x + t.y * t.y + t.z * t.z + t.w * t.w;
        }
    }
    ss = block_sum(ss, red);
    const float scale = 1.0f / sqrtf(ss / (float)a.n + a.eps);
    /* n is a multiple of 256 when a quantized output is asked for, so waves stay whole in these loops */
    if (in_regs) {
        UNROLL for (int k = 0; k < KEEP; ++k) {
            const int i = threadIdx.x + k * nt;
            if (i < n4) {
                const float4 o = make_float4(v[k].x * scale * w[k].x, v[k].y * scale * w[k].y, v[k].z * scale * w[k].z, v[k].w * scale * w[k].w);
                if (y4) y4[i] = o;
                if (a.qout.qs) quantize_out4(a.qout, i, o);
            }
        }
    } else {
        for (int i = threadIdx.x; i < n4; i += nt) {
            float4 t = store_sum ? xo4[i] : x4[i];
            const float4 ww = w4[i];
            if (!store_sum && d4) {                    /* the sum was not stored: add the delta again */
                const float4 d = d4[i];
                t.x += d.x; t.y += d.y; t.z += d.z; t.w += d.w;
            }
            const float4 o = make_float4(t.x * scale * ww.x, t.y * scale * ww.y, t.z * scale * ww.z, t.w * scale * ww.w);
            if (y4) y4[i] = o;
            if (a.qout.qs) quantize_out4(a.qout, i, o);
        }
    }
}

/* one rotary pair; explicit roundings so that every kernel that rotates gives the same bits */
PSN_DEV void rope_pair(float x0, float x1, float cs, float sn, float &r0, float &r1) {
    r0 = __fsub_rn(__fmul_rn(x0, cs), __fmul_rn(x1, sn));
    r1 = __fadd_rn(__fmul_rn(x0, sn), __fmul_rn(x1, cs));
}
PSN_DEV void rope_coeff(float theta_base, int head_dim, int pos, int i, float &cs, float &sn) {
    const float freq = powf(theta_base, -2.0f * (float)i / (float)head_dim);
    sincosf((float)pos * freq, &sn, &cs);
}

/* cos / sin of every rotary pair at one position: computed once per token, read by every layer */
extern "C" __global__ void __launch_bounds__(64) psn_rope_table(const psn_rope_table_args a) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= a.head_dim / 2) return;
    float cs, sn;
    rope_coeff(a.theta_base, a.head_dim, a.pos, i, cs, sn);
    a.table[2 * i] = cs;
    a.table[2 * i + 1] = sn;
}

/* Rotary embedding of q (in place) and k at position pos, pairs (2i, 2i+1), angle pos * base^(-2i/d);
 * k and v are appended to the fp16 cache row of that position.  One thread per pair. */
extern "C" __global__ void __launch_bounds__(256) psn_rope_kv_store(const psn_rope_args a) {
    const int half = a.head_dim >> 1;
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    const int nq = a.n_heads * half, nk = a.n_kv_heads * half;
    if (t >= nq + nk) return;
    const bool is_q = t < nq;
    const int idx = is_q ? t : t - nq;
    const int head = idx / half, i = idx % half;
    float sn, cs, r0, r1;
    rope_coeff(a.theta_base, a.head_dim, a.pos, i, cs, sn);
    float *src = (is_q ? a.q : a.k) + head * a.head_dim + 2 * i;
    rope_pair(src[0], src[1], cs, sn, r0, r1);
    if (is_q) {
        src[0] = r0;
        src[1] = r1;
    } else {
        const int64_t row = ((int64_t)a.pos * a.n_kv_heads + head) * a.head_dim + 2 * i;
        reinterpret_cast<f16 *>(a.k_cache)[row] = (f16)r0;
        reinterpret_cast<f16 *>(a.k_cache)[row + 1] = (f16)r1;
        const float *v = a.v + head * a.head_dim + 2 * i;
        reinterpret_cast<f16 *>(a.v_cache)[row] = (f16)v[0];
        reinterpret_cast<f16 *>(a.v_cache)[row + 1] = (f16)v[1];
    }
}

/* Attention of one new token over cache positions 0 .. n_ctx-1, head_dim 128.  Workgroup = (kv head,
 * 64 consecutive positions), one wave per query head of the group (up to 8).  The 64 K rows and 64 V
 * rows of the split (256 bytes each, n_kv_heads * 256 bytes apart) are fetched four rows per
 * instruction, 16 lanes per row, 16 bytes per lane: lane (q = lane >> 4, s = lane & 15) holds dims
 * 8 s .. 8 s + 7 of rows 4 j + q, j = 0 .. 15 -- every load instruction reads four contiguous 256-byte
 * rows, and all 32 of them are requested before anything is used (one memory round trip).  A row's
 * score is the sum over its 16 lanes of an eight-dim partial dot product (the lane's eight query dims
 * stay in registers); the softmax weights of a lane's own rows are then already in its registers, so
 * the weighted V sum needs no lane-to-lane traffic until the four row quarters are added at the end.
 * Rows past the context re-read the last valid one and get weight 0.  Writes the unnormalized partial
 * output plus (max, sum) per head and split. */
PSN_DEV float quarters_sum(float v) {                        /* over lanes l, l ^ 16, l ^ 32, l ^ 48 */
    v += __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(v), 0x401F));
    return v + __shfl_xor(v, 32, 64);
}
PSN_DEV float quarters_max(float v) {
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(v), 0x401F)));
    return fmaxf(v, __shfl_xor(v, 32, 64));
}
PSN_DEV u32 pack_h2(float lo, float hi) {
    const f16 a = (f16)lo, b = (f16)hi;
    return (u32)__builtin_bit_cast(unsigned short, a) | ((u32)__builtin_bit_cast(unsigned short, b) << 16);
}

template <bool ROPE>
PSN_DEV void attn_partial_body(const psn_attn_args &a) {
    constexpr int D = 128;
    __shared__ float qs[8][D];
    __shared__ uint4 knew_row[16];                            /* the new token's rotated key row, fp16 */
    const int lane = threadIdx.x & 63, g = threadIdx.x >> 6;
    const int quarter = lane >> 4, sub = lane & 15;
    const int kvh = blockIdx.x % a.n_kv_heads, split = blockIdx.x / a.n_kv_heads;
    const int group = a.n_heads / a.n_kv_heads;                  /* == blockDim.x / 64 */
    const int head = kvh * group + g;
    const int last = a.n_ctx - 1 - split * 64;                   /* last valid position of this split, >= 0 */
    uint4 kreg[16], vreg[16];
    {
        const int64_t row16 = (int64_t)a.n_kv_heads * (D / 8);   /* 16-byte words between positions */
        const uint4 *kb = reinterpret_cast<const uint4 *>(a.k_cache) + ((int64_t)split * 64 * a.n_kv_heads + kvh) * (D / 8) + sub;
        const uint4 *vb = reinterpret_cast<const uint4 *>(a.v_cache) + ((int64_t)split * 64 * a.n_kv_heads + kvh) * (D / 8) + sub;
        UNROLL for (int j = 0; j < 16; ++j) kreg[j] = kb[(int64_t)min(4 * j + quarter, last) * row16];
        UNROLL for (int j = 0; j < 16; ++j) vreg[j] = vb[(int64_t)min(4 * j + quarter, last) * row16];
    }
    if constexpr (ROPE) {
        /* lane i rotates pair i of this wave's query head; wave 0 of the split that owns the token's
         * position also rotates the new key row, rounds it to fp16 like a cached row, leaves it in LDS and
         * appends it to the cache */
        const float2 tc = *reinterpret_cast<const float2 *>(a.rope_table + 2 * lane);
        const float cs = tc.x, sn = tc.y;
        float r0, r1;
        const float2 qv = *reinterpret_cast<const float2 *>(a.q + head * D + 2 * lane);
        rope_pair(qv.x, qv.y, cs, sn, r0, r1);
        qs[g][2 * lane] = r0;
        qs[g][2 * lane + 1] = r1;
        if (g == 0 && split == ((a.n_ctx - 1) >> 6)) {
            const int pos = a.n_ctx - 1;
            const float2 kv = *reinterpret_cast<const float2 *>(a.k_new + kvh * D + 2 * lane);
            float k0, k1;
            rope_pair(kv.x, kv.y, cs, sn, k0, k1);
            const u32 packed = pack_h2(k0, k1);
            reinterpret_cast<u32 *>(knew_row)[lane] = packed;
            reinterpret_cast<u32 *>(reinterpret_cast<f16 *>(a.k_cache_w) + ((int64_t)pos * a.n_kv_heads + kvh) * D)[lane] = packed;
        }
    } else {
        qs[g][lane] = a.q[head * D + lane];
        qs[g][lane + 64] = a.q[head * D + lane + 64];
    }
    __syncthreads();
    if constexpr (ROPE) {
        /* the token's own position is not in the cache yet: the split that owns it takes the key row from
         * LDS (see above) and the value row from the fresh projection, rounded to fp16 like a cached row;
         * wave 0 appends the value row to the cache.  Rows behind the token's position were loaded from
         * cache rows that nothing has written yet: they get weight 0, but 0 * (a stale Inf/NaN pattern)
         * would still poison the sum, so they are replaced as well. */
        const int pos = a.n_ctx - 1;
        const bool own = split == (pos >> 6);                    /* uniform */
        const float4 va = *reinterpret_cast<const float4 *>(a.v_new + kvh * D + 8 * sub), vb4 = *reinterpret_cast<const float4 *>(a.v_new + kvh * D + 8 * sub + 4);
        uint4 vnew;
        vnew.x = pack_h2(va.x, va.y); vnew.y = pack_h2(va.z, va.w); vnew.z = pack_h2(vb4.x, vb4.y); vnew.w = pack_h2(vb4.z, vb4.w);
        int pl_v = own ? (pos & 63) : 64;                        /* first row to replace (64: none) */
        asm volatile("" : "+v"(pl_v));
        UNROLL for (int j = 0; j < 16; ++j) {
            const bool behind = 4 * j + quarter >= pl_v;
            vreg[j].x = behind ? vnew.x : vreg[j].x; vreg[j].y = behind ? vnew.y : vreg[j].y;
            vreg[j].z = behind ? vnew.z : vreg[j].z; vreg[j].w = behind ? vnew.w : vreg[j].w;
        }
        if (own) {
            const uint4 kn = knew_row[sub];
            UNROLL for (int j = 0; j < 16; ++j) {
                const bool mine = 4 * j + quarter == pl_v;
                kreg[j].x = mine ? kn.x : kreg[j].x; kreg[j].y = mine ? kn.y : kreg[j].y;
                kreg[j].z = mine ? kn.z : kreg[j].z; kreg[j].w = mine ? kn.w : kreg[j].w;
            }
            if (g == 0 && quarter == 0) reinterpret_cast<uint4 *>(reinterpret_cast<f16 *>(a.v_cache_w) + ((int64_t)pos * a.n_kv_heads + kvh) * D)[sub] = vnew;
        }
    }
    const float4 qa = *reinterpret_cast<const float4 *>(&qs[g][8 * sub]), qb = *reinterpret_cast<const float4 *>(&qs[g][8 * sub + 4]);
    float sc[16];
    float m = -INFINITY;
    UNROLL for (int j = 0; j < 16; ++j) {
        const u32 kw[4] = {kreg[j].x, kreg[j].y, kreg[j].z, kreg[j].w};
        float s = h2f_lo(kw[0]) * qa.x + h2f_hi(kw[0]) * qa.y + h2f_lo(kw[1]) * qa.z + h2f_hi(kw[1]) * qa.w;
        s += h2f_lo(kw[2]) * qb.x + h2f_hi(kw[2]) * qb.y + h2f_lo(kw[3]) * qb.z + h2f_hi(kw[3]) * qb.w;
        s = group_sum<16>(s);
        sc[j] = 4 * j + quarter <= last ? s * a.scale : -INFINITY;
        m = fmaxf(m, sc[j]);
    }
    m = quarters_max(m);                                         /* row 0 of the split is always live: m is finite */
    float sum = 0.f;
    float o[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    UNROLL for (int j = 0; j < 16; ++j) {
        const float w = 4 * j + quarter <= last ? __expf(sc[j] - m) : 0.f;
        sum += w;
        const u32 vw[4] = {vreg[j].x, vreg[j].y, vreg[j].z, vreg[j].w};
        UNROLL for (int t = 0; t < 4; ++t) {
            o[2 * t] += w * h2f_lo(vw[t]);
            o[2 * t + 1] += w * h2f_hi(vw[t]);
        }
    }
    sum = quarters_sum(sum);
    UNROLL for (int t = 0; t < 8; ++t) o[t] = quarters_sum(o[t]);
    float *dst = a.partial + ((int64_t)head * a.n_splits + split) * (D + 2);
    if (quarter == 0) {
        /* (D + 2) floats per split: rows start on 8-byte, not 16-byte, boundaries */
        UNROLL for (int t = 0; t < 4; ++t) *reinterpret_cast<float2 *>(dst + 8 * sub + 2 * t) = make_float2(o[2 * t], o[2 * t + 1]);
    }
    if (lane == 0) { dst[D] = m; dst[D + 1] = sum; }
}

/* Long contexts: a split is a.chunks chunks of 64 positions, walked sixteen positions at a time (row 4 j + quarter of
 * a step in lane quarter `quarter`, j = 0 .. 3) with the next step's K and V rows already requested while the
 * current ones are multiplied, and a running (max, sum, output) per lane quarter in the manner of a streaming
 * softmax: the cross-lane sums and the partial store, which the kernel above pays per 64 positions, are paid once
 * per split, and a workgroup's loads overlap its arithmetic.  Same partial format, same combine kernel. */
template <bool ROPE>
PSN_DEV void attn_partial_long_body(const psn_attn_args &a) {
    constexpr int D = 128;
    __shared__ float qs[8][D];
    __shared__ uint4 knew_row[16];
    const int lane = threadIdx.x & 63, g = threadIdx.x >> 6;
    const int quarter = lane >> 4, sub = lane & 15;
    const int kvh = blockIdx.x % a.n_kv_heads, split = blockIdx.x / a.n_kv_heads;
    const int group = a.n_heads / a.n_kv_heads;
    const int head = kvh * group + g;
    const int pos_last = a.n_ctx - 1;
    const int p_begin = split * a.chunks * 64;                   /* < n_ctx: the host launches no empty split */
    const int p_end = min(p_begin + a.chunks * 64, a.n_ctx);     /* one past the split's last valid position */
    const int nsteps = (p_end - p_begin + 15) >> 4;
    const bool own = ROPE && pos_last >= p_begin && pos_last < p_end;   /* uniform: the split that holds the token's position */
    const int64_t row16 = (int64_t)a.n_kv_heads * (D / 8);       /* 16-byte words between positions */
    const uint4 *kb = reinterpret_cast<const uint4 *>(a.k_cache) + (int64_t)kvh * (D / 8) + sub;
    const uint4 *vb = reinterpret_cast<const uint4 *>(a.v_cache) + (int64_t)kvh * (D / 8) + sub;
    auto fetch = [&](int it, uint4 (&k)[4], uint4 (&v)[4]) {
        UNROLL for (int j = 0; j < 4; ++j) {
            const int p = min(p_begin + 16 * it + 4 * j + quarter, p_end - 1);
            k[j] = kb[(int64_t)p * row16];
            v[j] = vb[(int64_t)p * row16];
        }
    };
    uint4 ka[4], va[4], kbuf[4], vbuf[4];
    fetch(0, ka, va);
    uint4 vnew = make_uint4(0, 0, 0, 0);
    if constexpr (ROPE) {
        const float2 tc = *reinterpret_cast<const float2 *>(a.rope_table + 2 * lane);
        const float cs = tc.x, sn = tc.y;
        float r0, r1;
        const float2 qv = *reinterpret_cast<const float2 *>(a.q + head * D + 2 * lane);
        rope_pair(qv.x, qv.y, cs, sn, r0, r1);
        qs[g][2 * lane] = r0;
        qs[g][2 * lane + 1] = r1;
        if (g == 0 && own) {
            const float2 kv = *reinterpret_cast<const float2 *>(a.k_new + kvh * D + 2 * lane);
            float k0, k1;
            rope_pair(kv.x, kv.y, cs, sn, k0, k1);
            const u32 packed = pack_h2(k0, k1);
            reinterpret_cast<u32 *>(knew_row)[lane] = packed;
            reinterpret_cast<u32 *>(reinterpret_cast<f16 *>(a.k_cache_w) + ((int64_t)pos_last * a.n_kv_heads + kvh) * D)[lane] = packed;
        }
        const float4 x0 = *reinterpret_cast<const float4 *>(a.v_new + kvh * D + 8 * sub), x1 = *reinterpret_cast<const float4 *>(a.v_new + kvh * D + 8 * sub + 4);
        vnew.x = pack_h2(x0.x, x0.y); vnew.y = pack_h2(x0.z, x0.w); vnew.z = pack_h2(x1.x, x1.y); vnew.w = pack_h2(x1.z, x1.w);
        if (own && g == 0 && quarter == 0)
            reinterpret_cast<uint4 *>(reinterpret_cast<f16 *>(a.v_cache_w) + ((int64_t)pos_last * a.n_kv_heads + kvh) * D)[sub] = vnew;
    } else {
        qs[g][lane] = a.q[head * D + lane];
        qs[g][lane + 64] = a.q[head * D + lane + 64];
    }
    __syncthreads();
    uint4 knew = make_uint4(0, 0, 0, 0);
    if (own) knew = knew_row[sub];
    const float4 qa = *reinterpret_cast<const float4 *>(&qs[g][8 * sub]), qb = *reinterpret_cast<const float4 *>(&qs[g][8 * sub + 4]);
    float m_run = -INFINITY, l_run = 0.f;
    float o[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    auto step = [&](int it, uint4 (&k)[4], uint4 (&v)[4]) {
        float sc[4];
        float m_new = m_run;
        UNROLL for (int j = 0; j < 4; ++j) {
            const int p = p_begin + 16 * it + 4 * j + quarter;
            if (own) {
                /* the token's own row is not in the cache yet (its key comes from LDS, its value from the fresh
                 * projection, both rounded to fp16 like a cached row); rows behind it were loaded from the row at its
                 * position, which nothing has written: they get weight 0, but 0 * (a stale Inf / NaN pattern) would
                 * still poison the sum, so their values are replaced as well */
                const bool mine = p == pos_last, behind = p >= pos_last;
                k[j].x = mine ? knew.x : k[j].x; k[j].y = mine ? knew.y : k[j].y; k[j].z = mine ? knew.z : k[j].z; k[j].w = mine ? knew.w : k[j].w;
                v[j].x = behind ? vnew.x : v[j].x; v[j].y = behind ? vnew.y : v[j].y; v[j].z = behind ? vnew.z : v[j].z; v[j].w = behind ? vnew.w : v[j].w;
            }
            const u32 kw[4] = {k[j].x, k[j].y, k[j].z, k[j].w};
            float s = h2f_lo(kw[0]) * qa.x + h2f_hi(kw[0]) * qa.y + h2f_lo(kw[1]) * qa.z + h2f_hi(kw[1]) * qa.w;
            s += h2f_lo(kw[2]) * qb.x + h2f_hi(kw[2]) * qb.y + h2f_lo(kw[3]) * qb.z + h2f_hi(kw[3]) * qb.w;
            s = group_sum<16>(s);
            sc[j] = p < p_end ? s * a.scale : -INFINITY;
            m_new = fmaxf(m_new, sc[j]);
        }
        /* a quarter that has seen no valid row yet keeps max = -inf: subtract 0 then, every weight is exp(-inf) = 0 */
        const float m_use = m_new == -INFINITY ? 0.f : m_new;
        const float r = __expf(m_run - m_use);
        l_run *= r;
        UNROLL for (int t = 0; t < 8; ++t) o[t] *= r;
        UNROLL for (int j = 0; j < 4; ++j) {
            const float w = __expf(sc[j] - m_use);
            l_run += w;
            const u32 vw[4] = {v[j].x, v[j].y, v[j].z, v[j].w};
            UNROLL for (int t = 0; t < 4; ++t) {
                o[2 * t] += w * h2f_lo(vw[t]);
                o[2 * t + 1] += w * h2f_hi(vw[t]);
            }
        }
        m_run = m_new;
    };
    for (int it = 0; it < nsteps; it += 2) {
        if (it + 1 < nsteps) fetch(it + 1, kbuf, vbuf);
        step(it, ka, va);
        if (it + 1 < nsteps) {
            if (it + 2 < nsteps) fetch(it + 2, ka, va);
            step(it + 1, kbuf, vbuf);
        }
    }
    /* the four quarters' running states meet: common maximum (row p_begin is valid, so it is finite), rescaled sums */
    const float m = quarters_max(m_run);
    const float f = __expf(m_run - m);
    const float sum = quarters_sum(l_run * f);
    UNROLL for (int t = 0; t < 8; ++t) o[t] = quarters_sum(o[t] * f);
    float *dst = a.partial + ((int64_t)head * a.n_splits + split) * (D + 2);
    if (quarter == 0) {
        UNROLL for (int t = 0; t < 4; ++t) *reinterpret_cast<float2 *>(dst + 8 * sub + 2 * t) = make_float2(o[2 * t], o[2 * t + 1]);
    }
    if (lane == 0) { dst[D] = m; dst[D + 1] = sum; }
}

/* The same for groups of four or eight query heads per kv head, with the roles turned: a wave takes sixteen of a
 * step's 64 positions for four heads (HB blocks of four heads, four waves each) instead of all 64 for one head.  Every K and V row is then fetched by
 * one wave only (a quarter of the requests, four times the distinct bytes in flight per compute unit, which is
 * what bounds a long context), converted to fp32 once and used four times.  The four waves' running states meet
 * through LDS at the end of the split. */
template <bool ROPE, int HB>
PSN_DEV void attn_partial_long4_body(const psn_attn_args &a) {
    constexpr int D = 128, H = 4, GROUP = H * HB;
    __shared__ float qs[GROUP][D];
    __shared__ uint4 knew_row[16];
    __shared__ float part_o[HB][4][H][D];
    __shared__ float part_ml[HB][4][H][2];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int w = wave & 3, hb = wave >> 2;                      /* position quarter of a step, block of four heads */
    const int quarter = lane >> 4, sub = lane & 15;
    const int kvh = blockIdx.x % a.n_kv_heads, split = blockIdx.x / a.n_kv_heads;
    const int pos_last = a.n_ctx - 1;
    const int p_begin = split * a.chunks * 64;
    const int p_end = min(p_begin + a.chunks * 64, a.n_ctx);
    const int nsteps = (p_end - p_begin + 63) >> 6;
    const bool own = ROPE && pos_last >= p_begin && pos_last < p_end;
    const int64_t row16 = (int64_t)a.n_kv_heads * (D / 8);
    const uint4 *kb = reinterpret_cast<const uint4 *>(a.k_cache) + (int64_t)kvh * (D / 8) + sub;
    const uint4 *vb = reinterpret_cast<const uint4 *>(a.v_cache) + (int64_t)kvh * (D / 8) + sub;
    auto fetch = [&](int it, uint4 (&k)[4], uint4 (&v)[4]) {
        UNROLL for (int j = 0; j < 4; ++j) {
            const int p = min(p_begin + 64 * it + 16 * w + 4 * j + quarter, p_end - 1);
            k[j] = kb[(int64_t)p * row16];
            v[j] = vb[(int64_t)p * row16];
        }
    };
    uint4 ka[4], va[4], kbuf[4], vbuf[4];
    fetch(0, ka, va);
    uint4 vnew = make_uint4(0, 0, 0, 0);
    if constexpr (ROPE) {
        /* wave i rotates query head i of the group; wave 0 of the split that owns the token's position the new key */
        const float2 tc = *reinterpret_cast<const float2 *>(a.rope_table + 2 * lane);
        const float cs = tc.x, sn = tc.y;
        float r0, r1;
        const float2 qv = *reinterpret_cast<const float2 *>(a.q + (kvh * GROUP + wave) * D + 2 * lane);
        rope_pair(qv.x, qv.y, cs, sn, r0, r1);
        qs[wave][2 * lane] = r0;
        qs[wave][2 * lane + 1] = r1;
        if (wave == 0 && own) {
            const float2 kv = *reinterpret_cast<const float2 *>(a.k_new + kvh * D + 2 * lane);
            float k0, k1;
            rope_pair(kv.x, kv.y, cs, sn, k0, k1);
            const u32 packed = pack_h2(k0, k1);
            reinterpret_cast<u32 *>(knew_row)[lane] = packed;
            reinterpret_cast<u32 *>(reinterpret_cast<f16 *>(a.k_cache_w) + ((int64_t)pos_last * a.n_kv_heads + kvh) * D)[lane] = packed;
        }
        const float4 x0 = *reinterpret_cast<const float4 *>(a.v_new + kvh * D + 8 * sub), x1 = *reinterpret_cast<const float4 *>(a.v_new + kvh * D + 8 * sub + 4);
        vnew.x = pack_h2(x0.x, x0.y); vnew.y = pack_h2(x0.z, x0.w); vnew.z = pack_h2(x1.x, x1.y); vnew.w = pack_h2(x1.z, x1.w);
        if (own && wave == 0 && quarter == 0)
            reinterpret_cast<uint4 *>(reinterpret_cast<f16 *>(a.v_cache_w) + ((int64_t)pos_last * a.n_kv_heads + kvh) * D)[sub] = vnew;
    } else {
        qs[wave][lane] = a.q[(kvh * GROUP + wave) * D + lane];
        qs[wave][lane + 64] = a.q[(kvh * GROUP + wave) * D + lane + 64];
    }
    __syncthreads();
    uint4 knew = make_uint4(0, 0, 0, 0);
    if (own) knew = knew_row[sub];
    float q[H][8];
    UNROLL for (int h = 0; h < H; ++h) {
        const float4 lo = *reinterpret_cast<const float4 *>(&qs[hb * H + h][8 * sub]), hi = *reinterpret_cast<const float4 *>(&qs[hb * H + h][8 * sub + 4]);
        q[h][0] = lo.x; q[h][1] = lo.y; q[h][2] = lo.z; q[h][3] = lo.w; q[h][4] = hi.x; q[h][5] = hi.y; q[h][6] = hi.z; q[h][7] = hi.w;
    }
    float m_run[H], l_run[H], o[H][8];
    UNROLL for (int h = 0; h < H; ++h) {
        m_run[h] = -INFINITY;
        l_run[h] = 0.f;
        UNROLL for (int t = 0; t < 8; ++t) o[h][t] = 0.f;
    }
    auto step = [&](int it, uint4 (&k)[4], uint4 (&v)[4]) {
        float sc[H][4];
        UNROLL for (int j = 0; j < 4; ++j) {
            const int p = p_begin + 64 * it + 16 * w + 4 * j + quarter;
            if (own) {                                           /* see attn_partial_long_body */
                const bool mine = p == pos_last, behind = p >= pos_last;
                k[j].x = mine ? knew.x : k[j].x; k[j].y = mine ? knew.y : k[j].y; k[j].z = mine ? knew.z : k[j].z; k[j].w = mine ? knew.w : k[j].w;
                v[j].x = behind ? vnew.x : v[j].x; v[j].y = behind ? vnew.y : v[j].y; v[j].z = behind ? vnew.z : v[j].z; v[j].w = behind ? vnew.w : v[j].w;
            }
            const u32 kw[4] = {k[j].x, k[j].y, k[j].z, k[j].w};
            float kf[8];
            UNROLL for (int t = 0; t < 4; ++t) { kf[2 * t] = h2f_lo(kw[t]); kf[2 * t + 1] = h2f_hi(kw[t]); }
            UNROLL for (int h = 0; h < H; ++h) {
                /* the order of the one-head kernels: two sums of four products */
                float s = kf[0] * q[h][0] + kf[1] * q[h][1] + kf[2] * q[h][2] + kf[3] * q[h][3];
                s += kf[4] * q[h][4] + kf[5] * q[h][5] + kf[6] * q[h][6] + kf[7] * q[h][7];
                s = group_sum<16>(s);
                sc[h][j] = p < p_end ? s * a.scale : -INFINITY;
            }
        }
        float m_use[H];
        UNROLL for (int h = 0; h < H; ++h) {
            const float m_new = fmaxf(fmaxf(m_run[h], fmaxf(sc[h][0], sc[h][1])), fmaxf(sc[h][2], sc[h][3]));
            m_use[h] = m_new == -INFINITY ? 0.f : m_new;
            const float r = __expf(m_run[h] - m_use[h]);
            l_run[h] *= r;
            UNROLL for (int t = 0; t < 8; ++t) o[h][t] *= r;
            m_run[h] = m_new;
        }
        UNROLL for (int j = 0; j < 4; ++j) {
            const u32 vw[4] = {v[j].x, v[j].y, v[j].z, v[j].w};
            float vf[8];
            UNROLL for (int t = 0; t < 4; ++t) { vf[2 * t] = h2f_lo(vw[t]); vf[2 * t + 1] = h2f_hi(vw[t]); }
            UNROLL for (int h = 0; h < H; ++h) {
                const float wt = __expf(sc[h][j] - m_use[h]);
                l_run[h] += wt;
                UNROLL for (int t = 0; t < 8; ++t) o[h][t] += wt * vf[t];
            }
        }
    };
    for (int it = 0; it < nsteps; it += 2) {
        if (it + 1 < nsteps) fetch(it + 1, kbuf, vbuf);
        step(it, ka, va);
        if (it + 1 < nsteps) {
            if (it + 2 < nsteps) fetch(it + 2, ka, va);
            step(it + 1, kbuf, vbuf);
        }
    }
    /* quarters meet inside the wave, waves through LDS (a wave that saw no valid position contributes weight 0) */
    UNROLL for (int h = 0; h < H; ++h) {
        const float m = quarters_max(m_run[h]);
        const float mu = m == -INFINITY ? 0.f : m;
        const float f = __expf(m_run[h] - mu);
        const float l = quarters_sum(l_run[h] * f);
        UNROLL for (int t = 0; t < 8; ++t) o[h][t] = quarters_sum(o[h][t] * f);
        if (quarter == 0) {
            UNROLL for (int t = 0; t < 8; ++t) part_o[hb][w][h][8 * sub + t] = o[h][t];
        }
        if (lane == 0) { part_ml[hb][w][h][0] = m; part_ml[hb][w][h][1] = l; }
    }
    __syncthreads();
    {
        const int h = w;                                         /* wave (hb, w) finishes head w of its block */
        float mw[4], M = -INFINITY;
        UNROLL for (int i = 0; i < 4; ++i) { mw[i] = part_ml[hb][i][h][0]; M = fmaxf(M, mw[i]); }
        float L = 0.f, o0 = 0.f, o1 = 0.f;
        UNROLL for (int i = 0; i < 4; ++i) {
            const float f = __expf(mw[i] - M);                   /* M is finite: wave 0 saw position p_begin */
            L += part_ml[hb][i][h][1] * f;
            o0 += part_o[hb][i][h][2 * lane] * f;
            o1 += part_o[hb][i][h][2 * lane + 1] * f;
        }
        float *dst = a.partial + ((int64_t)(kvh * GROUP + hb * H + h) * a.n_splits + split) * (D + 2);
        *reinterpret_cast<float2 *>(dst + 2 * lane) = make_float2(o0, o1);
        if (lane == 0) { dst[D] = M; dst[D + 1] = L; }
    }
}

extern "C" __global__ void __launch_bounds__(512) psn_attn_partial(const psn_attn_args a) { attn_partial_body<false>(a); }
/* the same with the rotary embedding of q and k and the KV-cache append of the new token folded in */
extern "C" __global__ void __launch_bounds__(512) psn_attn_partial_rope(const psn_attn_args a) { attn_partial_body<true>(a); }
extern "C" __global__ void __launch_bounds__(512) psn_attn_partial_long(const psn_attn_args a) { attn_partial_long_body<false>(a); }
extern "C" __global__ void __launch_bounds__(512) psn_attn_partial_rope_long(const psn_attn_args a) { attn_partial_long_body<true>(a); }
extern "C" __global__ void __launch_bounds__(256) psn_attn_partial_long4(const psn_attn_args a) { attn_partial_long4_body<false, 1>(a); }
extern "C" __global__ void __launch_bounds__(256) psn_attn_partial_rope_long4(const psn_attn_args a) { attn_partial_long4_body<true, 1>(a); }
extern "C" __global__ void __launch_bounds__(512) psn_attn_partial_long8(const psn_attn_args a) { attn_partial_long4_body<false, 2>(a); }
extern "C" __global__ void __launch_bounds__(512) psn_attn_partial_rope_long8(const psn_attn_args a) { attn_partial_long4_body<true, 2>(a); }

/* out[head][d] = sum_s o_s[d] e^(m_s - M) / sum_s l_s e^(m_s - M).  One wave per head, two heads per
 * workgroup; a lane owns two output dims.  The splits are taken 32 at a time and everything a wave needs
 * of them -- the (max, sum) pairs and its two dims of every partial output -- is requested before
 * anything is used, so 32 splits cost one trip to memory; the running sums are rescaled when the maximum
 * moves.  With a quantized output the two heads (256 consecutive values, one Q8_K super-block or eight
 * Q8_0 blocks) are regrouped through LDS into the four-values-per-lane layout the quantizers work on. */
extern "C" __global__ void __launch_bounds__(128) psn_attn_combine(const psn_attn_args a) {
    constexpr int D = 128;
    __shared__ float regroup[2 * D];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int head = min(2 * (int)blockIdx.x + w, a.n_heads - 1);      /* an odd head count: the spare wave repeats the last head */
    const float *base = a.partial + (int64_t)head * a.n_splits * (D + 2);
    float M = -INFINITY, n0 = 0.f, n1 = 0.f, den = 0.f;
    for (int c0 = 0; c0 < a.n_splits; c0 += 32) {
        const int cnt = min(32, a.n_splits - c0);
        const float2 ml = *reinterpret_cast<const float2 *>(base + (int64_t)(c0 + min(lane, cnt - 1)) * (D + 2) + D);
        float2 o[32];
        UNROLL for (int u = 0; u < 32; ++u)
            o[u] = *reinterpret_cast<const float2 *>(base + (int64_t)(c0 + min(u, cnt - 1)) * (D + 2) + 2 * lane);
        const float Mn = fmaxf(M, group_max<64>(lane < cnt ? ml.x : -INFINITY));
        const float keep = __expf(M - Mn);                            /* 0 on the first round (M = -inf) */
        const float wt = lane < cnt ? __expf(ml.x - Mn) : 0.f;
        n0 *= keep;
        n1 *= keep;
        den = den * keep + group_sum<64>(ml.y * wt);
        UNROLL for (int u = 0; u < 32; ++u) {
            const float wi = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(wt), u));   /* 0 past cnt */
            n0 += wi * o[u].x;
            n1 += wi * o[u].y;
        }
        M = Mn;
    }
    const float r0 = n0 / den, r1 = n1 / den;
    const bool mine = 2 * (int)blockIdx.x + w < a.n_heads;
    if (a.out && mine) *reinterpret_cast<float2 *>(a.out + head * D + 2 * lane) = make_float2(r0, r1);
    if (a.qout.qs) {                                                     /* the host asks for this with an even head count only */
        regroup[w * D + 2 * lane] = r0;
        regroup[w * D + 2 * lane + 1] = r1;
        __syncthreads();
        if (w == 0) quantize_out4(a.qout, blockIdx.x * 64 + lane, *reinterpret_cast<const float4 *>(&regroup[4 * lane]));
    }
}

/* out = silu(gate) * up */
extern "C" __global__ void __launch_bounds__(256) psn_swiglu(const psn_swiglu_args a) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= a.n / 4) return;
    const float4 g = reinterpret_cast<const float4 *>(a.gate)[i], u = reinterpret_cast<const float4 *>(a.up)[i];
    float4 o;
    o.x = g.x / (1.f + __expf(-g.x)) * u.x;
    o.y = g.y / (1.f + __expf(-g.y)) * u.y;
    o.z = g.z / (1.f + __expf(-g.z)) * u.z;
    o.w = g.w / (1.f + __expf(-g.w)) * u.w;
    if (a.out) reinterpret_cast<float4 *>(a.out)[i] = o;
    if (a.qout.qs) quantize_out4(a.qout, i, o);        /* n % 256 == 0 then: whole waves reach this point */
}
