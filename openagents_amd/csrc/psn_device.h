/*
 * psn_device.h -- device-side helpers for the gfx950 quantized kernels (wave64 only).
 */
#ifndef PSN_DEVICE_H
#define PSN_DEVICE_H

#include <hip/hip_runtime.h>
#include <stdint.h>

typedef unsigned int u32;
typedef _Float16 f16;

#define PSN_DEV __device__ __forceinline__

PSN_DEV float h2f_lo(u32 v) { return (float)__builtin_bit_cast(f16, (unsigned short)(v & 0xffffu)); }
PSN_DEV float h2f_hi(u32 v) { return (float)__builtin_bit_cast(f16, (unsigned short)(v >> 16)); }

/* signed int8x4 . int8x4 + c  (v_dot4_i32_i8) */
PSN_DEV int dot4(u32 a, u32 b, int c) { return __builtin_amdgcn_sdot4((int)a, (int)b, c, false); }

/* the dword that starts two bytes into lo: bytes {lo[2], lo[3], hi[0], hi[1]} */
PSN_DEV u32 align2(u32 hi, u32 lo) { return __builtin_amdgcn_alignbyte(hi, lo, 2); }

template <int CTRL>
PSN_DEV float dpp_f(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}
template <int CTRL>
PSN_DEV int dpp_i(int v) {
    return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xf, 0xf, true);
}

/* Sum over aligned groups of G consecutive lanes (G = 1..64, power of two); every lane of the
 * group ends with the group's sum.  quad_perm swaps, then row_half_mirror / row_mirror inside a
 * 16-lane DPP row, a ds_swizzle for the 16<->16 exchange and one bpermute across the halves. */
template <int G>
PSN_DEV float group_sum(float v) {
    if (G >= 2) v += dpp_f<0xB1>(v);    /* quad_perm [1,0,3,2] */
    if (G >= 4) v += dpp_f<0x4E>(v);    /* quad_perm [2,3,0,1] */
    if (G >= 8) v += dpp_f<0x141>(v);   /* row_half_mirror */
    if (G >= 16) v += dpp_f<0x140>(v);  /* row_mirror */
    if (G >= 32) v += __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(v), 0x401F)); /* lane ^ 16 */
    if (G >= 64) v += __shfl_xor(v, 32, 64);
    return v;
}
template <int G>
PSN_DEV int group_sum_i(int v) {
    if (G >= 2) v += dpp_i<0xB1>(v);
    if (G >= 4) v += dpp_i<0x4E>(v);
    if (G >= 8) v += dpp_i<0x141>(v);
    if (G >= 16) v += dpp_i<0x140>(v);
    if (G >= 32) v += __builtin_amdgcn_ds_swizzle(v, 0x401F);
    if (G >= 64) v += __shfl_xor(v, 32, 64);
    return v;
}
template <int G>
PSN_DEV float group_max(float v) {
    if (G >= 2) v = fmaxf(v, dpp_f<0xB1>(v));
    if (G >= 4) v = fmaxf(v, dpp_f<0x4E>(v));
    if (G >= 8) v = fmaxf(v, dpp_f<0x141>(v));
    if (G >= 16) v = fmaxf(v, dpp_f<0x140>(v));
    if (G >= 32) v = fmaxf(v, __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(v), 0x401F)));
    if (G >= 64) v = fmaxf(v, __shfl_xor(v, 32, 64));
    return v;
}
/* the same for values that are neither negative nor NaN: their bit patterns order like the values, and an unsigned
 * maximum needs no canonicalization of its operands (one instruction per step instead of three) */
template <int G>
PSN_DEV float group_max_nonneg(float v) {
    u32 b = __float_as_uint(v);
    if (G >= 2) b = max(b, (u32)dpp_i<0xB1>((int)b));
    if (G >= 4) b = max(b, (u32)dpp_i<0x4E>((int)b));
    if (G >= 8) b = max(b, (u32)dpp_i<0x141>((int)b));
    if (G >= 16) b = max(b, (u32)dpp_i<0x140>((int)b));
    if (G >= 32) b = max(b, (u32)__builtin_amdgcn_ds_swizzle((int)b, 0x401F));
    if (G >= 64) b = max(b, (u32)__shfl_xor((int)b, 32, 64));
    return __uint_as_float(b);
}
template <int G>
PSN_DEV int group_min_i(int v) {
    if (G >= 2) v = min(v, dpp_i<0xB1>(v));
    if (G >= 4) v = min(v, dpp_i<0x4E>(v));
    if (G >= 8) v = min(v, dpp_i<0x141>(v));
    if (G >= 16) v = min(v, dpp_i<0x140>(v));
    if (G >= 32) v = min(v, __builtin_amdgcn_ds_swizzle(v, 0x401F));
    if (G >= 64) v = min(v, __shfl_xor(v, 32, 64));
    return v;
}

/* ---- activation quantizers (bit-exact restatements of the GGUF Q8_0 / Q8_K row quantizers); used by
 *      the stand-alone quantize kernels, the matvec staging and the fused decode-step kernels ---- */

/* Q8_0: the four elements a lane owns of a 32-element block shared by 8 adjacent lanes.
 * d = amax/127, q = round-half-away(x/d); returns the packed int8x4, the fp16-rounded scale
 * (widened) and the block's sum of q. */
/* IEEE-754 quotients in three or four instructions instead of the compiler's eleven.  v_rcp_f32 is accurate to one
 * ulp; one Newton step on it, r + r (1 - b r) in two fused multiply-adds, returns the correctly rounded 1 / b, and
 * a quotient a / b follows from a r corrected by its own remainder.  This is arithmetic of THIS device's v_rcp_f32:
 * psn_selftest_arith (psn_calib.hip) compares the shortcuts with the compiler's IEEE division for every float of
 * the range they are used on, 2^-100 ... 2^100 in magnitude, both signs, and found no difference; outside
 * fast_div_range the callers divide the long way. */
PSN_DEV float rcp_rn(float b) {
    const float r = __builtin_amdgcn_rcpf(b);
    return __builtin_fmaf(__builtin_fmaf(-b, r, 1.f), r, r);
}
/* a / b with r = rcp_rn(b), or for a constant b its rounded reciprocal */
PSN_DEV float div_rn(float a, float b, float r) {
    const float q = a * r;
    return __builtin_fmaf(__builtin_fmaf(-q, b, a), r, q);
}
PSN_DEV bool fast_div_range(float magnitude) { return magnitude >= 0x1p-90f && magnitude <= 0x1p90f; }

/* roundf (halves away from zero) of |t| < 2^22 as a conversion that truncates: t + copysign(c, t) with c the
 * largest float below 0.5 lands on the right side of every integer (with 0.5 itself, 0.5 - 2^-25 would round up
 * to 1).  Checked against roundf for every float below 4096 in magnitude (tests/test_oracle_formats.py restates
 * the check for the range the quantizers produce). */
PSN_DEV int round_half_away(float t) {
    /* t is a rounded product: the addition must not be fused with the multiplication that made it (a fused
     * multiply-add sees the exact product, which can lie on the other side of a half-integer than t does; the
     * compiler contracts across the inlined call, and HIP's __fadd_rn / __fmul_rn do not stop it).  The empty asm
     * makes t opaque: the product is rounded to a register before the half is added. */
    asm volatile("" : "+v"(t));
    return (int)(t + __builtin_copysignf(__uint_as_float(0x3effffffu), t));
}
/* the low bytes of four ints as one dword */
PSN_DEV u32 pack_bytes4(int q0, int q1, int q2, int q3) {
    const u32 lo = __builtin_amdgcn_perm((u32)q1, (u32)q0, 0x0c0c0400u), hi = __builtin_amdgcn_perm((u32)q3, (u32)q2, 0x0c0c0400u);
    return (hi << 16) | lo;
}
PSN_DEV void q8_0_quant4(const float4 v, u32 &packed, float &d_out, int &sum) {
    float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
    amax = group_max_nonneg<8>(amax);
    float d, id;
    if (fast_div_range(amax)) {                    /* amax / 127 stays inside the checked range of rcp_rn */
        d = div_rn(amax, 127.f, 1.f / 127.f);
        id = rcp_rn(d);
    } else {
        d = amax / 127.f;
        id = d != 0.f ? 1.f / d : 0.f;
    }
    const int q0 = round_half_away(v.x * id), q1 = round_half_away(v.y * id);
    const int q2 = round_half_away(v.z * id), q3 = round_half_away(v.w * id);
    sum = group_sum_i<8>(q0 + q1 + q2 + q3);
    packed = pack_bytes4(q0, q1, q2, q3);
    d_out = (float)(f16)d;            /* what a reader of the fp16 field would see */
}

/* Q8_K: one wave owns a 256-element super-block, four elements per lane.
 * iscale = -127/(signed element of largest magnitude, first one on ties), q = min(127, rint(iscale*x)),
 * d = 1/iscale; s16 = sum of q over the lane's 16-element group (valid in every lane of the quad). */
PSN_DEV void q8_K_quant_wave(const float4 v, int lane, u32 &packed, float &d_out, int &s16) {
    const float e[4] = {v.x, v.y, v.z, v.w};
    float amax = 0.f;
    int first = 4;
    /* >= scanning downwards leaves the lowest index among equal magnitudes */
    _Pragma("unroll") for (int i = 3; i >= 0; --i) if (fabsf(e[i]) >= amax) { amax = fabsf(e[i]); first = i; }
    const float wmax = group_max_nonneg<64>(amax);
    /* the first element of largest magnitude: the lowest lane that holds the maximum (a ballot and a scalar
     * find-first instead of a second wave-wide reduction), and in it the lowest index (`first`) */
    float mine = e[0];
    _Pragma("unroll") for (int i = 1; i < 4; ++i) mine = first == i ? e[i] : mine;
    const unsigned long long holders = __builtin_amdgcn_ballot_w64(amax == wmax);
    const int src = holders ? __builtin_ctzll(holders) : 0;          /* no holder: a NaN among the inputs */
    const float vmax = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(mine), src));
    (void)lane;
    packed = 0;
    int s4 = 0;
    d_out = 0.f;
    if (wmax != 0.f) {
        const bool fast = fast_div_range(wmax);    /* wave-uniform */
        const float iscale = fast ? div_rn(-127.f, vmax, rcp_rn(vmax)) : -127.f / vmax;
        int q[4];
        _Pragma("unroll") for (int i = 0; i < 4; ++i) {
            q[i] = (int)__builtin_rintf(iscale * e[i]);
            q[i] = q[i] > 127 ? 127 : q[i];
            s4 += q[i];
        }
        packed = pack_bytes4(q[0], q[1], q[2], q[3]);
        d_out = fast ? rcp_rn(iscale) : 1.f / iscale;
    }
    s16 = group_sum_i<4>(s4);
}

/* Q8_K with sixteen lanes to a super-block, four super-blocks to a wave: lane l15 of the sixteen holds the 16-byte
 * words l15, 16 + l15, 32 + l15, 48 + l15 of the block (v[0..3]), i.e. elements (16 i + l15) * 4 + e.  All
 * reductions stay inside a 16-lane DPP row (no trip through the LDS crossbar), and a wave runs through one
 * dependent chain for four blocks instead of four chains.  Same results as q8_K_quant_wave: packed[i] are the
 * int8 of v[i], d_out the block's scale, s16[i] the sum over the 16-element group that word 16 i + l15 belongs to
 * (valid in every lane of its quad).  A block of zeros gives zeros. */
PSN_DEV u32 row16_max_u(u32 b) {
    b = max(b, (u32)dpp_i<0xB1>((int)b));
    b = max(b, (u32)dpp_i<0x4E>((int)b));
    b = max(b, (u32)dpp_i<0x141>((int)b));
    return max(b, (u32)dpp_i<0x140>((int)b));
}
PSN_DEV u32 row16_min_u(u32 b) {
    b = min(b, (u32)dpp_i<0xB1>((int)b));
    b = min(b, (u32)dpp_i<0x4E>((int)b));
    b = min(b, (u32)dpp_i<0x141>((int)b));
    return min(b, (u32)dpp_i<0x140>((int)b));
}
PSN_DEV u32 row16_or(u32 b) {
    b |= (u32)dpp_i<0xB1>((int)b);
    b |= (u32)dpp_i<0x4E>((int)b);
    b |= (u32)dpp_i<0x141>((int)b);
    return b | (u32)dpp_i<0x140>((int)b);
}
PSN_DEV void q8_K_quant_row16(const float4 (&v)[4], int lane, u32 (&packed)[4], float &d_out, int (&s16)[4]) {
    float e[16];
    _Pragma("unroll") for (int i = 0; i < 4; ++i) { e[4 * i] = v[i].x; e[4 * i + 1] = v[i].y; e[4 * i + 2] = v[i].z; e[4 * i + 3] = v[i].w; }
    /* the lane's element of largest magnitude, the earlier one on ties (its own elements are in index order):
     * a tournament that carries the signed value along */
    float ab[16], sg[16];
    _Pragma("unroll") for (int p = 0; p < 16; ++p) { ab[p] = fabsf(e[p]); sg[p] = e[p]; }
    _Pragma("unroll") for (int w = 1; w < 16; w *= 2)
        _Pragma("unroll") for (int p = 0; p < 16; p += 2 * w) {
            const bool later = ab[p + w] > ab[p];
            sg[p] = later ? sg[p + w] : sg[p];
            ab[p] = later ? ab[p + w] : ab[p];
        }
    const float amax = ab[0], mine = sg[0];
    const float gmax = __uint_as_float(row16_max_u(__float_as_uint(amax)));
    const bool zero = gmax == 0.f;
    /* the block's first element of largest magnitude.  One lane of the sixteen holds the maximum, except on exact
     * ties between lanes: then the element indices decide (a second and third reduction, taken by the whole wave) */
    const bool holds = amax == gmax && !zero;
    const unsigned long long holders = __builtin_amdgcn_ballot_w64(holds);
    bool tie = false;
    _Pragma("unroll") for (int g = 0; g < 4; ++g) {
        const unsigned b = (unsigned)(holders >> (16 * g)) & 0xffffu;
        tie = tie || (b & (b - 1u)) != 0u;
    }
    float vmax;
    if (!tie) {                                             /* wave-uniform */
        vmax = __uint_as_float(row16_or(holds ? __float_as_uint(mine) : 0u));
    } else {
        u32 pos = 0xffffffffu;                              /* index of the lane's `mine` inside the block */
        _Pragma("unroll") for (int p = 15; p >= 0; --p)
            if (fabsf(e[p]) == amax) pos = (u32)(((p >> 2) * 16 + (lane & 15)) * 4 + (p & 3));
        pos = holds ? pos : 0xffffffffu;
        const u32 first = row16_min_u(pos);
        vmax = __uint_as_float(row16_or(holds && pos == first ? __float_as_uint(mine) : 0u));
    }
    const float vm = zero ? 1.f : vmax;
    const bool fast = __builtin_amdgcn_ballot_w64(!(zero || fast_div_range(gmax))) == 0ull;   /* every block of the wave */
    const float iscale = fast ? div_rn(-127.f, vm, rcp_rn(vm)) : -127.f / vm;
    _Pragma("unroll") for (int i = 0; i < 4; ++i) {
        int q[4], s4 = 0;
        _Pragma("unroll") for (int k = 0; k < 4; ++k) {
            q[k] = (int)__builtin_rintf(iscale * e[4 * i + k]);
            q[k] = q[k] > 127 ? 127 : q[k];
            s4 += q[k];
        }
        packed[i] = pack_bytes4(q[0], q[1], q[2], q[3]);
        s16[i] = group_sum_i<4>(s4);
    }
    const float d = fast ? rcp_rn(iscale) : 1.f / iscale;
    d_out = zero ? 0.f : d;
}

/* ---- hand-scheduled memory access ------------------------------------------------------------
 * Kernels that keep several direct-to-LDS loads in flight place every wait themselves: the compiler's
 * wait insertion cannot tell ring buffers in dynamic LDS apart and would drain ALL outstanding loads
 * before any LDS read.  LDS is therefore accessed through inline assembly the compiler does not model
 * as memory traffic, and vmcnt / lgkmcnt waits are explicit (loads complete in issue order, so "at
 * most n younger loads outstanding" identifies what has landed). */
typedef u32 u32x4 __attribute__((ext_vector_type(4)));
typedef u32 u32x2 __attribute__((ext_vector_type(2)));

/* wave-uniform n: wait until at most n vector-memory loads are outstanding */
PSN_DEV void wait_vmcnt(int n) {
#define PSN_W(k) case k: asm volatile("s_waitcnt vmcnt(" #k ")" ::: "memory"); break;
    switch (n) {
        PSN_W(1) PSN_W(2) PSN_W(3) PSN_W(4) PSN_W(5) PSN_W(6) PSN_W(7) PSN_W(8) PSN_W(9) PSN_W(10) PSN_W(11) PSN_W(12)
        PSN_W(13) PSN_W(14) PSN_W(15) PSN_W(16) PSN_W(17) PSN_W(18) PSN_W(19) PSN_W(20) PSN_W(21) PSN_W(22) PSN_W(23)
        PSN_W(24) PSN_W(25) PSN_W(26) PSN_W(27) PSN_W(28) PSN_W(29) PSN_W(30) PSN_W(31) PSN_W(32) PSN_W(33) PSN_W(34)
        PSN_W(35) PSN_W(36) PSN_W(37) PSN_W(38) PSN_W(39) PSN_W(40) PSN_W(41) PSN_W(42) PSN_W(43) PSN_W(44) PSN_W(45)
        PSN_W(46) PSN_W(47) PSN_W(48) PSN_W(49) PSN_W(50) PSN_W(51) PSN_W(52) PSN_W(53) PSN_W(54) PSN_W(55) PSN_W(56)
        PSN_W(57) PSN_W(58) PSN_W(59) PSN_W(60) PSN_W(61) PSN_W(62) PSN_W(63)
        default:
            /* more than the 6-bit counter can hold: never more than 63 are outstanding, nothing to wait for */
            if (n <= 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            break;
    }
#undef PSN_W
}
/* LDS and global accesses the compiler does not see as memory operations (no automatic waits) */
template <int OFF> PSN_DEV u32x4 lds_read128(u32 addr) {
    u32x4 v;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF) : "memory");
    return v;
}
PSN_DEV u32 lds_read32(u32 addr) {
    u32 v;
    asm volatile("ds_read_b32 %0, %1" : "=v"(v) : "v"(addr) : "memory");
    return v;
}
template <int OFF> PSN_DEV u32 lds_read32o(u32 addr) {
    u32 v;
    asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF) : "memory");
    return v;
}
template <int OFF> PSN_DEV u32x2 lds_read64o(u32 addr) {          /* addr + OFF: a multiple of 8 */
    u32x2 v;
    asm volatile("ds_read_b64 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF) : "memory");
    return v;
}
/* two dwords at addr + 4 * D0 and addr + 4 * D1 (addr a multiple of 4, not necessarily of 8) */
template <int D0, int D1> PSN_DEV u32x2 lds_read2_b32(u32 addr) {
    u32x2 v;
    asm volatile("ds_read2_b32 %0, %1 offset0:%2 offset1:%3" : "=v"(v) : "v"(addr), "n"(D0), "n"(D1) : "memory");
    return v;
}
PSN_DEV u32 lds_read_u16(u32 addr) {
    u32 v;
    asm volatile("ds_read_u16 %0, %1" : "=v"(v) : "v"(addr) : "memory");
    return v;
}
PSN_DEV void lds_write128(u32 addr, u32x4 v) { asm volatile("ds_write_b128 %0, %1" ::"v"(addr), "v"(v) : "memory"); }
PSN_DEV void lds_write32(u32 addr, u32 v) { asm volatile("ds_write_b32 %0, %1" ::"v"(addr), "v"(v) : "memory"); }
PSN_DEV void lds_write16(u32 addr, u32 v) { asm volatile("ds_write_b16 %0, %1" ::"v"(addr), "v"(v) : "memory"); }
PSN_DEV u32x4 global_read128(const void *p) {
    u32x4 v;
    asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(v) : "v"(p) : "memory");
    return v;
}
/* the values written by the reads above may be used after this (volatile asm statements stay in order) */
PSN_DEV void lds_wait() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }
template <int N> PSN_DEV void tie(u32x4 (&v)[N]) { _Pragma("unroll") for (int i = 0; i < N; ++i) asm volatile("" : "+v"(v[i])); }
PSN_DEV void tie1(u32 &v) { asm volatile("" : "+v"(v)); }
/* workgroup barrier that waits for this wave's LDS traffic only, not for loads still in flight */
PSN_DEV void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }


PSN_DEV void unpack4(const uint4 v, u32 *dst) { dst[0] = v.x; dst[1] = v.y; dst[2] = v.z; dst[3] = v.w; }

#endif
