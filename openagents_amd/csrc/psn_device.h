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

PSN_DEV void unpack4(const uint4 v, u32 *dst) { dst[0] = v.x; dst[1] = v.y; dst[2] = v.z; dst[3] = v.w; }

#endif
