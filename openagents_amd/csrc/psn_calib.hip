/*
 * psn_calib.hip -- calibration kernels: what a launch that ONLY reads a byte range achieves on this
 * machine.  The matvec kernels are judged against the 8 TB/s HBM peak; these kernels tell how much of
 * that a dependent launch of the same size can reach at all (launch ramp, drain and the memory fabric
 * included), which is the number a kernel's own overhead has to be compared with.
 *
 *   psn_calib_read      16-byte vector loads into registers, xor-folded, one dword stored per wave;
 *   psn_calib_read_lds  16-byte direct-to-LDS loads (the path the streaming matvec uses), each wave
 *                       cycling through `depth` 1 KB slots of its own LDS region.
 */
#include "psn_args.h"
#include "psn_device.h"

extern "C" __global__ void __launch_bounds__(1024) psn_calib_read(const psn_calib_args a) {
    const int lane = threadIdx.x & 63;
    /* every_wg: each workgroup reads the whole range (the access pattern of an operand all workgroups share) */
    const int64_t wave = a.every_wg ? (threadIdx.x >> 6) : (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const int64_t nwaves = a.every_wg ? (blockDim.x >> 6) : (int64_t)gridDim.x * (blockDim.x >> 6);
    const int64_t slab = 64 * 16 * 4;                       /* 4 KB per wave and iteration */
    const int64_t nslabs = a.bytes / slab;
    uint4 acc = make_uint4(0, 0, 0, 0);
    for (int64_t s = wave; s < nslabs; s += nwaves) {
        const uint4 *p = reinterpret_cast<const uint4 *>(a.src + s * slab) + lane;
        const uint4 v0 = p[0], v1 = p[64], v2 = p[128], v3 = p[192];
        acc.x ^= v0.x ^ v1.x ^ v2.x ^ v3.x;
        acc.y ^= v0.y ^ v1.y ^ v2.y ^ v3.y;
        acc.z ^= v0.z ^ v1.z ^ v2.z ^ v3.z;
        acc.w ^= v0.w ^ v1.w ^ v2.w ^ v3.w;
    }
    u32 r = acc.x ^ acc.y ^ acc.z ^ acc.w;
    r ^= (u32)__shfl_xor((int)r, 32, 64);
    if (lane == 0 && a.out) a.out[(int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)] = r;
}

extern "C" __global__ void __launch_bounds__(1024) psn_calib_read_lds(const psn_calib_args a) {
    extern __shared__ uint4 psn_smem[];
    const int lane = threadIdx.x & 63, wib = threadIdx.x >> 6;
    const int64_t wave = a.every_wg ? wib : (int64_t)blockIdx.x * (blockDim.x >> 6) + wib;
    const int64_t nwaves = a.every_wg ? (blockDim.x >> 6) : (int64_t)gridDim.x * (blockDim.x >> 6);
    const int depth = a.depth;                              /* 1 KB slots per wave */
    const int64_t slab = (int64_t)depth << 10;
    const int64_t nslabs = a.bytes / slab;
    char *buf = reinterpret_cast<char *>(psn_smem) + (int64_t)wib * slab;
    u32 r = 0;
    for (int64_t s = wave; s < nslabs; s += nwaves) {
        const uint8_t *src = a.src + s * slab + lane * 16;
        for (int i = 0; i < depth; ++i)
            __builtin_amdgcn_global_load_lds((const void *)(src + i * 1024), (__attribute__((address_space(3))) void *)(buf + i * 1024), 16, 0, 0);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        r ^= reinterpret_cast<const u32 *>(buf)[lane];
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    }
    if (lane == 0 && a.out) a.out[(int64_t)blockIdx.x * (blockDim.x >> 6) + wib] = r;
}

/* The activation quantizers replace IEEE divisions by rcp_rn / div_rn (psn_device.h).  This kernel walks every
 * float x with bit pattern lo .. hi and counts, per identity, the values for which the shortcut and the compiler's
 * division differ in any bit:
 *   0  rcp_rn(x)  vs  1 / x              1  rcp_rn(-x)  vs  1 / -x
 *   2  div_rn(-127, x, rcp_rn(x))  vs  -127 / x      3  the same for -x
 *   4  div_rn(x, 127, RN(1/127))  vs  x / 127        5  rcp_rn(x / 127)  vs  1 / (x / 127)
 *   6  rcp_rn(-127 / x)  vs  1 / (-127 / x)          7  the same for -x
 * (5 - 7: the reciprocals the quantizers take of their own quotients.) */
extern "C" __global__ void __launch_bounds__(256) psn_selftest_arith(const psn_selftest_args a) {
    const unsigned long long stride = (unsigned long long)gridDim.x * blockDim.x;
    unsigned c[PSN_SELFTEST_COUNTERS];
    _Pragma("unroll") for (int i = 0; i < PSN_SELFTEST_COUNTERS; ++i) c[i] = 0;
    auto differ = [](float p, float q) { return __float_as_uint(p) != __float_as_uint(q) ? 1u : 0u; };
    for (unsigned long long b = a.lo + (unsigned long long)blockIdx.x * blockDim.x + threadIdx.x; b <= a.hi; b += stride) {
        const float x = __uint_as_float((u32)b);
        c[0] += differ(rcp_rn(x), 1.f / x);
        c[1] += differ(rcp_rn(-x), 1.f / -x);
        c[2] += differ(div_rn(-127.f, x, rcp_rn(x)), -127.f / x);
        c[3] += differ(div_rn(-127.f, -x, rcp_rn(-x)), -127.f / -x);
        const float d = x / 127.f;
        c[4] += differ(div_rn(x, 127.f, 1.f / 127.f), d);
        c[5] += differ(rcp_rn(d), 1.f / d);
        const float sp = -127.f / x, sn = -127.f / -x;
        c[6] += differ(rcp_rn(sp), 1.f / sp);
        c[7] += differ(rcp_rn(sn), 1.f / sn);
    }
    _Pragma("unroll") for (int i = 0; i < PSN_SELFTEST_COUNTERS; ++i) if (c[i]) atomicAdd(&a.bad[i], (unsigned long long)c[i]);
}
