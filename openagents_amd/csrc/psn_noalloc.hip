/*
 * psn_noalloc.hip -- the device-resident scratch of psn_qmatvec_noalloc.
 *
 * Callers that cannot allocate (code under graph capture, tight serving loops, harnesses that forbid
 * hipMalloc) still need somewhere to put the quantized activations between the quantize launch and the
 * int8 matvec launch.  That memory is a file-scope __device__ array of a fixed, modest size: it is part
 * of this library's device image, so every GPU the library runs on holds its own copy, at its own
 * address, from the moment the image is loaded until the process ends.
 *
 * In host code the array's name is only a stand-in for that symbol -- it is not a device address and
 * must never be handed to a kernel or a memset.  The address is looked up once per device with
 * hipGetSymbolAddress (with that device current) and kept; everything else uses the looked-up pointer.
 * This file is compiled by hipcc (host and gfx950 device code in one translation unit), unlike the rest
 * of the host library, because the symbol has to be registered together with its device image.
 */
#include <hip/hip_runtime.h>

#include <mutex>

#include "psn_noalloc.h"

/* No `used` attribute here: the host-side reference below is what makes the compiler export the
 * (otherwise file-local) device symbol from the device image, and `used` suppresses exactly that --
 * the runtime then cannot find the registered name and ends the process inside hipGetSymbolAddress. */
static __device__ __align__(256) unsigned char scratch[PSN_NOALLOC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_mu;
void *g_ptr[kMaxDevices];          /* per device: the address of that GPU's copy of `scratch` */
bool g_known[kMaxDevices];
}  // namespace

int psn_noalloc_scratch(int device, void **ptr, size_t *bytes, int *hip_error) {
    if (hip_error) *hip_error = 0;
    if (device < 0 || device >= kMaxDevices || !ptr) return -1;
    std::lock_guard<std::mutex> lk(g_mu);
    if (!g_known[device]) {
        int cur = -1;
        hipError_t e = hipGetDevice(&cur);
        if (e == hipSuccess && cur != device) e = hipSetDevice(device);
        void *p = nullptr;
        if (e == hipSuccess) e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e == hipSuccess && cur >= 0 && cur != device) e = hipSetDevice(cur);
        if (e != hipSuccess || !p) {
            if (hip_error) *hip_error = (int)e;
            return -2;
        }
        g_ptr[device] = p;
        g_known[device] = true;
    }
    *ptr = g_ptr[device];
    if (bytes) *bytes = PSN_NOALLOC_SCRATCH_BYTES;
    return 0;
}
