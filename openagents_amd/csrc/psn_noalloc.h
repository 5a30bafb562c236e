/*
 * psn_noalloc.h -- internal interface between the host library and the translation unit that owns the
 * static device scratch (psn_noalloc.hip).  Not part of the C ABI.
 */
#ifndef PSN_NOALLOC_H
#define PSN_NOALLOC_H

#include <stddef.h>

/* Size of the per-GPU scratch array.  It holds one quantized activation tensor [batch][K]
 * (int8 values, per-block scales and sums): 1 MiB covers batch 8 at K = 65536 twice over. */
#define PSN_NOALLOC_SCRATCH_BYTES (1u << 20)

/* Device address and size of `device`'s copy of the scratch array; the first call per device looks it
 * up (hipGetSymbolAddress with that device current), later calls return the kept pointer.
 * Returns 0, -1 for a bad argument, -2 when the lookup failed (*hip_error carries the hipError_t). */
__attribute__((visibility("hidden"))) int psn_noalloc_scratch(int device, void **ptr, size_t *bytes, int *hip_error);

#endif
