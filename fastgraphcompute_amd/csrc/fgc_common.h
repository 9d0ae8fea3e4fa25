// Shared declarations of the HIP sources of libfgc_hip.so (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "../../include/fgc_hip.h"

#define FGC_WAVE 64

// Layout of the float32[FGC_GEOM_FLOATS] geometry record in device memory.
//   [0..4]  per-dimension minimum subtracted before binning
//   [5]     bin width (same in every binned dimension)
//   [6..10] bins per dimension, int32 bit patterns
//   [11]    flags (int32 bit pattern, FGC_ST_* bits)
#define FGC_GEOM_MIN 0
#define FGC_GEOM_BW 5
#define FGC_GEOM_NB 6
#define FGC_GEOM_FLAGS 11

#define FGC_LAUNCH_CHECK()                         \
    do {                                           \
        hipError_t e__ = hipGetLastError();        \
        if (e__ != hipSuccess) return (int)e__;    \
    } while (0)

static inline int64_t fgc_cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }
static inline size_t fgc_align(size_t x) { return (x + 255) & ~(size_t)255; }

// ---- device helpers -------------------------------------------------------
__device__ __forceinline__ int fgc_lane() { return (int)(threadIdx.x & 63); }

__device__ __forceinline__ float fgc_readlane_f(float v, int lane)
{
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}
__device__ __forceinline__ int fgc_readlane_i(int v, int lane)
{
    return __builtin_amdgcn_readlane(v, lane);
}
__device__ __forceinline__ unsigned long long fgc_ballot(bool p)
{
    return __builtin_amdgcn_ballot_w64(p);
}
// number of set bits of `m` below this lane
__device__ __forceinline__ int fgc_mbcnt(unsigned long long m)
{
    return (int)__builtin_amdgcn_mbcnt_hi((unsigned)(m >> 32),
                                          __builtin_amdgcn_mbcnt_lo((unsigned)m, 0u));
}

// internal launchers shared between translation units (all enqueue on `s`)
int fgc_fill_u32(void *d, uint32_t v, int64_t n_words, hipStream_t s);
int fgc_copy_u32(void *dst, const void *src, int64_t n_words, hipStream_t s);
