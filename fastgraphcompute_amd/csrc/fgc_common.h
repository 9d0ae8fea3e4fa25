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

// sum of v over the 64 lanes (returned in every lane): four DPP steps inside each row of 16 lanes
// (quad swaps, half-row mirror, row mirror), then the four row sums are combined through scalar reads
__device__ __forceinline__ float fgc_wave_sum(float v)
{
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xf, 0xf, true));   // quad_perm [1,0,3,2]
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xf, 0xf, true));   // quad_perm [2,3,0,1]
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xf, 0xf, true));  // row_half_mirror
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xf, 0xf, true));  // row_mirror
    return (fgc_readlane_f(v, 0) + fgc_readlane_f(v, 16)) + (fgc_readlane_f(v, 32) + fgc_readlane_f(v, 48));
}

// maximum of v over the 64 lanes (returned in every lane), same data movement as fgc_wave_sum
__device__ __forceinline__ int fgc_wave_max_i(int v)
{
    v = max(v, __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xf, 0xf, true));
    v = max(v, __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xf, 0xf, true));
    v = max(v, __builtin_amdgcn_update_dpp(0, v, 0x141, 0xf, 0xf, true));
    v = max(v, __builtin_amdgcn_update_dpp(0, v, 0x140, 0xf, 0xf, true));
    return max(max(fgc_readlane_i(v, 0), fgc_readlane_i(v, 16)), max(fgc_readlane_i(v, 32), fgc_readlane_i(v, 48)));
}

// internal launchers shared between translation units (all enqueue on `s`)
int fgc_fill_u32(void *d, uint32_t v, int64_t n_words, hipStream_t s);
int fgc_copy_u32(void *dst, const void *src, int64_t n_words, hipStream_t s);
