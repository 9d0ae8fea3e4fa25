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

// ---- sums of several per-lane values over a group of lanes, by exchange-halving ----
// One step over partner distance DIST for a pair of values: lanes whose DIST bit is clear keep `lo`, the others
// `hi`; each lane hands the value it does not keep to its partner (lane ^ DIST) and adds what it receives.  After
// the step every lane carries ONE value where it carried two - so summing 2^k values over a group costs little
// more than summing one.
template <int DIST> __device__ __forceinline__ float fgc_halve_pair(float lo, float hi, int lane)
{
    if constexpr (DIST == 32) {        // upper half of the first operand <-> lower half of the second
        const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(lo), __float_as_uint(hi), false, false);
        return __uint_as_float(r[0]) + __uint_as_float(r[1]);
    } else if constexpr (DIST == 16) { // odd rows of the first operand <-> even rows of the second
        const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(lo), __float_as_uint(hi), false, false);
        return __uint_as_float(r[0]) + __uint_as_float(r[1]);
    } else {
        const bool up = (lane & DIST) != 0;
        const float keep = up ? hi : lo, send = up ? lo : hi;
        int t = __float_as_int(send);
        if constexpr (DIST == 8) t = __builtin_amdgcn_update_dpp(0, t, 0x128, 0xf, 0xf, true);            // row_ror:8
        else if constexpr (DIST == 4) {
            t = __builtin_amdgcn_update_dpp(0, t, 0x141, 0xf, 0xf, true);                                // row_half_mirror: ^7
            t = __builtin_amdgcn_update_dpp(0, t, 0x1B, 0xf, 0xf, true);                                 // quad_perm [3,2,1,0]: ^3
        } else if constexpr (DIST == 2) t = __builtin_amdgcn_update_dpp(0, t, 0x4E, 0xf, 0xf, true);     // quad_perm [2,3,0,1]
        else t = __builtin_amdgcn_update_dpp(0, t, 0xB1, 0xf, 0xf, true);                                // quad_perm [1,0,3,2]
        return keep + __int_as_float(t);
    }
}
// plain butterfly step: v + v of lane ^ DIST (DIST <= 8: inside a row of 16 lanes)
template <int DIST> __device__ __forceinline__ float fgc_add_xor(float v)
{
    int t = __float_as_int(v);
    if constexpr (DIST == 8) t = __builtin_amdgcn_update_dpp(0, t, 0x128, 0xf, 0xf, true);
    else if constexpr (DIST == 4) {
        t = __builtin_amdgcn_update_dpp(0, t, 0x141, 0xf, 0xf, true);
        t = __builtin_amdgcn_update_dpp(0, t, 0x1B, 0xf, 0xf, true);
    } else if constexpr (DIST == 2) t = __builtin_amdgcn_update_dpp(0, t, 0x4E, 0xf, 0xf, true);
    else t = __builtin_amdgcn_update_dpp(0, t, 0xB1, 0xf, 0xf, true);
    return v + __int_as_float(t);
}
// Sums of eight per-lane values over each aligned group of PW lanes (PW = 16, 32 or 64).  Returns, in the lane
// at position pl of its group, the total of value number pl * 8 / PW (each total ends up in PW / 8 adjacent lanes).
template <int PW> __device__ __forceinline__ float fgc_group_reduce8(const float (&v)[8], int lane)
{
    float a[4], b[2];
#pragma unroll
    for (int t = 0; t < 4; t++) a[t] = fgc_halve_pair<PW / 2>(v[t], v[t + 4], lane);
#pragma unroll
    for (int t = 0; t < 2; t++) b[t] = fgc_halve_pair<PW / 4>(a[t], a[t + 2], lane);
    float c = fgc_halve_pair<PW / 8>(b[0], b[1], lane);
    if constexpr (PW >= 64) c = fgc_add_xor<4>(c);
    if constexpr (PW >= 32) c = fgc_add_xor<2>(c);
    if constexpr (PW >= 16) c = fgc_add_xor<1>(c);
    return c;
}

// internal launchers shared between translation units (all enqueue on `s`)
int fgc_fill_u32(void *d, uint32_t v, int64_t n_words, hipStream_t s);
int fgc_copy_u32(void *dst, const void *src, int64_t n_words, hipStream_t s);
