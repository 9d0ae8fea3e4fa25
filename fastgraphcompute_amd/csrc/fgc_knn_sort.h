// Bitonic sorting network over the 64 lanes of a wavefront (and NSEG registers per lane), shared by the kNN search
// kernels: no LDS traffic, exchanges are DPP moves and the lane-swap instructions of gfx950.
#pragma once
#include "fgc_common.h"

// ---- bitonic network across the lanes without LDS traffic ----
// partner value for lane ^ JJ: DPP moves inside a row of 16 lanes, the lane-swap instructions of gfx950 across rows
__device__ __forceinline__ int fgc_sel_i(unsigned long long mask, int if_set, int if_clear)
{
    int r;
    asm("v_cndmask_b32_e64 %0, %1, %2, %3" : "=v"(r) : "v"(if_clear), "v"(if_set), "s"(mask));
    return r;
}
template <int JJ> __device__ __forceinline__ int fgc_xor_lane(int v)
{
    if constexpr (JJ == 1) return __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xf, 0xf, true);        // quad_perm [1,0,3,2]
    else if constexpr (JJ == 2) return __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xf, 0xf, true);   // quad_perm [2,3,0,1]
    else if constexpr (JJ == 4) {
        const int t = __builtin_amdgcn_update_dpp(0, v, 0x141, 0xf, 0xf, true);                   // row_half_mirror: ^7
        return __builtin_amdgcn_update_dpp(0, t, 0x1B, 0xf, 0xf, true);                           // quad_perm [3,2,1,0]: ^3
    } else if constexpr (JJ == 8) return __builtin_amdgcn_update_dpp(0, v, 0x128, 0xf, 0xf, true);  // row_ror:8
    else if constexpr (JJ == 16) {
        // odd rows of the first operand are swapped with the even rows of the second
        const auto r = __builtin_amdgcn_permlane16_swap((unsigned)v, (unsigned)v, false, false);
        return fgc_sel_i(0xffff0000ffff0000ull, (int)r[0], (int)r[1]);
    } else {
        // upper half of the first operand is swapped with the lower half of the second
        const auto r = __builtin_amdgcn_permlane32_swap((unsigned)v, (unsigned)v, false, false);
        return fgc_sel_i(0xffffffff00000000ull, (int)r[0], (int)r[1]);
    }
}
// lanes that keep the smaller key in the step (k, jj) of the network over elements e = s * 64 + lane
constexpr unsigned long long fgc_keep_min_mask(int k, int jj, int s)
{
    unsigned long long m = 0;
    for (int l = 0; l < 64; l++) {
        const int e = s * 64 + l;
        if (((e & jj) == 0) == ((e & k) == 0)) m |= 1ull << l;
    }
    return m;
}
// one compare-exchange step with partners jj < 64 lanes apart; equal keys never move
template <int KK, int JJ, int NSEG> __device__ __forceinline__ void fgc_bitonic_step(float (&L)[NSEG], int (&I)[NSEG])
{
#pragma unroll
    for (int s = 0; s < NSEG; s++) {
        const unsigned long long km = fgc_keep_min_mask(KK, JJ, s);
        const float pd = __int_as_float(fgc_xor_lane<JJ>(__float_as_int(L[s])));
        const int pv = fgc_xor_lane<JJ>(I[s]);
        const unsigned long long lt = fgc_ballot(pd < L[s]), gt = fgc_ballot(pd > L[s]);
        const unsigned long long take = (lt & km) | (gt & ~km);
        L[s] = __int_as_float(fgc_sel_i(take, __float_as_int(pd), __float_as_int(L[s])));
        I[s] = fgc_sel_i(take, pv, I[s]);
    }
}
template <int KK, int JJ, int NSEG> struct FgcBitonic {
    static __device__ __forceinline__ void run(float (&L)[NSEG], int (&I)[NSEG])
    {
        if constexpr (JJ >= 64) {
            // partners are two registers of one lane; each pair once, ascending iff (e & k) == 0
#pragma unroll
            for (int s = 0; s < NSEG; s++) {
                const int s2 = s ^ (JJ >> 6);
                if (s2 > s) {
                    const bool asc = ((s * 64) & KK) == 0;
                    const bool swap = asc ? (L[s2] < L[s]) : (L[s2] > L[s]);
                    const float d0 = swap ? L[s2] : L[s], d1 = swap ? L[s] : L[s2];
                    const int v0 = swap ? I[s2] : I[s], v1 = swap ? I[s] : I[s2];
                    L[s] = d0; L[s2] = d1; I[s] = v0; I[s2] = v1;
                }
            }
        } else {
            fgc_bitonic_step<KK, JJ, NSEG>(L, I);
        }
        if constexpr (JJ > 1) FgcBitonic<KK, JJ / 2, NSEG>::run(L, I);
        else if constexpr (KK < NSEG * 64) FgcBitonic<KK * 2, KK, NSEG>::run(L, I);
    }
};
