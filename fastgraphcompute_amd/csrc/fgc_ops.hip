// index_replacer, kNN gradient, select_with_default and the fused GravNet
// neighbour aggregation (forward / backward).  gfx950, wave64.
#include "fgc_common.h"
#include "fgc_internal.h"

// ---------------------------------------------------------------------------
// index_replacer
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void k_index_replacer(const int64_t *__restrict__ in,
                                                        const int64_t *__restrict__ repl,
                                                        int64_t *__restrict__ out, int64_t n, int64_t n_repl)
{
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    int64_t r = in[i];
    out[i] = (r < 0 || r >= n_repl) ? r : repl[r];
}

extern "C" int fgc_index_replacer_i64(const int64_t *d_in, const int64_t *d_repl, int64_t *d_out,
                                      int64_t n, int64_t n_repl, void *stream)
{
    if (n < 0 || n_repl < 0) return FGC_EINVAL;
    if (n == 0) return FGC_OK;
    hipLaunchKernelGGL(k_index_replacer, dim3((unsigned)fgc_cdiv(n, 256)), dim3(256), 0, (hipStream_t)stream,
                       d_in, d_repl, d_out, n, n_repl);
    FGC_LAUNCH_CHECK();
    return FGC_OK;
}

// Overflow of the per-wavefront table: the lanes flagged `ovf` add their float4 `add` to the four coordinates
// c0 .. c0 + 3 of row `target` of gx (row stride ld).  The values are exchanged between the lanes so that each
// atomic instruction carries 16 targets with their four coordinates in adjacent lanes: the memory side then sees
// one 16-byte update per target instead of one per coordinate, and it is the number of such updates that bounds
// the atomic rate (also with only a few lanes flagged: N=1M, D=3, K=64 0.54 -> 0.47 ms against issuing them from
// the flagged lanes directly).  Wave-uniform call (all lanes, same c0).
__device__ __forceinline__ void grad_overflow_add(unsigned long long ovf_mask, bool ovf, int target, float4 add,
                                                  int c0, int D, int ld, float *__restrict__ gx, int lane)
{
    const int tgt = ovf ? target : -1;
    const int comp = lane & 3;
#pragma unroll
    for (int r = 0; r < 4; r++) {
        if (!((ovf_mask >> (16 * r)) & 0xffffull)) continue;   // none of these 16 lanes overflowed
        const int e = r * 16 + (lane >> 2);
        const int te = __shfl(tgt, e, 64);
        const float v0 = __shfl(add.x, e, 64), v1 = __shfl(add.y, e, 64);
        const float v2 = __shfl(add.z, e, 64), v3 = __shfl(add.w, e, 64);
        const float v = comp == 0 ? v0 : comp == 1 ? v1 : comp == 2 ? v2 : v3;
        if (te >= 0 && c0 + comp < D) atomicAdd(&gx[(int64_t)te * ld + c0 + comp], v);
    }
}

// The same for points of five or more coordinates: the float4 groups c0 .. c0 + 3 (`lo`) and c0 + 4 .. c0 + 7 (`hi`)
// of a target go out together, eight adjacent lanes per target and eight targets per instruction - one 32-byte
// update per target instead of two 16-byte ones (N=500 k, D=8, K=100, where nearly every pair overflows: 3.6 ms
// with one group per update).  Wave-uniform call.
__device__ __forceinline__ void grad_overflow_add8(unsigned long long ovf_mask, bool ovf, int target, float4 lo,
                                                   float4 hi, int c0, int D, int ld, float *__restrict__ gx, int lane)
{
    if (__popcll(ovf_mask) <= 3) {
        if (ovf) {
            const float v[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
#pragma unroll
            for (int e = 0; e < 8; e++)
                if (c0 + e < D) atomicAdd(&gx[(int64_t)target * ld + c0 + e], v[e]);
        }
        return;
    }
    const int tgt = ovf ? target : -1;
    const int comp = lane & 7;
#pragma unroll
    for (int r = 0; r < 8; r++) {
        if (!((ovf_mask >> (8 * r)) & 0xffull)) continue;     // none of these 8 lanes overflowed
        const int e = r * 8 + (lane >> 3);
        const int te = __shfl(tgt, e, 64);
        const float v0 = __shfl(lo.x, e, 64), v1 = __shfl(lo.y, e, 64), v2 = __shfl(lo.z, e, 64), v3 = __shfl(lo.w, e, 64);
        const float v4 = __shfl(hi.x, e, 64), v5 = __shfl(hi.y, e, 64), v6 = __shfl(hi.z, e, 64), v7 = __shfl(hi.w, e, 64);
        const float va = (comp & 2) ? ((comp & 1) ? v3 : v2) : ((comp & 1) ? v1 : v0);
        const float vb = (comp & 2) ? ((comp & 1) ? v7 : v6) : ((comp & 1) ? v5 : v4);
        const float v = (comp & 4) ? vb : va;
        if (te >= 0 && c0 + comp < D) atomicAdd(&gx[(int64_t)te * ld + c0 + comp], v);
    }
}

// ---------------------------------------------------------------------------
// gradient of distsq wrt the coordinates
// ---------------------------------------------------------------------------
// g[m] += 2 gd[i,k] (x_m - x_i) for every neighbour m = idx[i,k] and
// g[i] -= sum_k of the same terms.  A wavefront takes GW queries - consecutive
// in the bin-sorted order when `order` is given, so their neighbourhoods
// overlap - lane k owning neighbour slot k, and first combines all contributions
// to the same target point in its own LDS hash table (open addressing).  The
// table is private to the wavefront and within one instruction every slot is
// updated by one lane only, so the update is a plain LDS read-add-write of one
// float4 - no float atomics on chip.  The neighbours of one query are normally
// distinct points; a row that names a point twice is legal input, and the lanes
// that then share a slot are told apart through an owner byte (see below).
// Only the distinct targets of the wavefront go to global memory, one float
// atomic per coordinate with a target's coordinates in adjacent lanes.  Pairs
// that find no table slot within a few probes go to global memory directly.
#ifndef GW
#define GW 24          // queries per wavefront
#endif
#ifndef GU
#define GU 4           // queries a wavefront processes together (loads in flight)
#endif
#ifndef GRAD_H
#define GRAD_H 512     // hash table slots per wavefront (upper bound, shrunk for wide points)
#endif
#define GRAD_PROBES 8
#define GRAD_EMPTY 0xffffffffu

__global__ __launch_bounds__(256) void k_knn_grad(const float *__restrict__ gd, const int64_t *__restrict__ idx,
                                                  const float *__restrict__ x, float *__restrict__ gx,
                                                  const uint32_t *__restrict__ order, int64_t n, int K, int D,
                                                  int H, int *__restrict__ status)
{
    extern __shared__ __align__(16) unsigned char s_raw[];
    const int lane = fgc_lane();
    const int wv = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));   // uniform by construction
    const int D4 = (D + 3) >> 2;                       // float4 groups per point
    const size_t wave_bytes = (size_t)H * (8 + 16 * (size_t)D4);
    float4 *vals = (float4 *)(s_raw + wave_bytes * wv);                  // [H][D4]
    unsigned *keys = (unsigned *)(s_raw + wave_bytes * wv + (size_t)H * 16 * D4);   // [H]
    unsigned char *owner = s_raw + wave_bytes * wv + (size_t)H * (16 * (size_t)D4 + 4);   // [H]
    for (int t = lane; t < H; t += 64) keys[t] = GRAD_EMPTY;
    for (int t = lane; t < H * D4; t += 64) vals[t] = make_float4(0.f, 0.f, 0.f, 0.f);
    const unsigned hmask = (unsigned)H - 1u;
    bool bad = false;

    // slot of target m in the wavefront's table, or -1 when no slot is free within a few probes
    auto slot_of = [&](unsigned m) -> int {
        unsigned h = (m * 2654435761u) >> 7;
        for (int p = 0; p < GRAD_PROBES; p++) {
            const unsigned sl = (h + p) & hmask;
            const unsigned old = atomicCAS(&keys[sl], GRAD_EMPTY, m);
            if (old == GRAD_EMPTY || old == m) return (int)sl;
        }
        return -1;
    };

    const int64_t wave0 = ((int64_t)blockIdx.x * 4 + wv) * GW;
    for (int q0 = 0; q0 < GW; q0 += GU) {
        int64_t qi[GU];
        bool qv[GU];
#pragma unroll
        for (int u = 0; u < GU; u++) {
            const int64_t pos = wave0 + q0 + u;
            qv[u] = pos < n;
            qi[u] = qv[u] ? (order ? (int64_t)order[pos] : pos) : 0;
        }
        for (int k0 = 0; k0 < K; k0 += 64) {
            const int k = k0 + lane;
            int64_t m[GU];
            float g[GU];
            int sl[GU];
#pragma unroll
            for (int u = 0; u < GU; u++) {
                m[u] = -1; g[u] = 0.f;
                if (k < K && qv[u]) { m[u] = idx[qi[u] * K + k]; g[u] = gd[qi[u] * K + k]; }
            }
#pragma unroll
            for (int u = 0; u < GU; u++) {
                if (m[u] >= n) { bad = true; m[u] = -1; }
                sl[u] = (m[u] >= 0) ? slot_of((unsigned)m[u]) : -1;
                // a row may name the same point twice (any index tensor can be passed to this op): the lanes that
                // share a slot in this instruction write their number into the slot's owner byte, the one that
                // reads its own number back updates the table, the others add to memory directly
                if (sl[u] >= 0) owner[sl[u]] = (unsigned char)lane;
                asm volatile("" ::: "memory");             // the byte is read back from LDS, not from the register
                if (sl[u] >= 0 && owner[sl[u]] != (unsigned char)lane) sl[u] = -1;
                asm volatile("" ::: "memory");
            }
            float4 addp[GU];       // the even float4 group of an overflowing pair, until its partner is known
#pragma unroll
            for (int u = 0; u < GU; u++) addp[u] = make_float4(0.f, 0.f, 0.f, 0.f);
            for (int c4 = 0; c4 < D4; c4++) {
#pragma unroll
                for (int u = 0; u < GU; u++) {
                    float add[4], self[4];
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const int c = c4 * 4 + e;
                        add[e] = 0.f;
                        if (c < D && m[u] >= 0) add[e] = 2.f * g[u] * (x[m[u] * D + c] - x[qi[u] * D + c]);
                        self[e] = (c < D) ? fgc_wave_sum(add[e]) : 0.f;
                    }
                    if (m[u] >= 0 && sl[u] >= 0) {
                        // one lane per slot within the instruction, private table: plain read-add-write
                        float4 v = vals[sl[u] * D4 + c4];
                        v.x += add[0]; v.y += add[1]; v.z += add[2]; v.w += add[3];
                        vals[sl[u] * D4 + c4] = v;
                    }
                    const bool ovf = m[u] >= 0 && sl[u] < 0;
                    const unsigned long long om = fgc_ballot(ovf);
                    if (om) {
                        // float4 groups leave in pairs (one 32-byte update per target), an unpaired last one alone
                        const float4 a4 = make_float4(add[0], add[1], add[2], add[3]);
                        if (!(c4 & 1) && c4 + 1 < D4) addp[u] = a4;
                        else if (c4 & 1) grad_overflow_add8(om, ovf, (int)m[u], addp[u], a4, (c4 - 1) * 4, D, D, gx, lane);
                        else grad_overflow_add(om, ovf, (int)m[u], a4, c4 * 4, D, D, gx, lane);
                    }
                    // the query's own share, after the neighbours' updates of this instruction
                    if (qv[u]) {
                        int ss = -1;
                        if (lane == 0) ss = slot_of((unsigned)qi[u]);
                        ss = fgc_readlane_i(ss, 0);
                        if (lane == 0) {
                            if (ss >= 0) {
                                float4 v = vals[ss * D4 + c4];
                                v.x -= self[0]; v.y -= self[1]; v.z -= self[2]; v.w -= self[3];
                                vals[ss * D4 + c4] = v;
                            } else {
#pragma unroll
                                for (int e = 0; e < 4; e++)
                                    if (c4 * 4 + e < D) atomicAdd(&gx[qi[u] * D + c4 * 4 + e], -self[e]);
                            }
                        }
                    }
                }
            }
        }
    }
    // flush: one lane per (slot, coordinate), the atomics of one target sit in adjacent lanes
    const float *vflat = (const float *)vals;
    for (int t = lane; t < H * D4 * 4; t += 64) {
        const int sl = t / (D4 * 4), c = t - sl * (D4 * 4);
        const unsigned m = keys[sl];
        if (m == GRAD_EMPTY || c >= D) continue;
        const float v = vflat[t];
        if (v != 0.f) atomicAdd(&gx[(int64_t)m * D + c], v);
    }
    if (bad && status) atomicOr(&status[0], FGC_ST_BAD_INDEX);
}

static int grad_table_size(int D)
{
    int H = GRAD_H;
    const size_t d4 = (size_t)((D + 3) / 4);
    while (H > 64 && (size_t)H * (8 + 16 * d4) > 12288) H >>= 1;       // at most 12 KB per wavefront
    return H;
}

extern "C" int fgc_binned_select_knn_grad_f32(const float *d_grad_distsq, const int64_t *d_idx,
                                              const float *d_coords, float *d_grad_coords, int64_t n_vert,
                                              int32_t K, int32_t n_coords, const int32_t *d_order,
                                              int32_t *d_status, void *stream)
{
    if (n_vert < 0 || K < 1 || n_coords < 1 || n_coords > 128) return FGC_EINVAL;
    if (n_vert >= (1ll << 32) - 1) return FGC_EINVAL;
    if (n_vert == 0) return FGC_OK;
    hipStream_t s = (hipStream_t)stream;
    int rc = fgc_fill_u32(d_grad_coords, 0u, n_vert * n_coords, s);
    if (rc) return rc;
    const int H = grad_table_size(n_coords);
    const size_t lds = 4 * (size_t)H * (8 + 16 * (size_t)((n_coords + 3) / 4));
    const unsigned blocks = (unsigned)fgc_cdiv(n_vert, 4 * GW);
    hipLaunchKernelGGL(k_knn_grad, dim3(blocks), dim3(256), lds, s, d_grad_distsq, d_idx, d_coords,
                       d_grad_coords, (const uint32_t *)d_order, n_vert, (int)K, (int)n_coords, H, d_status);
    FGC_LAUNCH_CHECK();
    return FGC_OK;
}

// ---------------------------------------------------------------------------
// the same gradient from the search's sorted-space neighbour rows
// ---------------------------------------------------------------------------
// The kernel above gathers x[m] from the original order, where the neighbours of a query sit in 64 different
// cache lines: 64 M gathers pull 8 GB of lines out of L2 for 0.8 GB of payload, and that transfer is what bounds
// it.  In the search's sorted order neighbours are memory neighbours.  This variant reads the neighbour rows the
// search wrote in that order (int32, streaming), a padded array-of-points copy of the coordinates in the same
// order (one 16-byte gather per neighbour and four coordinates), and only the upstream gradient row and the
// final atomics go through the permutation.
__global__ __launch_bounds__(256) void k_sorted_points(const float *__restrict__ x, int ldx,
                                                       const uint32_t *__restrict__ order, int64_t n, int D, int D4,
                                                       float4 *__restrict__ xs, float4 *__restrict__ gxs)
{
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= n * D4) return;
    int64_t r = t;
    int c4 = 0;
    if (D4 > 1) { r = t / D4; c4 = (int)(t - r * D4); }
    const int64_t o = order[r];
    float v[4];
#pragma unroll
    for (int e = 0; e < 4; e++) v[e] = (c4 * 4 + e < D) ? x[o * ldx + c4 * 4 + e] : 0.f;
    xs[t] = make_float4(v[0], v[1], v[2], v[3]);
    gxs[t] = make_float4(0.f, 0.f, 0.f, 0.f);       // the gradient accumulator in the same order starts at zero
}

#ifndef GSH
#define GSH 512      // table slots per wavefront where an entry is 16 bytes (D <= 3)
#endif
#ifndef GSW
#define GSW 24       // rows per wavefront where an entry is 16 bytes (N=1M, D=3, K=64: 16 rows 0.53 ms, 20 0.44, 24 0.43,
#endif               // 32 0.47, 48 0.49: fewer rows share less, more rows fill the table and wait longer for their loads)

// Totals of 16 per-lane values over the 64 lanes, in 36 instead of 16 x 11 instructions: each exchange step
// halves the number of values a lane still carries (the lane keeps the half its own bit selects and hands the
// other half to its partner).  Returns, in every lane L, the total of value number L >> 2.
__device__ __forceinline__ float fgc_wave_reduce16(const float (&v)[16], int lane)
{
    float a[8], b[4], c[2];
#pragma unroll
    for (int t = 0; t < 8; t++) {      // partner lane ^ 32: lower half keeps values 0..7, upper half 8..15
        const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v[t]), __float_as_uint(v[t + 8]), false, false);
        a[t] = __uint_as_float(r[0]) + __uint_as_float(r[1]);
    }
#pragma unroll
    for (int t = 0; t < 4; t++) {      // partner lane ^ 16: even rows keep t, odd rows t + 4
        const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(a[t]), __float_as_uint(a[t + 4]), false, false);
        b[t] = __uint_as_float(r[0]) + __uint_as_float(r[1]);
    }
    const bool b3 = (lane & 8) != 0, b2 = (lane & 4) != 0;
#pragma unroll
    for (int t = 0; t < 2; t++) {      // partner lane ^ 8
        const float keep = b3 ? b[t + 2] : b[t], send = b3 ? b[t] : b[t + 2];
        c[t] = keep + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(send), 0x128, 0xf, 0xf, true));
    }
    const float keep = b2 ? c[1] : c[0], send = b2 ? c[0] : c[1];
    float z = keep;
    {                                   // partner lane ^ 4 = mirror the half row (^7), then reverse the quad (^3)
        const int t = __builtin_amdgcn_update_dpp(0, __float_as_int(send), 0x141, 0xf, 0xf, true);
        z += __int_as_float(__builtin_amdgcn_update_dpp(0, t, 0x1B, 0xf, 0xf, true));
    }
    z += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(z), 0x4E, 0xf, 0xf, true));   // ^ 2
    z += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(z), 0xB1, 0xf, 0xf, true));   // ^ 1
    return z;
}

#ifndef GRAD_OWNER_T
#define GRAD_OWNER_T unsigned char
#endif

// A wavefront (= one block: nothing is shared inside a block, and small blocks pack the LDS of a CU best) takes NQ
// consecutive rows of the sorted order, four at a time, lane k owning neighbour slot k, and combines the
// contributions per target in a two-way LDS table: the first slot of target m is m mod H.  Targets are sorted
// positions and the neighbours of consecutive rows are mostly positions close by, which this mapping sends to
// distinct slots - the table is a dense window around the tile that wraps around for the far targets; a target
// whose first slot holds another point tries a second one, shifted by a hash of m / H (so a far run of
// consecutive positions stays a run of consecutive slots).  Who may use a slot is settled per instruction without
// compare-and-swap loops: every lane writes its lane number into the slot's owner cell and reads it back; the
// lane that finds its own number owns the slot for this instruction and may use it if the slot's tag is its
// target (or the slot is empty: it takes it).  Everybody else - the loser of a collision, a second lane with the
// same target (repeated index in a row), a target whose slots both hold other points - sends its contribution to
// memory directly.  So the update of a table entry is a plain LDS read-add-write that no two lanes of an
// instruction share.  The rows' own shares (-sum over the slots) are summed for four rows and four coordinates
// at once (fgc_wave_reduce16) and go to slots taken for the tile's own rows up front.
// Loads run two steps ahead of the arithmetic: while step s is combined on chip, the neighbour coordinates of
// step s + 1 are being gathered and the index / upstream-gradient rows of step s + 2 are on their way.
// The gradient is accumulated in the sorted order too (gxs, rows of D4 * 4 floats): the tables are flushed with
// the coordinates of a target in adjacent lanes and neighbouring targets in neighbouring lanes, which for the
// window part are neighbouring addresses; k_unsort_grad moves the rows to the original order.
// PACK (D <= 3): a table entry is one float4 (x, y, z, tag) - value and tag in one 16-byte LDS access.
// D4T: float4 groups per point where the kernel is built for exactly that many (1 or 2: up to 8 coordinates), 0 = any.
template <bool PACK, int D4T>
__global__ __launch_bounds__(64) void k_knn_grad_sorted(const float *__restrict__ gd, const int *__restrict__ nbr,
                                                        const float4 *__restrict__ xs,
                                                        const uint32_t *__restrict__ order, float *__restrict__ gxs,
                                                        int64_t n, int K, int D, int H, int *__restrict__ status)
{
    extern __shared__ __align__(16) unsigned char s_raw[];
    const int lane = fgc_lane();
    const int D4 = PACK ? 1 : (D4T ? D4T : (D + 3) >> 2);
    const int ld = D4 * 4;                     // floats per row of xs and gxs
    float4 *vals = (float4 *)s_raw;            // [H][D4]
    unsigned *tags = PACK ? (unsigned *)vals + 3 : (unsigned *)(s_raw + (size_t)H * 16 * D4);
    GRAD_OWNER_T *owner = (GRAD_OWNER_T *)(s_raw + (PACK ? (size_t)H * 16 : (size_t)H * (16 * (size_t)D4 + 4)));
    constexpr int KS = PACK ? 4 : 1;           // words between the tags of consecutive slots
    constexpr int NQ = PACK ? GSW : GW;        // rows per wavefront
    static_assert(GU == 4 && NQ % GU == 0 && NQ <= 64, "fgc_wave_reduce16 sums four rows of four coordinates");
    if (PACK) {
        for (int t = lane; t < H; t += 64) vals[t] = make_float4(0.f, 0.f, 0.f, __uint_as_float(GRAD_EMPTY));
    } else {
        for (int t = lane; t < H; t += 64) tags[t] = GRAD_EMPTY;
        for (int t = lane; t < H * D4; t += 64) vals[t] = make_float4(0.f, 0.f, 0.f, 0.f);
    }
    const unsigned hmask = (unsigned)H - 1u;
    const int hbits = 31 - __builtin_clz((unsigned)H);
    const int64_t wave0 = (int64_t)blockIdx.x * NQ;
    // slots of the tile's own rows (consecutive positions: distinct slots); lane q keeps row q's original index
    unsigned my_order = 0u;
    if (lane < NQ && wave0 + lane < n) {
        tags[(((unsigned)(wave0 + lane)) & hmask) * KS] = (unsigned)(wave0 + lane);
        my_order = order[wave0 + lane];
    }
    const int *__restrict__ nb0 = nbr + wave0 * K;           // the tile's neighbour rows
    bool bad = false;

#ifdef FGC_GRAD_COUNTERS
    unsigned n_pairs = 0, n_ovf = 0;
#endif

    // stage A of a step (rows q .. q + 3, slots k0 .. k0 + 63): neighbour positions and upstream gradients
    auto stage_a = [&](int q, int k0, int (&m)[GU], float (&g)[GU]) {
        const int k = k0 + lane;
#pragma unroll
        for (int u = 0; u < GU; u++) {
            m[u] = -1; g[u] = 0.f;
            if (q + u < NQ && wave0 + q + u < n && k < K) {
                m[u] = nb0[(q + u) * K + k];
                g[u] = gd[(int64_t)fgc_readlane_i((int)my_order, q + u) * K + k];
            }
        }
    };
    // stage B: the neighbours' coordinates (first float4 group)
    auto stage_b = [&](int (&m)[GU], float4 (&x)[GU]) {
#pragma unroll
        for (int u = 0; u < GU; u++) {
            if (m[u] >= n) { bad = true; m[u] = -1; }
            x[u] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (m[u] >= 0) x[u] = xs[(int64_t)m[u] * D4];
        }
    };
    // may this lane use slot s for target mm in this instruction?
    auto try_slot = [&](bool want, unsigned s, unsigned mm) -> bool {
        const unsigned tag = want ? tags[s * KS] : 0u;
        if (want) owner[s] = (GRAD_OWNER_T)lane;
        asm volatile("" ::: "memory");                     // the cell is read back from LDS, not from the register
        const bool win = want && owner[s] == (GRAD_OWNER_T)lane;
        const bool ok = win && (tag == mm || tag == GRAD_EMPTY);
        if (ok && tag == GRAD_EMPTY) tags[s * KS] = mm;
        asm volatile("" ::: "memory");
        return ok;
    };

    int m1[GU], m2[GU];
    float g1[GU], g2[GU];
    float4 x1[GU];
    int qa = 0, ka = 0;                        // step whose stage A is issued next
    auto next_step = [&](int &q, int &k0) { k0 += 64; if (k0 >= K) { k0 = 0; q += GU; } };
    stage_a(qa, ka, m1, g1); next_step(qa, ka);
    stage_b(m1, x1);
    stage_a(qa, ka, m2, g2); next_step(qa, ka);
    int qc = 0, kc = 0;                        // step being combined
    while (qc < NQ) {
        int m[GU];
        float g[GU];
        float4 xm[GU];
#pragma unroll
        for (int u = 0; u < GU; u++) { m[u] = m1[u]; g[u] = g1[u]; xm[u] = x1[u]; m1[u] = m2[u]; g1[u] = g2[u]; }
        stage_b(m1, x1);
        stage_a(qa, ka, m2, g2); next_step(qa, ka);

        int sl[GU];
#pragma unroll
        for (int u = 0; u < GU; u++) {
            const bool valid = m[u] >= 0;
            const unsigned mm = (unsigned)m[u];
            const unsigned s1 = mm & hmask;
            bool ok = try_slot(valid, s1, mm);
            unsigned s = s1;
            const bool again = valid && !ok;
            if (fgc_ballot(again)) {
                // an odd shift: never the first slot again (its owner of this instruction may be a lane with
                // the same target)
                const unsigned s2 = (s1 + ((((mm >> hbits) * 2654435761u) >> 20) | 1u)) & hmask;
                const bool ok2 = try_slot(again, s2, mm);
                if (again) { ok = ok2; s = s2; }
            }
            sl[u] = ok ? (int)s : -1;
#ifdef FGC_GRAD_COUNTERS
            n_pairs += (unsigned)__popcll(fgc_ballot(valid));
            n_ovf += (unsigned)__popcll(fgc_ballot(valid && !ok));
#endif
        }
        float4 addp[GU];       // the even float4 group of an overflowing pair, until its partner is known
#pragma unroll
        for (int u = 0; u < GU; u++) addp[u] = make_float4(0.f, 0.f, 0.f, 0.f);
        for (int c4 = 0; c4 < D4; c4++) {
            float red[16];
#pragma unroll
            for (int u = 0; u < GU; u++) {
                const int64_t row = (wave0 + qc + u < n) ? wave0 + qc + u : 0;
                const float4 xi = xs[row * D4 + c4];
                float4 add = make_float4(0.f, 0.f, 0.f, 0.f);
                if (m[u] >= 0) {
                    const float4 xn = (PACK || c4 == 0) ? xm[u] : xs[(int64_t)m[u] * D4 + c4];
                    const float gg = 2.f * g[u];
                    add = make_float4(gg * (xn.x - xi.x), gg * (xn.y - xi.y), gg * (xn.z - xi.z), gg * (xn.w - xi.w));
                }
                red[u * 4 + 0] = add.x; red[u * 4 + 1] = add.y; red[u * 4 + 2] = add.z; red[u * 4 + 3] = add.w;
                if (sl[u] >= 0) {
                    float4 v = vals[sl[u] * D4 + c4];
                    v.x += add.x; v.y += add.y; v.z += add.z;
                    if (!PACK) v.w += add.w;              // PACK: the fourth word is the tag, written back as read
                    vals[sl[u] * D4 + c4] = v;
                }
                const bool ovf = m[u] >= 0 && sl[u] < 0;
                const unsigned long long om = fgc_ballot(ovf);
                if (om) {
                    // float4 groups leave in pairs (one 32-byte update per target), an unpaired last one alone
                    if (!PACK && !(c4 & 1) && c4 + 1 < D4) addp[u] = add;
                    else if (!PACK && (c4 & 1)) grad_overflow_add8(om, ovf, m[u], addp[u], add, (c4 - 1) * 4, D, ld, gxs, lane);
                    else grad_overflow_add(om, ovf, m[u], add, c4 * 4, D, ld, gxs, lane);
                }
            }
            // the rows' own shares: lane L holds the total of row L >> 4, coordinate c4 * 4 + ((L >> 2) & 3)
            const float tot = fgc_wave_reduce16(red, lane);
            const int su = lane >> 4, se = (lane >> 2) & 3;
            const int64_t sr = wave0 + qc + su;
            if ((lane & 3) == 0 && sr < n && c4 * 4 + se < D) {
                float *p = (float *)vals + ((size_t)(((unsigned)sr) & hmask) * D4 + c4) * 4 + se;
                *p -= tot;
            }
        }
        next_step(qc, kc);
    }
    // flush: one lane per (slot, coordinate); for the window part of the table neighbouring lanes hold
    // neighbouring addresses
    const float *vflat = (const float *)vals;
    for (int t = lane; t < H * ld; t += 64) {
        const int sl = t / ld, c = t - sl * ld;
        const unsigned m = tags[sl * KS];
        if (m == GRAD_EMPTY || c >= D) continue;
        const float v = vflat[t];
        if (v != 0.f) atomicAdd(&gxs[(int64_t)m * ld + c], v);
    }
    if (bad && status) atomicOr(&status[0], FGC_ST_BAD_INDEX);
#ifdef FGC_GRAD_COUNTERS
    if (status && lane == 0) { atomicAdd(&status[2], (int)(n_pairs >> 6)); atomicAdd(&status[3], (int)(n_ovf >> 6)); }
#endif
}

// rows of the sorted-space gradient to the original order: gx[order[r], :] = gxs[r, :D]; one thread per float4 group
__global__ __launch_bounds__(256) void k_unsort_grad(const float4 *__restrict__ gxs, const uint32_t *__restrict__ order,
                                                     int64_t n, int D, int D4, float *__restrict__ gx, int ldg)
{
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= n * D4) return;
    int64_t r = t;
    int c4 = 0;
    if (D4 > 1) { r = t / D4; c4 = (int)(t - r * D4); }
    const float4 v = gxs[t];
    float *dst = gx + (int64_t)order[r] * ldg + c4 * 4;
    dst[0] = v.x;
    if (c4 * 4 + 1 < D) dst[1] = v.y;
    if (c4 * 4 + 2 < D) dst[2] = v.z;
    if (c4 * 4 + 3 < D) dst[3] = v.w;
}

extern "C" size_t fgc_binned_select_knn_grad_sorted_workspace_bytes(int64_t n_vert, int32_t n_coords)
{
    if (n_vert < 0 || n_coords < 1) return 0;
    // the sorted copy of the points and the gradient in sorted order, both padded to whole float4 groups
    return 2 * fgc_align((size_t)(n_vert > 0 ? n_vert : 1) * (size_t)((n_coords + 3) / 4) * 16);
}

extern "C" int fgc_binned_select_knn_grad_sorted_f32(const float *d_grad_distsq, const int32_t *d_nbr_sorted,
                                                     const float *d_coords, const int32_t *d_order,
                                                     float *d_grad_coords, int64_t n_vert, int32_t K,
                                                     int32_t n_coords, int32_t *d_status, void *d_ws,
                                                     size_t ws_bytes, void *stream)
{
    return fgc_binned_select_knn_grad_sorted_ld_f32(d_grad_distsq, d_nbr_sorted, d_coords, n_coords, d_order,
                                                    d_grad_coords, n_coords, n_vert, K, n_coords, d_status, d_ws,
                                                    ws_bytes, stream);
}

extern "C" int fgc_binned_select_knn_grad_sorted_ld_f32(const float *d_grad_distsq, const int32_t *d_nbr_sorted,
                                                        const float *d_coords, int32_t ld_coords,
                                                        const int32_t *d_order, float *d_grad_coords,
                                                        int32_t ld_grad_coords, int64_t n_vert, int32_t K,
                                                        int32_t n_coords, int32_t *d_status, void *d_ws,
                                                        size_t ws_bytes, void *stream)
{
    if (ld_coords < n_coords || ld_grad_coords < n_coords) return FGC_EINVAL;
    if (n_vert < 0 || K < 1 || n_coords < 1 || n_coords > 128) return FGC_EINVAL;
    if (n_vert >= (1ll << 31) - 1) return FGC_EINVAL;
    if (n_vert == 0) return FGC_OK;
    if (!d_grad_distsq || !d_nbr_sorted || !d_coords || !d_order || !d_grad_coords) return FGC_EINVAL;
    if (!d_ws || ws_bytes < fgc_binned_select_knn_grad_sorted_workspace_bytes(n_vert, n_coords)) return FGC_ENOSPACE;
    hipStream_t s = (hipStream_t)stream;
    const int D4 = (n_coords + 3) / 4;
    const size_t half = fgc_align((size_t)n_vert * D4 * 16);
    float4 *xs = (float4 *)d_ws;
    float *gxs = (float *)((char *)d_ws + half);
    hipLaunchKernelGGL(k_sorted_points, dim3((unsigned)fgc_cdiv(n_vert * D4, 256)), dim3(256), 0, s, d_coords,
                       (int)ld_coords, (const uint32_t *)d_order, n_vert, (int)n_coords, D4, xs, (float4 *)gxs);
    FGC_LAUNCH_CHECK();
    if (n_coords <= 3) {
        const unsigned blocks = (unsigned)fgc_cdiv(n_vert, GSW);
        hipLaunchKernelGGL((k_knn_grad_sorted<true, 1>), dim3(blocks), dim3(64), (size_t)GSH * (16 + sizeof(GRAD_OWNER_T)), s, d_grad_distsq,
                           d_nbr_sorted, (const float4 *)xs, (const uint32_t *)d_order, gxs, n_vert, (int)K,
                           (int)n_coords, GSH, d_status);
    } else {
        const int H = grad_table_size(n_coords);
        const unsigned blocks = (unsigned)fgc_cdiv(n_vert, GW);
#define FGC_GRAD_WIDE(D4T)                                                                                              \
    hipLaunchKernelGGL((k_knn_grad_sorted<false, D4T>), dim3(blocks), dim3(64), (size_t)H * (8 + 16 * (size_t)D4), s,   \
                       d_grad_distsq, d_nbr_sorted, (const float4 *)xs, (const uint32_t *)d_order, gxs, n_vert, (int)K, \
                       (int)n_coords, H, d_status)
        if (D4 == 1) FGC_GRAD_WIDE(1);
        else if (D4 == 2) FGC_GRAD_WIDE(2);
        else FGC_GRAD_WIDE(0);
#undef FGC_GRAD_WIDE
    }
    FGC_LAUNCH_CHECK();
    hipLaunchKernelGGL(k_unsort_grad, dim3((unsigned)fgc_cdiv(n_vert * D4, 256)), dim3(256), 0, s, (const float4 *)gxs,
                       (const uint32_t *)d_order, n_vert, (int)n_coords, D4, d_grad_coords, (int)ld_grad_coords);
    FGC_LAUNCH_CHECK();
    return FGC_OK;
}

// ---------------------------------------------------------------------------
// select_with_default
// ---------------------------------------------------------------------------
// T is the element as a bit pattern (uint32_t for float / int32, uint64_t for int64 / double).
// Narrow feature rows (F <= 8): one thread per (v, k) pair copies the whole row - one index load, no division.
template <typename T>
__global__ __launch_bounds__(256) void k_select_rows(const int64_t *__restrict__ idx, const T *__restrict__ feat,
                                                     T *__restrict__ out, int64_t n_pairs, int F, int64_t n_rows,
                                                     T dflt)
{
    const int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (p >= n_pairs) return;
    const int64_t raw = idx[p];
    int64_t m = raw;
    if (m < 0) m += n_rows;  // torch advanced indexing wraps negative indices other than the -1 default
    const bool take = !(raw == -1 || m < 0 || m >= n_rows);
    T v[8];
#pragma unroll
    for (int f = 0; f < 8; f++) v[f] = (take && f < F) ? feat[m * F + f] : dflt;
#pragma unroll
    for (int f = 0; f < 8; f++)
        if (f < F) out[p * F + f] = v[f];
}

// Wide feature rows: one thread per output element, consecutive lanes on consecutive features.
template <typename T>
__global__ __launch_bounds__(256) void k_select_elems(const int64_t *__restrict__ idx, const T *__restrict__ feat,
                                                      T *__restrict__ out, int64_t n_pairs, int F, int64_t n_rows,
                                                      T dflt)
{
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= n_pairs * F) return;
    int64_t p;
    if (n_pairs * F < (1ll << 31)) p = (int64_t)((unsigned)t / (unsigned)F); else p = t / F;
    const int f = (int)(t - p * F);
    const int64_t raw = idx[p];
    int64_t m = raw;
    if (m < 0) m += n_rows;
    out[t] = (raw == -1 || m < 0 || m >= n_rows) ? dflt : feat[m * F + f];
}

template <typename T>
static int select_with_default_launch(const int64_t *d_idx, const T *d_feat, T *d_out, int64_t n_vert, int32_t K,
                                      int32_t n_feat, int64_t n_feat_rows, T dflt, void *stream)
{
    if (n_vert < 0 || K < 0 || n_feat < 0) return FGC_EINVAL;
    const int64_t pairs = n_vert * K, total = pairs * n_feat;
    if (total == 0) return FGC_OK;
    if (n_feat <= 8)
        hipLaunchKernelGGL((k_select_rows<T>), dim3((unsigned)fgc_cdiv(pairs, 256)), dim3(256), 0,
                           (hipStream_t)stream, d_idx, d_feat, d_out, pairs, (int)n_feat, n_feat_rows, dflt);
    else
        hipLaunchKernelGGL((k_select_elems<T>), dim3((unsigned)fgc_cdiv(total, 256)), dim3(256), 0,
                           (hipStream_t)stream, d_idx, d_feat, d_out, pairs, (int)n_feat, n_feat_rows, dflt);
    FGC_LAUNCH_CHECK();
    return FGC_OK;
}

extern "C" int fgc_select_with_default_f32(const int64_t *d_idx, const float *d_feat, float *d_out,
                                           int64_t n_vert, int32_t K, int32_t n_feat, int64_t n_feat_rows,
                                           float default_value, void *stream)
{
    return select_with_default_launch<uint32_t>(d_idx, (const uint32_t *)d_feat, (uint32_t *)d_out, n_vert, K,
                                                n_feat, n_feat_rows, __builtin_bit_cast(uint32_t, default_value),
                                                stream);
}

extern "C" int fgc_select_with_default_b64(const int64_t *d_idx, const void *d_feat, void *d_out, int64_t n_vert,
                                           int32_t K, int32_t n_feat, int64_t n_feat_rows,
                                           uint64_t default_bits, void *stream)
{
    return select_with_default_launch<uint64_t>(d_idx, (const uint64_t *)d_feat, (uint64_t *)d_out, n_vert, K,
                                                n_feat, n_feat_rows, default_bits, stream);
}

// ---------------------------------------------------------------------------
// GravNet aggregation
// ---------------------------------------------------------------------------
// PW lanes (a power of two <= 64, >= min(P, 64)) own one point; lane p owns
// feature p (P > 64: p, p + 64, ... handled by an outer loop over feature
// blocks).  The neighbour loop runs over the K slots in order, so the float
// sum has the same order as a sequential reference.
template <int PW>
__global__ __launch_bounds__(256) void k_gravnet_fwd(const int64_t *__restrict__ idx,
                                                     const float *__restrict__ dsq,
                                                     const float *__restrict__ feat, int ldf, int64_t nf,
                                                     float *__restrict__ fmean, float *__restrict__ fmax, int ldo,
                                                     int *__restrict__ argmax, int64_t n, int K, int P,
                                                     int *__restrict__ status)
{
    constexpr int QPW = 64 / PW;
    const int lane = fgc_lane();
    const int sub = lane / PW, pl = lane % PW;
    const int64_t wave = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int64_t i = wave * QPW + sub;
    if (i >= n) return;
    // The PW lanes of a point first fetch PW neighbour slots together (one coalesced read of the index and
    // distance rows, one expf per slot instead of one per lane and slot), then every lane walks the slots in
    // order with the neighbour and its weight broadcast from the lane that fetched them; the gathers of eight
    // slots are in flight together.
    const int gbase = sub * PW;
    bool bad = false;
    for (int p0 = 0; p0 < P; p0 += PW) {
        const int p = p0 + pl;
        const bool pv = p < P;
        float s = 0.f, mx = 0.f;
        int am = 0;
        for (int kb = 0; kb < K; kb += PW) {
            const int kk = kb + pl;
            int m_l = -1;
            float w_l = 0.f;
            if (kk < K) {
                const int64_t mi = idx[i * K + kk];
                bad = bad || mi >= nf;             // a neighbour past the feature rows: flagged, counts as padding
                m_l = (mi >= nf) ? -1 : (int)mi;
                w_l = expf(-10.f * dsq[i * K + kk]);
            }
            const int cnt = min(PW, K - kb);
            for (int j0 = 0; j0 < cnt; j0 += 8) {
                float f[8], w[8];
#pragma unroll
                for (int u = 0; u < 8; u++) {
                    const int src = gbase + min(j0 + u, PW - 1);
                    const int m = __shfl(m_l, src, 64);
                    w[u] = __shfl(w_l, src, 64);
                    f[u] = (m >= 0 && pv && j0 + u < cnt) ? feat[(int64_t)m * ldf + p] : 0.f;
                }
#pragma unroll
                for (int u = 0; u < 8; u++) {
                    if (j0 + u < cnt) {
                        const float v = f[u] * w[u];
                        s += v;
                        if ((kb + j0 + u) == 0 || v > mx) { mx = v; am = kb + j0 + u; }
                    }
                }
            }
        }
        if (pv) {
            fmean[i * ldo + p] = s / (float)K;
            fmax[i * ldo + p] = mx;
            if (argmax) argmax[i * P + p] = am;
        }
    }
    if (bad && status) atomicOr(&status[0], FGC_ST_BAD_INDEX);
}

template <int PW>
__global__ __launch_bounds__(256) void k_gravnet_bwd(const int64_t *__restrict__ idx,
                                                     const float *__restrict__ dsq,
                                                     const float *__restrict__ feat, int ldf, int64_t nf,
                                                     const int *__restrict__ argmax,
                                                     const float *__restrict__ gmean,
                                                     const float *__restrict__ gmax, int ldg,
                                                     float *__restrict__ gfeat, int ldgf,
                                                     float *__restrict__ gdsq, int64_t n, int K, int P,
                                                     int *__restrict__ status)
{
    constexpr int QPW = 64 / PW;
    const int lane = fgc_lane();
    const int sub = lane / PW, pl = lane % PW;
    const int gbase = sub * PW;
    const int64_t wave = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int64_t i = wave * QPW + sub;
    const bool qv = i < n;
    const float invK = 1.0f / (float)K;
    // Slots are fetched PW at a time: lane j of the point's group reads slot kb + j (index, weight).  They are
    // then visited eight at a time: every lane takes its own feature(s) of the eight neighbours (gathers in
    // flight together), adds w * c to their feature gradients and keeps one partial dot product per slot; an
    // exchange-halving across the group's lanes (fgc_group_reduce8) leaves the eight dot products spread over
    // the group, and the lanes holding them write grad_distsq.
    bool bad = false;
    const bool single = P <= PW;      // one feature per lane: its upstream gradients stay in registers
    float cm0 = 0.f, gx0 = 0.f;
    int am0 = -1;
    if (single && qv && pl < P) {
        cm0 = gmean[i * ldg + pl] * invK;
        gx0 = gmax[i * ldg + pl];
        am0 = argmax[i * P + pl];
    }
    for (int kb = 0; kb < K; kb += PW) {
        const int kk = kb + pl;
        int m_l = -1;
        float w_l = 0.f;
        if (qv && kk < K) {
            const int64_t mi = idx[i * K + kk];
            bad = bad || mi >= nf;                 // as in the forward: flagged, counts as padding
            m_l = (mi >= nf) ? -1 : (int)mi;
            w_l = expf(-10.f * dsq[i * K + kk]);
        }
        const int cnt = min(PW, K - kb);
        for (int j0 = 0; j0 < cnt; j0 += 8) {
            float vals[8];
            int m[8];
            float w[8];
#pragma unroll
            for (int u = 0; u < 8; u++) {
                vals[u] = 0.f;
                m[u] = __shfl(m_l, gbase + ((j0 + u) & (PW - 1)), 64);
                w[u] = __shfl(w_l, gbase + ((j0 + u) & (PW - 1)), 64);
                if (j0 + u >= cnt) m[u] = -1;
            }
            for (int p0 = 0; p0 < P; p0 += PW) {
                const int p = p0 + pl;
                const bool pv = qv && p < P;
                float cm = cm0, gx = gx0;
                int am = am0;
                if (!single) {
                    cm = pv ? gmean[i * ldg + p] * invK : 0.f;
                    gx = pv ? gmax[i * ldg + p] : 0.f;
                    am = pv ? argmax[i * P + p] : -1;
                }
                float f[8];
#pragma unroll
                for (int u = 0; u < 8; u++) f[u] = (m[u] >= 0 && pv) ? feat[(int64_t)m[u] * ldf + p] : 0.f;
#pragma unroll
                for (int u = 0; u < 8; u++) {
                    if (m[u] >= 0 && pv) {
                        const float c = cm + (am == kb + j0 + u ? gx : 0.f);
                        vals[u] += f[u] * c;
                        atomicAdd(&gfeat[(int64_t)m[u] * ldgf + p], w[u] * c);
                    }
                }
            }
            // the eight dot products, summed over the group's lanes by exchange-halving (DPP and lane swaps, no
            // LDS permutes); the lane holds the total of slot j0 + ul and writes it with that slot's weight
            const float tot = fgc_group_reduce8<PW>(vals, lane);
            const int ul = pl * 8 / PW;
            const float wu = __shfl(w_l, gbase + ((j0 + ul) & (PW - 1)), 64);
            if (qv && (pl % (PW / 8)) == 0 && j0 + ul < cnt) gdsq[i * K + kb + j0 + ul] = -10.f * wu * tot;
        }
    }
    if (bad && status) atomicOr(&status[0], FGC_ST_BAD_INDEX);
}

// ---------------------------------------------------------------------------
// The same backward for callers that have the neighbour rows in the search's sorted order (the fused GravNet
// layer): the feature gradients of a tile of consecutive sorted rows are combined on chip before they go to memory.
// ---------------------------------------------------------------------------
// k_gravnet_bwd issues one atomic 128-byte row update per (point, slot) pair and is bound by the rate of those
// updates.  Rows that are consecutive in the sorted order share most of their neighbours, so a block of GT_WAVES
// wavefronts here takes GT_WAVES * GT consecutive sorted rows and
//   1. each wavefront loads what its GT rows need into LDS (per pair the weight and the target's original index -
//      the target's sorted position stays in a register; per row the upstream gradients and arg-max slots), then,
//      per row pair with lane = feature, gathers the neighbours' feature rows and forms the dot products for
//      grad_distsq as k_gravnet_bwd does - but does not touch grad_feat;
//   2. the block groups all its records by target with a counting sort on the low bits of the target's sorted
//      position (lane = record; LDS integer atomics for the ranks, one block-wide scan over the bucket counts);
//   3. each wavefront walks its share of the grouped records with lane = feature (64 / PW records per
//      instruction, four records per 16-byte LDS read, the next four requested before the current four are used),
//      recomputes each pair's contribution w * (g_mean / K + [argmax == slot] * g_max) from the rows kept in LDS,
//      sums it in a register while the target stays the same, and issues ONE row update per run of equal targets.
// For 32 rows with K = 40 (64) that is 3.5 (3.9) times fewer updates (sampled on learned 4-D coordinates, 1024
// buckets), and the result is the same sum in another order.  What the block needs in LDS decides how many
// wavefronts a CU holds, and the kernel's time follows that number: 9 bytes per (row, feature), 4 KB of bucket
// counts and 12 bytes per pair - 38 KB at K = 64, P = 32 (four blocks per CU), 29 KB at K = 40 (five).
#ifndef GT
#define GT 8             // sorted rows per wavefront
#endif
#ifndef GT_WAVES
#define GT_WAVES 4       // wavefronts per block: the block's tile is GT_WAVES * GT rows
#endif
#ifndef GT_BUCKETS
#define GT_BUCKETS 1024  // buckets of the counting sort (two targets that share a bucket split each other's runs)
#endif

template <int PW>
__global__ __launch_bounds__(GT_WAVES * 64) void k_gravnet_bwd_tile(
    const int *__restrict__ nbr, const uint32_t *__restrict__ order, const float *__restrict__ dsq,
    const float *__restrict__ feat, int ldf, const int *__restrict__ argmax, const float *__restrict__ gmean,
    const float *__restrict__ gmax, int ldg, float *__restrict__ gfeat, int ldgf, float *__restrict__ gdsq, int64_t n,
    int K, int P, int *__restrict__ status)
{
    constexpr int QPW = 64 / PW;               // rows per pass of step 1b, records per instruction of step 3
    constexpr int GTB = GT_WAVES * GT;         // rows of the block's tile
    constexpr int NSEG3 = GT_WAVES * QPW;      // lane groups that share the walk of step 3
    constexpr int BPT = GT_BUCKETS / (GT_WAVES * 64);   // buckets per thread in the scan
    static_assert(GT % QPW == 0 && GTB <= 256 && GT_BUCKETS % (GT_WAVES * 64) == 0, "tile shape");
    extern __shared__ __align__(16) unsigned char s_raw[];
    const int lane = fgc_lane();
    const int wv = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int sub = lane / PW, pl = lane % PW;
    // LDS: upstream rows [GTB][PW] (g_mean / K without and with g_max added, and the arg-max slot as a byte), bucket
    // counts, the wavefronts' record totals, then the pairs: first as two arrays (weight, target's original index)
    // indexed [row][slot], later - over the same bytes - as three arrays of the grouped records (target's original
    // index, weight, row and slot), padded for the walk of step 3
    const int KP = (K + 7) & ~7;               // slots per row in LDS, padded to whole groups of eight
    const int E = GTB * KP, EP = E + 4 * NSEG3;
    float2 *rows_cg = (float2 *)s_raw;
    int *hist = (int *)(rows_cg + GTB * PW);
    int *wsum = hist + GT_BUCKETS;
    unsigned char *rec0 = (unsigned char *)(wsum + 4 * ((GT_WAVES + 3) / 4));
    float *ew = (float *)rec0;
    int *eo = (int *)(ew + E);
    int *st = (int *)rec0;
    float *sw = (float *)(st + EP);
    int *sz = (int *)(sw + EP);
    unsigned char *rows_am = (unsigned char *)(sz + EP);
    const int tw0 = wv * GT;                                      // the wavefront's first row inside the tile
    const int64_t r0 = (int64_t)blockIdx.x * GTB + tw0;           // ... and in the sorted order
    const float invK = 1.0f / (float)K;
    const unsigned ldf4 = 4u * (unsigned)ldf;
    bool bad = false;
    for (int t = threadIdx.x; t < GT_BUCKETS; t += GT_WAVES * 64) hist[t] = 0;

    // ---- 1a. everything the wavefront's rows need except the feature gathers, all loads independent of each
    //      other: lane t keeps row t's original index; per row (lane = slot) the neighbour positions, their weights
    //      and original indices go to LDS (the positions also stay in registers for step 2); per QPW rows (lane =
    //      feature) the upstream gradients and arg-max slots ----
    const unsigned my_qo = (lane < GT && r0 + lane < n) ? order[r0 + lane] : 0u;
    int rm[GT];
#pragma unroll
    for (int t = 0; t < GT; t++) {
        const bool qv = r0 + t < n;
        const int64_t qo = (int64_t)(unsigned)fgc_readlane_i((int)my_qo, t);
        int m = -1, o = -1;                      // no neighbour: original index -1
        float w = 0.f;
        if (qv && lane < K) {
            m = nbr[(r0 + t) * K + lane];
            w = expf(-10.f * dsq[qo * K + lane]);
            if (m >= n) { bad = true; m = -1; }
            if (m >= 0) o = (int)order[m];
        }
        rm[t] = m;
        if (lane < KP) { ew[(tw0 + t) * KP + lane] = w; eo[(tw0 + t) * KP + lane] = o; }
    }
    for (int t0 = 0; t0 < GT; t0 += QPW) {
        const int t = t0 + sub;
        const bool qv = r0 + t < n;
        const int64_t qo = (int64_t)(unsigned)__shfl((int)my_qo, t, 64);
        float cm = 0.f, gx = 0.f;
        int am = 255;
        if (qv && pl < P) {
            cm = gmean[qo * ldg + pl] * invK;
            gx = gmax[qo * ldg + pl];
            am = argmax[qo * P + pl] & 255;          // slots are < 64; -1 (no neighbour) becomes 255
        }
        rows_cg[(tw0 + t) * PW + pl] = make_float2(cm, cm + gx);      // without and with the arg-max share
        rows_am[(tw0 + t) * PW + pl] = (unsigned char)am;
    }

    // Step 1b reads, with lane = feature, what step 1a wrote to LDS with lane = slot: other lanes of the same
    // wavefront.  The LDS queue of a wavefront keeps its order, so no block barrier is needed, but the compiler must
    // not move a read above a write of another lane: a wavefront-level fence pins the order.
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

    // ---- 1b. dot products for grad_distsq: lane = feature, QPW rows at a time, eight slots per step; the feature
    //      gathers of the next step are requested before the current one is reduced ----
    const int n_grp = (K + 7) >> 3;
    for (int t0 = 0; t0 < GT; t0 += QPW) {
        const int t = t0 + sub, tb = tw0 + t;
        const bool qv = r0 + t < n;
        const int64_t qo = (int64_t)(unsigned)__shfl((int)my_qo, t, 64);
        const float2 cg = rows_cg[tb * PW + pl];
        const float cm = cg.x, cmgx = cg.y;
        const int am = rows_am[tb * PW + pl];
        auto gather = [&](int g, float (&f)[8]) {
            // the eight original indices of the group with two 16-byte LDS reads
            const int4 oa = *(const int4 *)&eo[tb * KP + g * 8], ob = *(const int4 *)&eo[tb * KP + g * 8 + 4];
            const int oo[8] = {oa.x, oa.y, oa.z, oa.w, ob.x, ob.y, ob.z, ob.w};
#pragma unroll
            for (int u = 0; u < 8; u++) {
                f[u] = 0.f;
                if (oo[u] >= 0 && pl < P) f[u] = *(const float *)((const char *)feat + (__umul24((unsigned)oo[u], ldf4) + 4u * (unsigned)pl));
            }
        };
        float fcur[8], fnext[8];
        gather(0, fcur);
        for (int g = 0; g < n_grp; g++) {
            if (g + 1 < n_grp) gather(g + 1, fnext);
            float vals[8];
#pragma unroll
            for (int u = 0; u < 8; u++) vals[u] = fcur[u] * (am == g * 8 + u ? cmgx : cm);
            const float tot = fgc_group_reduce8<PW>(vals, lane);
            const int k = g * 8 + pl * 8 / PW;          // the slot whose total the lane holds
            if (qv && (pl % (PW / 8)) == 0 && k < K) gdsq[qo * K + k] = -10.f * ew[tb * KP + k] * tot;
#pragma unroll
            for (int u = 0; u < 8; u++) fcur[u] = fnext[u];
        }
    }

    // ---- 2. group the block's records by target: counting sort on the low bits of the target's sorted position ----
    __syncthreads();                                  // the bucket counts are zero
    int ro[GT], rp[GT];
    float rw[GT];
#pragma unroll
    for (int t = 0; t < GT; t++) {                    // lane = slot of the wavefront's row t
        ro[t] = 0; rp[t] = 0; rw[t] = 0.f;
        if (lane < K) { rw[t] = ew[(tw0 + t) * KP + lane]; ro[t] = eo[(tw0 + t) * KP + lane]; }
        if (rm[t] >= 0) rp[t] = atomicAdd(&hist[rm[t] & (GT_BUCKETS - 1)], 1);     // rank inside the bucket
    }
    __syncthreads();                                  // all ranks taken, every record of the block is in registers
    // exclusive scan of the bucket counts: consecutive buckets per thread, across the lanes, across the wavefronts
    int cntv[BPT], run = 0;
    const int b0 = (int)threadIdx.x * BPT;
#pragma unroll
    for (int b = 0; b < BPT; b++) { cntv[b] = hist[b0 + b]; run += cntv[b]; }
    int incl = run;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const int up = __shfl_up(incl, o, 64);
        if (lane >= o) incl += up;
    }
    if (lane == 63) wsum[wv] = incl;
    __syncthreads();
    int woff = 0, n_rec = 0;
#pragma unroll
    for (int v = 0; v < GT_WAVES; v++) { const int c = wsum[v]; woff += v < wv ? c : 0; n_rec += c; }
    int base = woff + incl - run;
#pragma unroll
    for (int b = 0; b < BPT; b++) { hist[b0 + b] = base; base += cntv[b]; }
    __syncthreads();                                  // bucket offsets complete
    // the grouped records overwrite the three arrays (every record is in registers since the second barrier); the
    // walk below takes whole groups of four records per lane group: the rest is padded with records of weight 0
    // for target -1
    const int per = ((n_rec + NSEG3 - 1) / NSEG3 + 3) & ~3;
#pragma unroll
    for (int t = 0; t < GT; t++) {
        if (rm[t] >= 0) {
            const int dst = hist[rm[t] & (GT_BUCKETS - 1)] + rp[t];
            st[dst] = ro[t]; sw[dst] = rw[t]; sz[dst] = (((tw0 + t) * PW) << 8) | lane;
        }
    }
    for (int j = n_rec + (int)threadIdx.x; j < NSEG3 * per; j += GT_WAVES * 64) { st[j] = -1; sw[j] = 0.f; sz[j] = 0; }
    __syncthreads();

    // ---- 3. one row update per run of equal targets; lane = feature, QPW records per instruction, the grouped
    //      records split evenly over the block's lane groups; the next four records are requested before the
    //      current four are used ----
    const int j_beg = (wv * QPW + sub) * per;
    const unsigned n_l = pl < P ? (unsigned)n : 0u;            // lanes without a feature never pass the bound check
    const unsigned ldgf4 = 4u * (unsigned)ldgf;
    char *const gbase = (char *)gfeat + 4 * pl;
    int cur = -1;
    float acc = 0.f;
    auto flush = [&]() {
        if ((unsigned)cur < n_l) atomicAdd((float *)(gbase + __umul24((unsigned)cur, ldgf4)), acc);
    };
    auto load4 = [&](int j, int4 &t4, int4 &z4, float4 &w4) {
        t4 = *(const int4 *)&st[j]; z4 = *(const int4 *)&sz[j]; w4 = *(const float4 *)&sw[j];
    };
    auto use4 = [&](const int4 &t4, const int4 &z4, const float4 &w4) {
        const int tg[4] = {t4.x, t4.y, t4.z, t4.w}, zz[4] = {z4.x, z4.y, z4.z, z4.w};
        const float ww[4] = {w4.x, w4.y, w4.z, w4.w};
        float2 cgv[4];
        int amv[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int ri = (zz[u] >> 8) + pl;            // the record names its row as row * PW
            cgv[u] = rows_cg[ri];
            amv[u] = rows_am[ri];
        }
#pragma unroll
        for (int u = 0; u < 4; u++) {
            if (tg[u] != cur) {
                flush();
                cur = tg[u];
                acc = 0.f;
            }
            acc += ww[u] * (amv[u] == (zz[u] & 255) ? cgv[u].y : cgv[u].x);
        }
    };
    int4 ta, za, tb4, zb;
    float4 wa, wb;
    load4(j_beg, ta, za, wa);                       // per = 0: reads inside the arrays, uses nothing
    int i = 0;
    for (; i + 8 <= per; i += 8) {                  // two groups of four per pass: no register copies
        load4(j_beg + i + 4, tb4, zb, wb);
        use4(ta, za, wa);
        if (i + 8 < per) load4(j_beg + i + 8, ta, za, wa);
        use4(tb4, zb, wb);
    }
    if (i < per) use4(ta, za, wa);
    flush();
    if (bad && status) atomicOr(&status[0], FGC_ST_BAD_INDEX);
}

static size_t gravnet_tile_lds(int pw, int K)
{
    const size_t rows = (size_t)GT_WAVES * GT, nseg3 = (size_t)GT_WAVES * (64 / pw);
    return rows * pw * 9 + (size_t)GT_BUCKETS * 4 + 16 * ((GT_WAVES + 3) / 4) + 12 * (rows * ((K + 7) & ~7) + 4 * nseg3);
}

static int pick_pw(int P)
{
    int pw = 64;
    while (pw > 8 && (pw >> 1) >= P) pw >>= 1;
    return pw;
}

extern "C" int fgc_gravnet_aggregate_fwd_f32(const int64_t *d_idx, const float *d_distsq, const float *d_feat,
                                             float *d_fmean, float *d_fmax, int32_t *d_argmax, int64_t n_vert,
                                             int32_t K, int32_t P, void *stream)
{
    return fgc_gravnet_aggregate_fwd_ld_f32(d_idx, d_distsq, d_feat, P, n_vert, d_fmean, d_fmax, P, d_argmax, n_vert, K,
                                            P, nullptr, stream);
}

extern "C" int fgc_gravnet_aggregate_fwd_ld_f32(const int64_t *d_idx, const float *d_distsq, const float *d_feat,
                                                int32_t ld_feat, int64_t n_feat_rows, float *d_fmean,
                                                float *d_fmax, int32_t ld_out, int32_t *d_argmax, int64_t n_vert,
                                                int32_t K, int32_t P, int32_t *d_status, void *stream)
{
    if (n_vert < 0 || K < 1 || P < 1 || ld_feat < P || ld_out < P || n_feat_rows < 0) return FGC_EINVAL;
    if (n_vert == 0) return FGC_OK;
    hipStream_t s = (hipStream_t)stream;
    const int pw = pick_pw(P);
    const unsigned blocks = (unsigned)fgc_cdiv(fgc_cdiv(n_vert, 64 / pw), 4);
#define FGC_L(PWW)                                                                                    \
    hipLaunchKernelGGL((k_gravnet_fwd<PWW>), dim3(blocks), dim3(256), 0, s, d_idx, d_distsq, d_feat, \
                       (int)ld_feat, n_feat_rows, d_fmean, d_fmax, (int)ld_out, d_argmax, n_vert, (int)K, (int)P, \
                       d_status)
    switch (pw) {
    case 8: FGC_L(8); break;
    case 16: FGC_L(16); break;
    case 32: FGC_L(32); break;
    default: FGC_L(64); break;
    }
#undef FGC_L
    FGC_LAUNCH_CHECK();
    return FGC_OK;
}

extern "C" int fgc_gravnet_aggregate_bwd_f32(const int64_t *d_idx, const float *d_distsq, const float *d_feat,
                                             const int32_t *d_argmax, const float *d_grad_fmean,
                                             const float *d_grad_fmax, float *d_grad_feat, float *d_grad_distsq,
                                             int64_t n_vert, int32_t K, int32_t P, void *stream)
{
    return fgc_gravnet_aggregate_bwd_ld_f32(d_idx, d_distsq, d_feat, P, n_vert, d_argmax, d_grad_fmean, d_grad_fmax, P,
                                            d_grad_feat, P, d_grad_distsq, n_vert, K, P, nullptr, stream);
}

extern "C" int fgc_gravnet_aggregate_bwd_ld_f32(const int64_t *d_idx, const float *d_distsq, const float *d_feat,
                                                int32_t ld_feat, int64_t n_feat_rows, const int32_t *d_argmax,
                                                const float *d_grad_fmean, const float *d_grad_fmax,
                                                int32_t ld_grad, float *d_grad_feat, int32_t ld_grad_feat,
                                                float *d_grad_distsq, int64_t n_vert, int32_t K, int32_t P,
                                                int32_t *d_status, void *stream)
{
    if (n_vert < 0 || K < 1 || P < 1 || ld_feat < P || ld_grad < P || ld_grad_feat < P || n_feat_rows < 0)
        return FGC_EINVAL;
    if (n_vert == 0) return FGC_OK;
    hipStream_t s = (hipStream_t)stream;
    const int pw = pick_pw(P);
    const unsigned blocks = (unsigned)fgc_cdiv(fgc_cdiv(n_vert, 64 / pw), 4);
#define FGC_L(PWW)                                                                                         \
    hipLaunchKernelGGL((k_gravnet_bwd<PWW>), dim3(blocks), dim3(256), 0, s, d_idx, d_distsq, d_feat,      \
                       (int)ld_feat, n_feat_rows, d_argmax, d_grad_fmean, d_grad_fmax, (int)ld_grad, d_grad_feat, \
                       (int)ld_grad_feat, d_grad_distsq, n_vert, (int)K, (int)P, d_status)
    switch (pw) {
    case 8: FGC_L(8); break;
    case 16: FGC_L(16); break;
    case 32: FGC_L(32); break;
    default: FGC_L(64); break;
    }
#undef FGC_L
    FGC_LAUNCH_CHECK();
    return FGC_OK;
}

extern "C" int fgc_gravnet_aggregate_bwd_sorted_supported(int64_t n_vert, int32_t K, int32_t P, int32_t ld_feat,
                                                          int32_t ld_grad_feat)
{
    if (K > 64 || P > 64 || P <= 8) return 0;
    // 32-bit byte offsets of the feature and gradient rows, formed with a 24-bit multiply
    if (n_vert >= (1 << 24) || ld_feat >= (1 << 22) || (uint64_t)n_vert * (uint64_t)ld_feat * 4ull >= 0xffffffffull ||
        ld_grad_feat >= (1 << 22) || (uint64_t)n_vert * (uint64_t)ld_grad_feat * 4ull >= 0xffffffffull)
        return 0;
    return 1;
}

extern "C" int fgc_gravnet_aggregate_bwd_sorted_f32(const int32_t *d_nbr_sorted, const int32_t *d_order,
                                                    const float *d_distsq, const float *d_feat, int32_t ld_feat,
                                                    const int32_t *d_argmax, const float *d_grad_fmean,
                                                    const float *d_grad_fmax, int32_t ld_grad, float *d_grad_feat,
                                                    int32_t ld_grad_feat, float *d_grad_distsq, int64_t n_vert,
                                                    int32_t K, int32_t P, int32_t *d_status, void *stream)
{
    if (n_vert < 0 || K < 1 || P < 1 || ld_feat < P || ld_grad < P || ld_grad_feat < P) return FGC_EINVAL;
    if (!fgc_gravnet_aggregate_bwd_sorted_supported(n_vert, K, P, ld_feat, ld_grad_feat)) return FGC_ESHAPE;
    if (n_vert == 0) return FGC_OK;
    if (!d_nbr_sorted || !d_order || !d_distsq || !d_feat || !d_argmax || !d_grad_fmean || !d_grad_fmax ||
        !d_grad_feat || !d_grad_distsq)
        return FGC_EINVAL;
    hipStream_t s = (hipStream_t)stream;
    const int pw = pick_pw(P);
    const unsigned blocks = (unsigned)fgc_cdiv(n_vert, GT_WAVES * GT);
    const size_t lds = gravnet_tile_lds(pw, K);          // at most 47 KB (P = K = 64)
#define FGC_L(PWW)                                                                                              \
    hipLaunchKernelGGL((k_gravnet_bwd_tile<PWW>), dim3(blocks), dim3(GT_WAVES * 64), lds, s, d_nbr_sorted,      \
                       (const uint32_t *)d_order, d_distsq, d_feat, (int)ld_feat, d_argmax, d_grad_fmean,      \
                       d_grad_fmax, (int)ld_grad, d_grad_feat, (int)ld_grad_feat, d_grad_distsq, n_vert, (int)K, \
                       (int)P, d_status)
    switch (pw) {
    case 16: FGC_L(16); break;
    case 32: FGC_L(32); break;
    default: FGC_L(64); break;
    }
#undef FGC_L
    FGC_LAUNCH_CHECK();
    return FGC_OK;
}
