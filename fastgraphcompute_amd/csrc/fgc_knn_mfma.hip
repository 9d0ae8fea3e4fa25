// Exact k-nearest-neighbour search for points with 5 to 8 coordinates: the candidates are screened on the matrix
// cores, the neighbours are chosen from exact distances (gfx950, wave64).
//
// Why a second search kernel.  With many coordinates the ball that holds a query's K neighbours reaches across most
// of its event, bounding boxes reject next to nothing and the search is brute force in effect; the per-pair
// subtract / multiply / add chain of k_knn then takes 4 D + 1 vector instructions per 64 pairs.  Here one
// v_mfma_f32_32x32x2f32 step handles 32 queries x 32 candidates x 2 coordinates, and the vector unit only sees the
// few pairs that can still matter.
//
// Work decomposition: one wavefront (= one block) owns 32 consecutive points of the sorted order as queries.  Lane l
// stands for query l % 32 in the matrix products (queries are the columns); the two halves of the wavefront
// (h = l / 32) hold one half of the coordinates each.  Per tile of 32 candidates (the rows) the accumulators receive
//     s = |c'|^2 (1 - m) - 2 q'.c' + |q'|^2 (1 - m),      q' = q - o,  c' = c - o,
// with o the wavefront's first query (centring keeps the cancellation error proportional to the squared distances
// inside the neighbourhood instead of the squared coordinates) and m a little more than the rounding errors, so that
// s is a lower bound of the pair's squared distance.  The first step (A below) runs in float32
// (v_mfma_f32_32x32x2f32, m = 2^-18); everything after it in float16 with float32 accumulation: one
// v_mfma_f32_32x32x16_f16 per tile, a sixteenth of the matrix-core time.  There the coordinates are scaled by a power
// of two sigma chosen so that every candidate that can matter has |c'| sigma < 245, converted with round-to-nearest
// (relative error 2^-11 per operand, so at most 2^-10 (|q'|^2 + |c'|^2) on -2 q'.c'), the norms enter as (high, low)
// pairs of float16, and m = 1.03 * 2^-10: s is at most 2^-9 * 1.03 (|q'|^2 + |c'|^2) below the squared distance.  A
// candidate too far away for the scale (|c'|^2 sigma^2 >= 60000) counts as infinitely far, which it is for this purpose.
//
// Selection without candidate pools in the inner loops.  The K-th smallest s of a query is found with histograms in
// LDS (one column of buckets per query, plain LDS integer adds):
//   A  the largest s among the first K or more candidates around the wavefront's own position bounds the K-th
//      smallest s: the range of the first histogram;
//   (the histogram scale is a power of two, so that it can be folded into the float16 operands exactly)
//   B  histogram of s over the seed chunks (the chunks of 64 points around the own position: spatial neighbours
//      thanks to the Hilbert order); the bucket where the running count reaches K gives a tighter bound E1;
//   C  histogram over the whole event with range E1; its cut E2 is within one bucket of the K-th smallest s;
//   D  every candidate with s below E2, widened by the screening error, is collected as a candidate number
//      (K plus a handful); there are at least K of them and every true neighbour is among them;
//   E  per query, one candidate per lane: exact squared distance in the reference's operation order, unfused, from
//      the coordinates in memory (binned_select_knn_cpu.cpp:10-19) - distsq is bit-identical to the vector search -
//      then the exact K-th value by bisection on ballot counts, and the row.
// Passes C and D skip aligned groups of 64 chunks whose bounding box no query's ball reaches, and chunks whose box
// the box of all 32 queries, widened by the largest bound, does not reach; both tests use the distance's own
// operations in the same order on interval ends, so they cannot reject a candidate the exact test would accept.  The
// bin grid is not used beyond the event boundaries.
//
// A query whose collected candidates do not fit its column (more near-ties at the K-th distance than the column has
// room for, or a wavefront whose queries lie so far apart that the screening error swamps the bound) is not written
// here: its flag in a.redo is set and the vector search, launched behind this kernel, handles the flagged queries.
#include "fgc_common.h"
#include "fgc_internal.h"
#include "fgc_knn_sort.h"
#include <type_traits>

typedef float fgc_f32x16 __attribute__((ext_vector_type(16)));
typedef _Float16 fgc_h8 __attribute__((ext_vector_type(8)));
typedef _Float16 fgc_h2 __attribute__((ext_vector_type(2)));
typedef float fgc_f2 __attribute__((ext_vector_type(2)));

#define MF_QT 32            // queries per wavefront
#ifndef MF_SEED_K
#define MF_SEED_K 40        // one seed chunk on either side of the own chunk per this many neighbours asked for
#endif

__device__ __forceinline__ float mf_wave_min_f(float v)
{
    v = fminf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xf, 0xf, true)));
    v = fminf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xf, 0xf, true)));
    v = fminf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xf, 0xf, true)));
    v = fminf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xf, 0xf, true)));
    return fminf(fminf(fgc_readlane_f(v, 0), fgc_readlane_f(v, 16)), fminf(fgc_readlane_f(v, 32), fgc_readlane_f(v, 48)));
}
__device__ __forceinline__ float mf_wave_max_f(float v) { return -mf_wave_min_f(-v); }

// value of the partner lane (lane ^ 32)
__device__ __forceinline__ int mf_other_half(int v) { return fgc_xor_lane<32>(v); }


using MfMax = std::integral_constant<int, 0>;
using MfHist = std::integral_constant<int, 1>;
using MfCollect = std::integral_constant<int, 2>;

constexpr float MF_SHRINK16 = 1.0f - 0x1.08p-10f;    // 1 - 1.03 * 2^-10

// Float16 operands of the candidates (see fgc_internal.h): one block per group of chunks, one wavefront per chunk,
// lane = point.
__global__ __launch_bounds__(64 * FGC_MF_GROUP_CHUNKS) void k_mf_operands(
    const float4 *__restrict__ sp4, const float *__restrict__ box_lo, const float *__restrict__ box_hi, int n, int D, int DH,
    int ldc, int n_chunks, float *__restrict__ grp, uint4 *__restrict__ spa, unsigned *__restrict__ mfstat)
{
    __shared__ unsigned s_wide, s_chunks;
    const int lane = fgc_lane();
    const int g = blockIdx.x;
    const int c = g * FGC_MF_GROUP_CHUNKS + (int)(threadIdx.x >> 6);
    if (threadIdx.x == 0) { s_wide = 0u; s_chunks = 0u; }
    __syncthreads();
    // bounding box of the group, coordinate d in lane d
    float lo = INFINITY, hi = -INFINITY;
    if (lane < D) {
        float l[FGC_MF_GROUP_CHUNKS], h[FGC_MF_GROUP_CHUNKS];
#pragma unroll
        for (int k = 0; k < FGC_MF_GROUP_CHUNKS; k++) {
            const int cc = g * FGC_MF_GROUP_CHUNKS + k;
            l[k] = cc < n_chunks ? box_lo[(size_t)lane * n_chunks + cc] : INFINITY;
            h[k] = cc < n_chunks ? box_hi[(size_t)lane * n_chunks + cc] : -INFINITY;
        }
#pragma unroll
        for (int k = 0; k < FGC_MF_GROUP_CHUNKS; k++) { lo = fminf(lo, l[k]); hi = fmaxf(hi, h[k]); }
    }
    // How wide is the group against its own chunks?  Where a group of 1024 points spans several clusters while its
    // chunks of 64 sit inside one, the float16 screening error (proportional to the group's squared radius) exceeds
    // the neighbour distances and the matrix-core search could only hand its queries on: counted here (one pair of
    // adds per group), decided there.
    if (c < n_chunks) {
        const float clo = lane < D ? box_lo[(size_t)lane * n_chunks + c] : 0.f;
        const float chi = lane < D ? box_hi[(size_t)lane * n_chunks + c] : 0.f;
        const float ch = (lane < D && fabsf(clo) < INFINITY && fabsf(chi) < INFINITY && chi >= clo) ? 0.5f * chi - 0.5f * clo : 0.f;
        const float gh = (lane < D && fabsf(lo) < INFINITY && fabsf(hi) < INFINITY && hi >= lo) ? 0.5f * hi - 0.5f * lo : 0.f;
        const float rc2 = fgc_wave_sum(ch * ch), rg2 = fgc_wave_sum(gh * gh);
        if (lane == 0 && c * 64 < n) {
            atomicAdd(&s_chunks, 1u);
            if (rg2 > 24.f * rc2) atomicAdd(&s_wide, 1u);
        }
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        if (s_chunks) atomicAdd(&mfstat[0], s_chunks);
        if (s_wide) atomicAdd(&mfstat[1], s_wide);
    }
    if (c >= n_chunks) return;
    float ctr = 0.5f * lo + 0.5f * hi, half = 0.5f * hi - 0.5f * lo;
    if (lane >= D) { ctr = 0.f; half = 0.f; }
    else if (!(fabsf(lo) < INFINITY && fabsf(hi) < INFINITY)) { ctr = 0.f; half = lo > hi ? 0.f : INFINITY; }   // lo > hi: no finite point
    const float R2 = fgc_wave_sum(half * half) * (1.0f + 0x1p-20f);
    // sigma: the power of two with 75 < R sigma <= 150
    float sigma;
    if (!(R2 < INFINITY)) sigma = 0x1p-40f;
    else if (!(R2 > 0.f)) sigma = 0x1p40f;
    else {
        const float want = 150.f / sqrtf(R2);
        sigma = __uint_as_float(min(max(__float_as_uint(want) & 0xff800000u, 0x20000000u), 0x5f000000u));
    }
    // the centre in the layout of sp: float f of a row is coordinate f (f < 4) or DH + f - 4
    float cf[8];
#pragma unroll
    for (int f = 0; f < 8; f++) {
        const int d = f < 4 ? f : DH + f - 4;
        const bool used = (f < 4 ? f < DH : true) && d < D;
        cf[f] = used ? fgc_readlane_f(ctr, d < 63 ? d : 63) : 0.f;
    }
    if (lane == 0 && c % FGC_MF_GROUP_CHUNKS == 0) {
        float *rec = grp + (size_t)g * FGC_MF_GRP_FLOATS;
#pragma unroll
        for (int f = 0; f < 8; f++) rec[f] = cf[f];
        rec[8] = sigma; rec[9] = R2;
#pragma unroll
        for (int f = 10; f < FGC_MF_GRP_FLOATS; f++) rec[f] = 0.f;
    }
    const int i = c * 64 + lane;
    const float4 x0 = sp4[(size_t)i * 2], x1 = sp4[(size_t)i * 2 + 1];
    const float x[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
    float r[8], rn = 0.f;
#pragma unroll
    for (int f = 0; f < 8; f++) {
        r[f] = __builtin_fmaf(x[f], sigma, -cf[f] * sigma);
        rn = __builtin_fmaf(r[f], r[f], rn);
    }
    const bool ok = i < n && rn < 60000.f;
    const float rne = rn * MF_SHRINK16;
    const _Float16 nh = (_Float16)rne;
    const _Float16 nl = (_Float16)(rne - (float)nh);
    union { fgc_h8 h; uint4 u; } a0, a1;
    const _Float16 zero = (_Float16)0.f, one = (_Float16)1.f, inf = (_Float16)INFINITY;
    a0.h = fgc_h8{ok ? (_Float16)r[0] : zero, ok ? (_Float16)r[1] : zero, ok ? (_Float16)r[2] : zero,
                  ok ? (_Float16)r[3] : zero, ok ? nh : inf, ok ? nl : zero, one, one};
    a1.h = fgc_h8{ok ? (_Float16)r[4] : zero, ok ? (_Float16)r[5] : zero, ok ? (_Float16)r[6] : zero,
                  ok ? (_Float16)r[7] : zero, zero, zero, zero, zero};
    spa[(size_t)i * 2] = a0.u;
    spa[(size_t)i * 2 + 1] = a1.u;
}

int fgc_launch_mf_operands(const float *sp, const float *box_lo, const float *box_hi, int n, int D, int ldc, float *grp,
                           void *spa, unsigned *mfstat, hipStream_t s)
{
    // (mfstat[0..1] start at zero: cleared by the kernel that wrote the boxes, fgc_launch_prepare_tail)
    const int n_chunks = ldc / 64;
    hipLaunchKernelGGL(k_mf_operands, dim3((unsigned)fgc_cdiv(n_chunks, FGC_MF_GROUP_CHUNKS)), dim3(64 * FGC_MF_GROUP_CHUNKS),
                       0, s, (const float4 *)sp, box_lo, box_hi, n, D, fgc_knn_sp_half(D), ldc, n_chunks, grp, (uint4 *)spa,
                       mfstat);
    FGC_LAUNCH_CHECK();
    return FGC_OK;
}

// D: coordinates per point, padded to an even number (6 or 8; a padding coordinate is 0 for every point and adds an
// exact +0 to every distance).  NSEG: ceil(K / 64).  PS: ceil(column height / 64).
template <int D, int NSEG, int PS, bool STATS>
__global__ __launch_bounds__(64, 4) void k_knn_mf(KnnArgs a)
{
    constexpr int DH = D / 2;             // coordinates per half of the wavefront
    extern __shared__ unsigned s_mf[];
    const int CAP = a.pool_cap;           // column height: histogram buckets = collected candidates per query at most
    unsigned short *col = (unsigned short *)s_mf;   // [CAP][32] 16-bit entries: per query (column) histogram counts,
                                          // later the collected candidates as positions inside their event - which is why
                                          // this kernel takes events of at most 65535 points.  Half the bytes of 32-bit
                                          // entries: four wavefronts per SIMD instead of two
    uint2 *rowbuf = (uint2 *)(s_mf + 16 * CAP);   // [NSEG * 64] one query's selected (distance, position) pairs

    const int lane = fgc_lane();
    const int q = lane & 31, h = lane >> 5;
    const int qbeg = blockIdx.x * MF_QT;
    if (qbeg >= a.n) return;
    const int nq = min(MF_QT, a.n - qbeg);
    const bool isq = q < nq;
    const int qs = qbeg + (isq ? q : 0);
    // strongly clustered points (counted by the preparation stage): everything goes to the vector search
    if (a.mfstat[1] * 4u > a.mfstat[0]) {
        if (h == 0 && isq) a.redo[qs] = 1;
        return;
    }
    const int K = a.K;
    const int Dn = a.D;                   // coordinates the points really have (D or D - 1)
    const float4 *__restrict__ sp4 = (const float4 *)a.sp;   // [ldc][2]: coordinates h * DH .. h * DH + DH - 1 in half h
    const int *__restrict__ bb = a.bb;

    // the query's coordinates in the layout of sp (both halves: the exact distance needs all of them)
    float qx[8];
    {
        const float4 q0 = sp4[(size_t)qs * 2], q1 = sp4[(size_t)qs * 2 + 1];
        qx[0] = q0.x; qx[1] = q0.y; qx[2] = q0.z; qx[3] = q0.w;
        qx[4] = q1.x; qx[5] = q1.y; qx[6] = q1.z; qx[7] = q1.w;
    }
    // centre: the wavefront's first query (a non-finite coordinate there must not spoil the other queries)
    float o[DH];
    {
        const float4 oc = sp4[(size_t)qbeg * 2 + h];
        const float t[4] = {oc.x, oc.y, oc.z, oc.w};
#pragma unroll
        for (int j = 0; j < DH; j++) o[j] = (fabsf(t[j]) < INFINITY) ? t[j] : 0.f;
    }
    // float32 B operands of step A (queries = columns): -2 q' for the coordinate steps, (1, |q'|^2 (1 - m)) for the
    // norm step
    float tq[DH];             // q' of this lane's half
    float bq[DH + 1];
    float qn;                 // |q'|^2
    {
        const float4 qm = sp4[(size_t)qs * 2 + h];
        const float t4[4] = {qm.x, qm.y, qm.z, qm.w};
        float part = 0.f;
#pragma unroll
        for (int j = 0; j < DH; j++) {
            tq[j] = t4[j] - o[j];
            bq[j] = -2.f * tq[j];
            part += tq[j] * tq[j];
        }
        qn = fgc_halve_pair<32>(part, part, lane);
        bq[DH] = h ? qn * (1.0f - 0x1p-18f) : 1.0f;
    }

    // events: bins per event = product of the bins per binned dimension
    int bpe = 1;
    for (int i = 0; i < a.nbd; i++) bpe *= __float_as_int(a.geom[FGC_GEOM_NB + i]);
    const int ev = (int)(a.skeys[qs] >> a.key_shift) / bpe;
    bool qactive = isq;
    if (a.sdir && isq) { const unsigned char dd = a.sdir[qs]; qactive = !(dd == 0 || dd == 2); }

    // ---- per-lane state (both lanes of a query hold the same values, except n_own) ----
    bool ing = false;        // the query belongs to the event that is being scanned
    float bound = INFINITY;  // bound on the query's K-th smallest squared distance
    float mx = -INFINITY;    // step A: largest finite s seen
    int n_own = 0;           // collected candidates of this lane: lane (0, q) fills column q from the top, (1, q) from the bottom
    bool over = false;       // the query is left to the vector search (column full, or out of the float16 range)
    const float NBm1 = (float)(CAP - 1);
    // float16 screening: the candidates' operands are relative to the centre of their group of 8 chunks, the query's
    // operand is recomputed whenever the scan enters another group
    const uint4 *__restrict__ spa4 = (const uint4 *)a.spa;
    float qh4[4];            // the query's coordinates of this lane's half
    {
        const float4 qm = sp4[(size_t)qs * 2 + h];
        qh4[0] = qm.x; qh4[1] = qm.y; qh4[2] = qm.z; qh4[3] = qm.w;
    }
    int cur_g = -1;          // group the B operand stands for
    int pg_id = -1;          // group whose record sits in pg_c / pg_s
    float4 pg_c = make_float4(0.f, 0.f, 0.f, 0.f);
    float2 pg_s = make_float2(1.f, 0.f);
    const int n_groups = (a.n_chunks + FGC_MF_GROUP_CHUNKS - 1) / FGC_MF_GROUP_CHUNKS;
    float hsc = 0.f;         // histogram pass: bucket = trunc(s * hsc), hsc a power of two (0: the query takes no part)
    float thr = -INFINITY;   // collect pass: candidates with accumulator below this are taken (units: sigma_g^2)
    int ev_base = 0;         // first sorted position of the query's event: collected candidates are stored relative to it
    bool collecting = false; // collect pass (accumulators in units of sigma_g^2) or histogram pass (units of 1 / hsc)
    fgc_h8 bh = {0, 0, 0, 0, 0, 0, 0, 0};   // B operand: (-2 q_g sigma S) x 4, then for h = 0: S, S, |q_g|^2 sigma^2 S (1 - m) as (high, low)

    unsigned long long nev = 0;
    unsigned nchunks = 0, n_range = 0, n_over = 0, n_coll = 0;

    // candidate jt + q of the event [ev_j0, ev_j1) usable?
    auto usable = [&](int jc, int ev_j0, int ev_j1) -> bool {
        bool valid = jc >= ev_j0 && jc < ev_j1;
        if (a.sdir && valid) { const unsigned char dd = a.sdir[jc]; if (dd == 1 || dd == 2) valid = false; }
        return valid;
    };

    // The float16 screening value s of a pair is at most 2^-9 * 1.02 (|q_g|^2 + |r|^2) below its squared distance
    // d^2 (q_g, r: query and candidate relative to the centre of the candidate's group); with |q_g| <= d + |r| and
    // |r|^2 <= R_g^2 that gives d^2 <= (s + 3 * 2^-9 * 1.02 R_g^2) / (1 - 2^-8 * 1.02).

    // ---- one tile in float32 (step A): the accumulators hold s ----
    auto tile_f32 = [&](int jt, const float4 cc, int ev_j0, int ev_j1, int &nok) -> fgc_f32x16 {
        const bool valid = usable(jt + q, ev_j0, ev_j1);
        const float ct[4] = {cc.x, cc.y, cc.z, cc.w};
        float ac[DH + 1];
        float part = 0.f;
#pragma unroll
        for (int j = 0; j < DH; j++) { ac[j] = ct[j] - o[j]; part += ac[j] * ac[j]; }
        const float cn = fgc_halve_pair<32>(part, part, lane);
        const bool ok = valid && cn < INFINITY;      // a candidate with a non-finite coordinate is nobody's neighbour
#pragma unroll
        for (int j = 0; j < DH; j++) ac[j] = ok ? ac[j] : 0.f;
        ac[DH] = h ? 1.0f : (ok ? cn * (1.0f - 0x1p-18f) : INFINITY);
        fgc_f32x16 acc = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j <= DH; j++) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(ac[j], bq[j], acc, 0, 0, 0);
        nok = __popcll(fgc_ballot(ok && h == 0));
        if (STATS) nev += (unsigned long long)nok * (unsigned)__popcll(fgc_ballot(ing && h == 0));
        return acc;
    };
    // ---- one tile in float16: the accumulators hold s sigma_g^2 S.  `inside`: every candidate of the tile belongs
    //      to the event and no direction flags are in use (nothing to mask) ----
    auto tile_f16 = [&](int jt, uint4 av, bool inside, int ev_j0, int ev_j1) -> fgc_f32x16 {
        if (!inside) {
            // an unusable candidate gets an infinite norm (element 4 of the first half)
            if (!usable(jt + q, ev_j0, ev_j1) && h == 0) av.z = 0x00007c00u;
        }
        union { uint4 u; fgc_h8 v; } cv;
        cv.u = av;
        fgc_f32x16 acc = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(cv.v, bh, acc, 0, 0, 0);
        if (STATS) nev += 32ull * (unsigned)__popcll(fgc_ballot(ing && h == 0));
        return acc;
    };
    // B operand of the float16 tiles for group g.  S is chosen so that the accumulators come out in the units of the
    // pass: sigma_g^2 S = hsc in a histogram pass, S = 1 in the collect pass (thr follows sigma_g).  A query whose
    // operands leave the float16 range gets an infinite accumulator if the group is farther away than its bound,
    // and is given up otherwise.
    auto set_group = [&](int g) {
        cur_g = g;
        // the record of the group: from the registers filled ahead of time when the scan moved on as expected
        if (g != pg_id) {
            const float *rec = a.grp + (size_t)g * FGC_MF_GRP_FLOATS;
            pg_c = *(const float4 *)(rec + 4 * h);
            pg_s = *(const float2 *)(rec + 8);
        }
        const float4 gc = pg_c;
        const float sg = pg_s.x, R2 = pg_s.y;
        {
            // ask for the next group's record now
            pg_id = min(g + 1, n_groups - 1);
            const float *rec = a.grp + (size_t)pg_id * FGC_MF_GRP_FLOATS;
            pg_c = *(const float4 *)(rec + 4 * h);
            pg_s = *(const float2 *)(rec + 8);
        }
        const float gcf[4] = {gc.x, gc.y, gc.z, gc.w};
        float qg[4] = {0.f, 0.f, 0.f, 0.f};
        float part = 0.f;
#pragma unroll
        for (int j = 0; j < DH; j++) {
            qg[j] = qh4[j] - gcf[j];
            part = __builtin_fmaf(qg[j], qg[j], part);
        }
        const float qgn = fgc_halve_pair<32>(part, part, lane);
        const float S = collecting ? 1.f : hsc / (sg * sg);          // powers of two (0 for a query that takes no part)
        const float f = -2.f * sg * S;
        float t[4];
#pragma unroll
        for (int j = 0; j < 4; j++) t[j] = qg[j] * f;
        // histogram pass: the group's share of the screening error goes on top, so that the histogram counts upper
        // bounds of the squared distances, s + 3 * 2^-9 * 1.02 R_g^2 (times 1 / (1 - 2^-8 * 1.02), applied at the cut):
        // a wide group far away only blurs its own candidates
        const float qs2 = (qgn * MF_SHRINK16 + (collecting ? 0.f : R2 * 0x1p-7f)) * (sg * sg) * S;
        const bool part_of = ing && !over && (collecting || hsc > 0.f);
        bool fits = S < 30000.f && qs2 < 60000.f && fabsf(t[0]) < 60000.f && fabsf(t[1]) < 60000.f &&
                    fabsf(t[2]) < 60000.f && fabsf(t[3]) < 60000.f;
        fits = fits && (fgc_ballot(fits) >> (lane ^ 32) & 1ull);    // both lanes of the query
        // the whole group beyond the query's bound?  (|q_g| - R_g)^2 > bound
        const float gapr = __builtin_amdgcn_sqrtf(qgn) * (1.0f - 0x1p-20f) - __builtin_amdgcn_sqrtf(R2) * (1.0f + 0x1p-20f);
        const bool beyond = gapr > 0.f && gapr * gapr > bound * (1.0f + 0x1p-10f);
        if (part_of && !fits && !beyond) { over = true; if (STATS) n_range++; }
        const bool on = part_of && fits && !over;
        const bool far = part_of && !fits && beyond;
        const _Float16 zero = (_Float16)0.f, inf = (_Float16)INFINITY;
        const _Float16 Sh = on ? (_Float16)S : (far ? (_Float16)1.f : zero);
        const _Float16 qh = on ? (_Float16)qs2 : (far ? inf : zero);
        const _Float16 ql = on ? (_Float16)(qs2 - (float)qh) : zero;
        bh[0] = on ? (_Float16)t[0] : zero; bh[1] = on ? (_Float16)t[1] : zero;
        bh[2] = on ? (_Float16)t[2] : zero; bh[3] = on ? (_Float16)t[3] : zero;
        bh[4] = h ? zero : Sh; bh[5] = h ? zero : Sh;
        bh[6] = h ? zero : qh; bh[7] = h ? zero : ql;
        if (collecting) thr = on ? bound * (sg * sg) * (1.0f + 0x1p-20f) : -INFINITY;
    };

    // accumulator v of lane (h, q): candidate row 8 (v / 4) + 4 h + v % 4, query q
    auto tile_post = [&](auto mode, int jt, const fgc_f32x16 acc) {
        if constexpr (decltype(mode)::value == 0) {
#pragma unroll
            for (int v = 0; v < 16; v++) mx = (acc[v] < INFINITY) ? fmaxf(mx, acc[v]) : mx;
        } else if constexpr (decltype(mode)::value == 1) {
            // two columns share a 32-bit word: the count of query q is its half (q & 1); no count passes 65535
            unsigned *mycol = s_mf + (q >> 1);
            const unsigned inc = (q & 1) ? 0x10000u : 1u;
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int b = (int)__builtin_amdgcn_fmed3f(acc[v], 0.f, NBm1);
                atomicAdd(mycol + (b << 4), inc);
            }
        } else {
            // the two lanes of a query share what is left of its column evenly for this tile; a candidate that
            // finds no room leaves the query to the vector search
            const int tot = n_own + mf_other_half(n_own);
            const int lim = n_own + ((CAP - tot) >> 1);
            const int jh = jt + 4 * h - ev_base;
#pragma unroll
            for (int v = 0; v < 16; v++) {
                if (acc[v] < thr) {
                    if (n_own < lim) {
                        col[((h ? CAP - 1 - n_own : n_own) << 5) + q] = (unsigned short)(jh + 8 * (v / 4) + (v % 4));
                        n_own++;
                    } else over = true;
                }
            }
        }
    };

    // both tiles of chunk c; the operands were requested by prefetch(c), those of chunk c_next (if >= 0) are
    // requested here, before the matrix products of this chunk are worked through
    float4 pre0, pre1;
    uint4 prh0, prh1;
    auto prefetch32 = [&](int c) {
        const int j = c << 6;
        pre0 = sp4[(size_t)(j + q) * 2 + h];
        pre1 = sp4[(size_t)(j + 32 + q) * 2 + h];
    };
    const unsigned lane_off = (unsigned)(q * 2 + h) * 16u;       // this lane's operand inside a tile of 32 x 32 bytes
    auto prefetch = [&](int c) {
        const char *base = (const char *)spa4 + (size_t)c * 2048;  // wave-uniform base + 32-bit lane offset
        prh0 = *(const uint4 *)(base + lane_off);
        prh1 = *(const uint4 *)(base + 1024 + lane_off);
    };
    auto chunk32 = [&](int c, int ev_j0, int ev_j1) -> int {
        const int j = c << 6;
        prefetch32(c);
        if (STATS) nchunks++;
        int nok0 = 0, nok1 = 0;
        const bool two = j + 32 < ev_j1;
        const fgc_f32x16 acc0 = tile_f32(j, pre0, ev_j0, ev_j1, nok0);
        tile_post(MfMax{}, j, acc0);
        if (two) {
            const fgc_f32x16 acc1 = tile_f32(j + 32, pre1, ev_j0, ev_j1, nok1);
            tile_post(MfMax{}, j + 32, acc1);
        }
        return nok0 + nok1;
    };
    auto chunk = [&](auto mode, int c, int c_next, int ev_j0, int ev_j1) {
        const int j = c << 6;
        const uint4 c0 = prh0, c1 = prh1;
        if (c_next >= 0) prefetch(c_next);
        if (STATS) nchunks++;
        if ((c / FGC_MF_GROUP_CHUNKS) != cur_g) set_group(c / FGC_MF_GROUP_CHUNKS);
        const bool inside = !a.sdir && j >= ev_j0 && j + 64 <= ev_j1;
        const bool two = j + 32 < ev_j1;
        const fgc_f32x16 acc0 = tile_f16(j, c0, inside, ev_j0, ev_j1);
        fgc_f32x16 acc1;
        if (two) acc1 = tile_f16(j + 32, c1, inside, ev_j0, ev_j1);
        tile_post(mode, j, acc0);
        if (two) tile_post(mode, j + 32, acc1);
    };
    // a chunk of an event that is collected whole: every usable candidate goes to every query of the event
    auto chunk_all = [&](int c, int ev_j0, int ev_j1) {
        for (int t = 0; t < 2; t++) {
            const int jt = (c << 6) + 32 * t;
            const unsigned um = (unsigned)fgc_ballot(h == 0 && usable(jt + q, ev_j0, ev_j1));
            const int tot = n_own + mf_other_half(n_own);
            const int lim = n_own + ((CAP - tot) >> 1);
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int r = 8 * (v / 4) + 4 * h + (v % 4);
                if (ing && ((um >> r) & 1u)) {
                    if (n_own < lim) {
                        col[((h ? CAP - 1 - n_own : n_own) << 5) + q] = (unsigned short)(jt + r - ev_base);
                        n_own++;
                    } else over = true;
                }
            }
        }
    };

    auto zero_columns = [&]() {
        for (int i = lane; i < 16 * CAP; i += 64) s_mf[i] = 0u;
    };

    // histogram scale: the largest power of two with bound * hsc <= CAP - 2, so that the range [0, bound) falls
    // on the buckets 0 .. CAP - 2 (the last bucket takes everything beyond)
    auto set_hist_scale = [&]() {
        hsc = 0.f;
        if (ing && bound < INFINITY && bound > 0.f && !over) {
            const float want = (NBm1 - 1.f) / bound;
            if (want < 0x1p100f && want > 0x1p-100f)
                hsc = __uint_as_float(__float_as_uint(want) & 0xff800000u);     // mantissa cleared: rounded down to 2^e
        }
        collecting = false;
        cur_g = -1;
    };
    // bucket where the running count of the query's histogram reaches K -> bound on the K-th smallest squared distance:
    // the upper edge of that bucket, widened by the screening error (unchanged when fewer than K candidates lie
    // inside the histogram's range)
    auto cut = [&]() {
        int cum = 0, bstar = CAP - 1;
        for (int b = 0; b < CAP - 1; b++) {
            cum += (int)col[(b << 5) + q];
            if (cum >= K && bstar == CAP - 1) bstar = b;
        }
        if (ing && bstar < CAP - 1 && hsc > 0.f && !over)
            bound = fminf(bound, (float)(bstar + 1) / hsc * (1.0f + 0x1.1p-8f) + 1e-30f);
    };

    // pass over the event's chunks outside [skip_lo, skip_hi] that the queries' balls of squared radius `reach`
    // (per lane) can touch, by aligned groups of 64 chunks, nearest group first
    auto scan_event = [&](auto mode, int ev_j0, int ev_j1, int skip_lo, int skip_hi, float reach, const float (&qlo)[D],
                          const float (&qhi)[D]) {
        const int c_lo = ev_j0 >> 6, c_hi = (ev_j1 - 1) >> 6;
        const int sb0 = qbeg >> 12, sb_lo = c_lo >> 6, sb_hi = c_hi >> 6;
        const int far = max(sb0 - sb_lo, sb_hi - sb0);
        const float rmax = mf_wave_max_f(ing ? reach : -INFINITY);
        for (int k = 0; k <= 2 * far; k++) {
            const int sb = sb0 + ((k & 1) ? (k + 1) / 2 : -(k / 2));
            if (sb < sb_lo || sb > sb_hi) continue;
            {
                // lane = query: does the query's ball reach the group's bounding box?
                float g2 = 0.f;
#pragma unroll
                for (int d = 0; d < D; d++) {
                    if (d < Dn) {      // the padding coordinate has no box
                        const int f = d < DH ? d : 4 + d - DH;
                        const float lo = a.sbox_lo[(size_t)d * a.n_super + sb], hi = a.sbox_hi[(size_t)d * a.n_super + sb];
                        const float g = fmaxf(fmaxf(lo - qx[f], qx[f] - hi), 0.f);
                        g2 = d == 0 ? g * g : g2 + g * g;
                    }
                }
                if (!fgc_ballot(ing && !(g2 > reach))) continue;
            }
            // lane = chunk: the chunk's box against the box of all queries of the group and the largest reach
            const int cb = sb << 6;
            const int c = cb + lane;
            const bool cv = c >= c_lo && c <= c_hi && (c < skip_lo || c > skip_hi);
            float g2 = 0.f;
#pragma unroll
            for (int d = 0; d < D; d++) {
                if (d < Dn) {
                    const float blo = cv ? a.box_lo[(size_t)d * a.n_chunks + c] : 0.f;
                    const float bhi = cv ? a.box_hi[(size_t)d * a.n_chunks + c] : 0.f;
                    const float g = fmaxf(fmaxf(blo - qhi[d], qlo[d] - bhi), 0.f);
                    g2 = d == 0 ? g * g : g2 + g * g;
                }
            }
            unsigned long long m = fgc_ballot(cv && !(g2 > rmax));
            if (m) prefetch(cb + __ffsll((long long)m) - 1);
            while (m) {
                const int l = __ffsll((long long)m) - 1;
                m &= m - 1;
                chunk(mode, cb + l, m ? cb + __ffsll((long long)m) - 1 : -1, ev_j0, ev_j1);
            }
        }
    };

    // ---- the events of the wavefront's queries, one after the other ----
    for (int pass = 0; pass < 2; pass++) {
        // pass 0: bounds (A, B, C) for every event; pass 1: collection (D).  The histograms and the collected
        // candidates share the columns, so all histograms are done before the first candidate is collected.
        unsigned long long todo = fgc_ballot(qactive);
        while (todo) {
            const int first = __ffsll((long long)todo) - 1;
            const int gev = fgc_readlane_i(ev, first);
            const unsigned long long gm = fgc_ballot(qactive && ev == gev);
            todo &= ~gm;
            ing = (gm >> lane) & 1ull;
            const int ev_j0 = bb[gev * bpe], ev_j1 = bb[(gev + 1) * bpe];
            if (ing) ev_base = ev_j0;
            if (ev_j1 - ev_j0 > 65535) {               // positions inside the event must fit 16 bits
                if (ing) over = true;
                continue;
            }
            const int c_lo = ev_j0 >> 6, c_hi = (ev_j1 - 1) >> 6;
            const int own = qbeg >> 6;
            const int seed_w = (K + MF_SEED_K - 1) / MF_SEED_K;
            const int s_lo = max(c_lo, own - seed_w), s_hi = min(c_hi, own + seed_w);
            if (pass == 0) {
                if (ev_j1 - ev_j0 <= CAP - 32) continue;    // a small event is collected whole: bound stays infinite
                // A: the largest s among the first K or more usable candidates, own chunk first, then alternately
                //    the chunks after and before it
                int seen = 0;
                const int far = max(own - c_lo, c_hi - own);
                for (int k = 0; k <= 2 * far && seen < K; k++) {
                    const int c = own + ((k & 1) ? (k + 1) / 2 : -(k / 2));
                    if (c < c_lo || c > c_hi) continue;
                    seen += chunk32(c, ev_j0, ev_j1);
                }
                mx = fmaxf(mx, __int_as_float(mf_other_half(__float_as_int(mx))));   // each lane saw half of the rows
                // fewer than K usable candidates in the whole event: everything is collected
                if (seen >= K && ing) bound = fminf(bound, fmaxf(mx, 0.f) * (1.0f + 0x1p-12f) + qn * 0x1p-14f + 1e-30f);
                mx = -INFINITY;
            }
            const bool bounded = fgc_ballot(ing && bound < INFINITY) != 0ull;   // the same for all queries of an event
            if (!bounded) {
                if (pass == 1) for (int c = c_lo; c <= c_hi; c++) chunk_all(c, ev_j0, ev_j1);
                continue;
            }
            // box of the group's queries (wave-uniform), original coordinate order
            float qlo[D], qhi[D];
#pragma unroll
            for (int d = 0; d < D; d++) {
                const int f = d < DH ? d : 4 + d - DH;
                qlo[d] = mf_wave_min_f(ing ? qx[f] : INFINITY);
                qhi[d] = mf_wave_max_f(ing ? qx[f] : -INFINITY);
            }
            if (pass == 0) {
                // B: histogram over the seed chunks
                set_hist_scale();
                if (fgc_ballot(hsc > 0.f)) {
                    zero_columns();
                    prefetch(s_lo);
                    for (int c = s_lo; c <= s_hi; c++) chunk(MfHist{}, c, c < s_hi ? c + 1 : -1, ev_j0, ev_j1);
                    cut();
                }
                // C: histogram over the event
                set_hist_scale();
                if (fgc_ballot(hsc > 0.f)) {
                    zero_columns();
                    prefetch(s_lo);
                    for (int c = s_lo; c <= s_hi; c++) chunk(MfHist{}, c, c < s_hi ? c + 1 : -1, ev_j0, ev_j1);
                    scan_event(MfHist{}, ev_j0, ev_j1, s_lo, s_hi, bound, qlo, qhi);
                    cut();
                }
                hsc = 0.f;
            } else {
                // D: collect everything whose screening value is below the bound
                collecting = true;
                cur_g = -1;
                prefetch(s_lo);
                for (int c = s_lo; c <= s_hi; c++) chunk(MfCollect{}, c, c < s_hi ? c + 1 : -1, ev_j0, ev_j1);
                scan_event(MfCollect{}, ev_j0, ev_j1, s_lo, s_hi, bound, qlo, qhi);
                thr = -INFINITY;
                collecting = false;
            }
        }
    }
    ing = false;

    // ---- E: per query, exact distances of the collected candidates, the K nearest, the row ----
    for (int qq = 0; qq < nq; qq++) {
        const int self = qbeg + qq;
        if (fgc_readlane_i((int)over, qq) | fgc_readlane_i((int)over, qq + 32)) {
            if (lane == 0) a.redo[self] = 1;
            if (STATS) n_over++;
            continue;
        }
        const long long orig_q = (long long)a.order[self];
        const int n0 = fgc_readlane_i(n_own, qq), n1 = fgc_readlane_i(n_own, qq + 32);
        const int c = n0 + n1;                    // <= CAP
        const int evb = fgc_readlane_i(ev_base, qq);
        if (STATS) n_coll += (unsigned)c;
        float qs_[8];
#pragma unroll
        for (int f = 0; f < 8; f++) qs_[f] = fgc_readlane_f(qx[f], qq);
        unsigned P[PS];
        int PI[PS];
        int nvalid = 0;
#pragma unroll
        for (int s = 0; s < PS; s++) {
            const int e = s * 64 + lane;
            const bool have = e < c;
            const int r = e < n0 ? e : CAP - 1 - (e - n0);
            const int id = have ? evb + (int)col[(r << 5) + qq] : self;
            const float4 c0 = sp4[(size_t)id * 2], c1 = sp4[(size_t)id * 2 + 1];
            const float cx[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w};
            float df = qs_[0] - cx[0];
            float dsq = df * df;
#pragma unroll
            for (int d = 1; d < D; d++) {
                const int f = d < DH ? d : 4 + d - DH;
                df = qs_[f] - cx[f];
                dsq += df * df;
            }
            const bool good = have && dsq < INFINITY;
            P[s] = good ? __float_as_uint(dsq) : 0xffffffffu;
            PI[s] = id;
            nvalid += __popcll(fgc_ballot(good));
        }
        // the K nearest: bisection on the bit patterns (monotone for non-negative floats) down to the K-th value,
        // ties at that value cut by position
        bool keep[PS];
#pragma unroll
        for (int s = 0; s < PS; s++) keep[s] = P[s] != 0xffffffffu;
        if (nvalid > K) {
            auto count_le = [&](unsigned t) -> int {
                int n = 0;
#pragma unroll
                for (int s = 0; s < PS; s++) n += __popcll(fgc_ballot(P[s] <= t));
                return n;
            };
            int mxb = 0;
#pragma unroll
            for (int s = 0; s < PS; s++) mxb = max(mxb, P[s] == 0xffffffffu ? 0 : (int)P[s]);
            float flo = 0.f, fhi = __int_as_float(fgc_wave_max_i(mxb));
            bool exact = false;
            for (int it = 0; it < 24; it++) {
                const float mid = 0.5f * (flo + fhi);
                const int cm = count_le(__float_as_uint(mid));
                if (cm >= K) { fhi = mid; if (cm == K) { exact = true; break; } }
                else flo = mid;
            }
            unsigned hi = __float_as_uint(fhi);
            if (exact) {
#pragma unroll
                for (int s = 0; s < PS; s++) keep[s] = P[s] <= hi;
            } else {
                unsigned lo = flo > 0.f ? __float_as_uint(flo) + 1u : 0u;
                while (lo < hi) {
                    const unsigned mid = lo + ((hi - lo) >> 1);
                    if (count_le(mid) >= K) hi = mid; else lo = mid + 1u;
                }
                int nless = 0;
#pragma unroll
                for (int s = 0; s < PS; s++) nless += __popcll(fgc_ballot(P[s] < hi));
                int need = K - nless, before = 0;
#pragma unroll
                for (int s = 0; s < PS; s++) {
                    const unsigned long long em = fgc_ballot(P[s] == hi);
                    keep[s] = (P[s] < hi) || (P[s] == hi && (before + fgc_mbcnt(em)) < need);
                    before += __popcll(em);
                }
            }
        }
        // the kept entries, compacted, one per lane and segment
        int cnt = 0;
#pragma unroll
        for (int s = 0; s < PS; s++) {
            const unsigned long long km = fgc_ballot(keep[s]);
            if (keep[s]) rowbuf[cnt + fgc_mbcnt(km)] = make_uint2(P[s], (unsigned)PI[s]);
            cnt += __popcll(km);
        }
        const int cc = cnt;                        // <= K
        if (a.any_order) {
            // rows in collection order: the query itself trades places with the entry in slot 0.  A row without the
            // query (direction flags, or more than K points at distance 0) takes the sorting path below.
            int es = -1;
            unsigned EX[NSEG], EY[NSEG];
#pragma unroll
            for (int s = 0; s < NSEG; s++) {
                const bool valid = (s * 64 + lane) < cc;
                const uint2 e = valid ? rowbuf[s * 64 + lane] : make_uint2(0x7f800000u, 0xffffffffu);
                EX[s] = e.x; EY[s] = e.y;
                const unsigned long long sm = fgc_ballot(valid && (int)e.y == self);
                if (sm) es = s * 64 + __ffsll((long long)sm) - 1;
            }
            if (es >= 0) {
#pragma unroll
                for (int s = 0; s < NSEG; s++) {
                    const int e = s * 64 + lane;
                    if (e < cc) {
                        const int slot = e == es ? 0 : (e == 0 ? es : e);
                        a.out_idx[orig_q * K + slot] = e == es ? orig_q : (long long)a.order[EY[s]];
                        a.out_dist[orig_q * K + slot] = e == es ? 0.f : __uint_as_float(EX[s]);
                        if (a.out_sorted) a.out_sorted[(long long)self * K + slot] = (int)EY[s];
                    } else if (e < K) {
                        a.out_idx[orig_q * K + e] = a.tf_compat ? orig_q : -1ll;
                        a.out_dist[orig_q * K + e] = 0.f;
                        if (a.out_sorted) a.out_sorted[(long long)self * K + e] = -1;
                    }
                }
                continue;
            }
        }
        float L[NSEG];
        int I[NSEG];
        bool has_self = false;
#pragma unroll
        for (int s = 0; s < NSEG; s++) {
            const bool valid = (s * 64 + lane) < cc;
            const uint2 e = valid ? rowbuf[s * 64 + lane] : make_uint2(0x7f800000u, 0xffffffffu);
            L[s] = __uint_as_float(e.x);
            I[s] = (int)e.y;
            const bool is_self = valid && I[s] == self;
            if (is_self) L[s] = -1.f;             // the query itself sorts first
            has_self = has_self || (fgc_ballot(is_self) != 0ull);
        }
        FgcBitonic<2, 1, NSEG>::run(L, I);        // the cc finite keys end up in elements 0 .. cc-1
        const int shift = has_self ? 0 : 1;       // without the query among the candidates its slot 0 is added here
        const int n_out = min(cc + shift, K);
#pragma unroll
        for (int s = 0; s < NSEG; s++) {
            const int rank = s * 64 + lane;
            const int slot = rank + shift;
            if (rank < cc && slot < K) {
                const bool is_self = I[s] == self;
                a.out_idx[orig_q * K + slot] = is_self ? orig_q : (long long)a.order[I[s]];
                a.out_dist[orig_q * K + slot] = is_self ? 0.f : L[s];
                if (a.out_sorted) a.out_sorted[(long long)self * K + slot] = I[s];
            }
            if (rank < K && rank >= n_out) {
                a.out_idx[orig_q * K + rank] = a.tf_compat ? orig_q : -1ll;
                a.out_dist[orig_q * K + rank] = 0.f;
                if (a.out_sorted) a.out_sorted[(long long)self * K + rank] = -1;
            }
            if (!has_self && rank == 0) {
                a.out_idx[orig_q * K] = orig_q;
                a.out_dist[orig_q * K] = 0.f;
                if (a.out_sorted) a.out_sorted[(long long)self * K] = self;
            }
        }
    }
    if (STATS && a.stats && lane == 0) {
        atomicAdd(&a.stats[0], nev);
        atomicAdd(&a.stats[1], (unsigned long long)nchunks);
        atomicAdd(&a.stats[3], (unsigned long long)n_over);          // queries left to the vector search
        atomicAdd(&a.stats[4], (unsigned long long)fgc_readlane_i((int)n_range, 0));
        atomicAdd(&a.stats[5], (unsigned long long)n_coll);          // candidates collected for the others
    }
}

bool fgc_knn_uses_mfma(int D, int K) { return D >= 5 && D <= 8 && K <= 256; }

// column height: histogram buckets, and room for the candidates of one query - K, the candidates that share the
// histogram bucket of the K-th and those inside the screening error (K = 100: 152 rows, 20 KB of LDS per wavefront,
// two wavefronts per SIMD)
static int mf_column_height(int K) { return max(64, (K + max(K >> 1, 32) + 7) & ~7); }

template <int D, int NSEG, int PS, bool STATS> static int launch_mf_t(const KnnArgs &a, hipStream_t s)
{
    const int blocks = (int)fgc_cdiv(a.n, MF_QT);
    const size_t lds = (size_t)32 * a.pool_cap * 2 + (size_t)NSEG * 64 * 8;
    if (lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute((const void *)k_knn_mf<D, NSEG, PS, STATS>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return (int)e;
    }
    hipLaunchKernelGGL((k_knn_mf<D, NSEG, PS, STATS>), dim3(blocks), dim3(64), lds, s, a);
    FGC_LAUNCH_CHECK();
    return FGC_OK;
}

template <int D, bool STATS> static int launch_mf_d(const KnnArgs &a, hipStream_t s)
{
    const int ps = (a.pool_cap + 63) / 64;
    if (a.K <= 64) {
        if (ps <= 1) return launch_mf_t<D, 1, 1, STATS>(a, s);
        return launch_mf_t<D, 1, 2, STATS>(a, s);
    }
    if (a.K <= 128) {
        if (ps <= 2) return launch_mf_t<D, 2, 2, STATS>(a, s);
        if (ps <= 3) return launch_mf_t<D, 2, 3, STATS>(a, s);
        return launch_mf_t<D, 2, 4, STATS>(a, s);
    }
    if (ps <= 4) return launch_mf_t<D, 4, 4, STATS>(a, s);
    if (ps <= 5) return launch_mf_t<D, 4, 5, STATS>(a, s);
    return launch_mf_t<D, 4, 6, STATS>(a, s);
}

template <bool STATS> static int launch_mf(const KnnArgs &a_in, hipStream_t s)
{
    KnnArgs a = a_in;
    if (a.n <= 0) return FGC_OK;
    if (!fgc_knn_uses_mfma(a.D, a.K) || !a.sp || !a.redo || a.K < 1) return FGC_EINVAL;
    a.pool_cap = mf_column_height(a.K);
    int rc = fgc_fill_u32(a.redo, 0u, (a.n + 3) / 4, s);
    if (rc) return rc;
    rc = a.D <= 6 ? launch_mf_d<6, STATS>(a, s) : launch_mf_d<8, STATS>(a, s);
    if (rc) return rc;
    // the queries this kernel left out (flags in a.redo), by the vector search
    return STATS ? fgc_launch_knn_stats(a, s) : fgc_launch_knn(a, s);
}

int fgc_launch_knn_mfma(const KnnArgs &a, hipStream_t s) { return launch_mf<false>(a, s); }
int fgc_launch_knn_mfma_stats(const KnnArgs &a, hipStream_t s) { return launch_mf<true>(a, s); }
