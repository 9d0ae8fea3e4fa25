// Exact k-nearest-neighbour search over bin-sorted points (gfx950, wave64).
//
// Work decomposition: one wavefront owns QT consecutive points of the
// bin-sorted order (spatially adjacent queries).  Candidates are streamed 64 at
// a time, one per lane, with coalesced loads from the structure-of-arrays
// coordinate copy; the wavefront then walks over its queries (query
// coordinates broadcast from the owning lane), so every loaded candidate is
// reused for all queries of the tile.  Each query's K best candidates are kept
// as a list sorted by distance, one slot per lane, in LDS; the current K-th
// distance (tau) of query q lives in lane q of a register.  A candidate chunk
// touches the list only when some lane beats tau, which is rare after warm-up,
// so the steady-state loop is subtract / multiply / add / compare.
//
// Search order per group of queries that share a bin row (all binned
// coordinates but the last): grow a Chebyshev cube of bins level by level until
// every query holds K candidates, then sweep exactly the bins that intersect
// the balls of radius sqrt(tau) around the queries.  Before each contiguous
// candidate range, the squared gap between every query and the range's bin box
// is compared with the query's tau, so queries skip ranges that cannot improve
// them.  The result is the exact kNN set of the reference's shell search
// (binned_select_knn_cuda_kernel.cu:101-248) with fewer distance evaluations.
#include "fgc_common.h"
#include "fgc_internal.h"

#define QT 16  // queries per wavefront

template <int NSEG> struct KnnCfg { static constexpr int WPB = (NSEG <= 2) ? 4 : 2; };

template <int DT, int NSEG>
__global__ __launch_bounds__(KnnCfg<NSEG>::WPB * 64) void k_knn(KnnArgs a)
{
    constexpr int KP = NSEG * 64;
    constexpr int WPB = KnnCfg<NSEG>::WPB;
    constexpr int DR = DT > 0 ? DT : 1;
    __shared__ float s_d[WPB][QT * KP];
    __shared__ int s_i[WPB][QT * KP];

    const int lane = fgc_lane();
    const int wv = threadIdx.x >> 6;
    const int qbeg = (blockIdx.x * WPB + wv) * QT;
    if (qbeg >= a.n) return;  // no block-wide barrier is used below
    const int nq = min(QT, a.n - qbeg);
    float *ld = s_d[wv];
    int *li = s_i[wv];
    for (int s = lane; s < QT * KP; s += 64) { ld[s] = INFINITY; li[s] = -1; }

    const int K = a.K, D = a.D, nbd = a.nbd, ldc = a.ldc;
    const float *__restrict__ sc = a.sc;
    const int *__restrict__ bb = a.bb;

    // ---- geometry (wave-uniform) ----
    float mn[FGC_MAX_BIN_DIMS];
    int nb[FGC_MAX_BIN_DIMS];
#pragma unroll
    for (int i = 0; i < FGC_MAX_BIN_DIMS; i++) {
        mn[i] = a.geom[FGC_GEOM_MIN + i];
        nb[i] = __float_as_int(a.geom[FGC_GEOM_NB + i]);
    }
    const float bw = a.geom[FGC_GEOM_BW];
    const float margin = 1e-4f * bw;
    int rnb[4];  // bins of the row dimensions (all binned dims but the last), padded with 1
#pragma unroll
    for (int i = 0; i < 4; i++) rnb[i] = (i < nbd - 1) ? nb[i] : 1;
    int nz = nb[0];
    float mnz = mn[0];
#pragma unroll
    for (int i = 1; i < FGC_MAX_BIN_DIMS; i++)
        if (i == nbd - 1) { nz = nb[i]; mnz = mn[i]; }
    const int rows_per_event = rnb[0] * rnb[1] * rnb[2] * rnb[3];

    // ---- per-lane query state (lane q < nq holds query qbeg + q) ----
    const bool isq = lane < nq;
    const int qs = qbeg + (isq ? lane : 0);
    float qx[DR];
    if (DT > 0) {
#pragma unroll
        for (int d = 0; d < DR; d++) qx[d] = sc[(size_t)d * ldc + qs];
    }
    float qb[4];  // normalised row-dimension coordinates
#pragma unroll
    for (int i = 0; i < 4; i++) qb[i] = (i < nbd - 1) ? sc[(size_t)i * ldc + qs] - mn[i] : 0.f;
    const float qzn = sc[(size_t)(nbd - 1) * ldc + qs] - mnz;
    const int key = (int)a.skeys[qs];
    const int row = key / nz;
    const int zq = key - row * nz;
    float tau = INFINITY;
    bool qactive = isq;
    if (a.sdir && isq) { unsigned char dd = a.sdir[qs]; qactive = !(dd == 0 || dd == 2); }

    unsigned long long nev = 0, nchunks = 0, nins = 0;

    // ---- insert the lanes of `pm` (distances dsq, sorted ids jbase + lane) into query q's list ----
    auto insert = [&](int q, unsigned long long pm, float dsq, int jbase) {
        float L[NSEG];
        int I[NSEG];
#pragma unroll
        for (int s = 0; s < NSEG; s++) { L[s] = ld[q * KP + s * 64 + lane]; I[s] = li[q * KP + s * 64 + lane]; }
        float t = fgc_readlane_f(tau, q);
        while (pm) {
            const int src = __ffsll((long long)pm) - 1;
            pm &= pm - 1;
            const float cd = fgc_readlane_f(dsq, src);
            if (!(cd < t)) continue;
            const int ci = jbase + src;
            int pos = 0;
#pragma unroll
            for (int s = 0; s < NSEG; s++) pos += __popcll(fgc_ballot(L[s] <= cd));
#pragma unroll
            for (int s = NSEG - 1; s >= 0; s--) {
                const int p = pos - s * 64;
                if (p >= 64) continue;
                float up = __shfl_up(L[s], 1, 64);
                int upi = __shfl_up(I[s], 1, 64);
                if (s > 0) {
                    const float cf = fgc_readlane_f(L[s - 1], 63);
                    const int cidx = fgc_readlane_i(I[s - 1], 63);
                    if (lane == 0) { up = cf; upi = cidx; }
                }
                if (p < 0 || lane > p) { L[s] = up; I[s] = upi; }
                else if (lane == p) { L[s] = cd; I[s] = ci; }
            }
            nins++;
#pragma unroll
            for (int s = 0; s < NSEG; s++)
                if (s == ((K - 1) >> 6)) t = fgc_readlane_f(L[s], (K - 1) & 63);
        }
#pragma unroll
        for (int s = 0; s < NSEG; s++) { ld[q * KP + s * 64 + lane] = L[s]; li[q * KP + s * 64 + lane] = I[s]; }
        tau = (lane == q) ? t : tau;
    };

    // ---- all candidates of bins [f0, f1] against the queries in `gm` whose gap2 does not exceed tau ----
    auto process_range = [&](int f0, int f1, float gap2, unsigned long long gm) {
        const int j0 = bb[f0], j1 = bb[f1 + 1];
        if (j0 >= j1) return;
        const unsigned long long act = gm & fgc_ballot(!(gap2 > tau));
        if (!act) return;
        const int nact = __popcll(act);
        for (int base = j0; base < j1; base += 64) {
            const int j = base + lane;
            const bool v = j < j1;
            float cx[DR];
            if (DT > 0) {
#pragma unroll
                for (int d = 0; d < DR; d++) cx[d] = v ? sc[(size_t)d * ldc + j] : 0.f;
                if (!v) cx[0] = INFINITY;
            }
            bool cand_ok = v;
            if (a.sdir && v) { unsigned char dd = a.sdir[j]; if (dd == 1 || dd == 2) cand_ok = false; }
            if (DT > 0 && !cand_ok) cx[0] = INFINITY;
            nev += (unsigned long long)nact * (unsigned)min(64, j1 - base);
            nchunks++;
            unsigned long long m = act;
            while (m) {
                const int q = __ffsll((long long)m) - 1;
                m &= m - 1;
                const float t = fgc_readlane_f(tau, q);
                float dsq;
                if (DT > 0) {
                    float df = fgc_readlane_f(qx[0], q) - cx[0];
                    dsq = df * df;
#pragma unroll
                    for (int d = 1; d < DR; d++) { df = fgc_readlane_f(qx[d], q) - cx[d]; dsq += df * df; }
                } else {
                    dsq = INFINITY;
                    if (cand_ok) {
                        float df = sc[qbeg + q] - sc[j];
                        dsq = df * df;
                        for (int d = 1; d < D; d++) {
                            df = sc[(size_t)d * ldc + qbeg + q] - sc[(size_t)d * ldc + j];
                            dsq += df * df;
                        }
                    }
                }
                const unsigned long long pm = fgc_ballot(dsq < t);
                if (pm) insert(q, pm, dsq, base);
            }
        }
    };

    // squared gap (with safety margin) of this lane's query to a bin interval [b0, b1] of extent nbn
    auto gap1 = [&](float x, int b0, int b1, int nbn) -> float {
        const float lo = (b0 <= 0) ? -INFINITY : ((float)b0 - 1e-3f) * bw;
        const float hi = (b1 >= nbn - 1) ? INFINITY : ((float)(b1 + 1) - 1e-3f) * bw;
        float g = fmaxf(fmaxf(lo - x, x - hi) - margin, 0.f);
        return g * g;
    };

    // ---- groups of queries sharing a bin row ----
    unsigned long long todo = fgc_ballot(qactive);
    while (todo) {
        const int first = __ffsll((long long)todo) - 1;
        const int grow = fgc_readlane_i(row, first);
        const unsigned long long gm = fgc_ballot(qactive && row == grow);
        todo &= ~gm;
        const int last = 63 - __clzll((long long)gm);
        const int zlo = fgc_readlane_i(zq, first), zhi = fgc_readlane_i(zq, last);
        const int ev = grow / rows_per_event;
        int rr = grow - ev * rows_per_event;
        int c[4];
        c[3] = rr % rnb[3]; rr /= rnb[3];
        c[2] = rr % rnb[2]; rr /= rnb[2];
        c[1] = rr % rnb[1]; rr /= rnb[1];
        c[0] = rr;
        const int evrow0 = ev * rows_per_event;

        // -- phase 1: grow the cube until every query of the group holds K candidates --
        int dl = -1;
        bool full = false;
        for (int d = 0;; d++) {
            int lo[4], hi[4];
#pragma unroll
            for (int i = 0; i < 4; i++) { lo[i] = max(c[i] - d, 0); hi[i] = min(c[i] + d, rnb[i] - 1); }
            const int z0 = max(zlo - d, 0), z1 = min(zhi + d, nz - 1);
            for (int a0 = lo[0]; a0 <= hi[0]; a0++)
                for (int a1 = lo[1]; a1 <= hi[1]; a1++)
                    for (int a2 = lo[2]; a2 <= hi[2]; a2++)
                        for (int a3 = lo[3]; a3 <= hi[3]; a3++) {
                            const int cheb = max(max(abs(a0 - c[0]), abs(a1 - c[1])),
                                                 max(abs(a2 - c[2]), abs(a3 - c[3])));
                            const float g01 = gap1(qb[0], a0, a0, rnb[0]) + gap1(qb[1], a1, a1, rnb[1]) +
                                              gap1(qb[2], a2, a2, rnb[2]) + gap1(qb[3], a3, a3, rnb[3]);
                            const int b0 = (evrow0 + ((a0 * rnb[1] + a1) * rnb[2] + a2) * rnb[3] + a3) * nz;
                            if (cheb == d) {
                                process_range(b0 + z0, b0 + z1, g01 + gap1(qzn, z0, z1, nz), gm);
                            } else {
                                if (zlo - d >= 0)
                                    process_range(b0 + zlo - d, b0 + zlo - d, g01 + gap1(qzn, zlo - d, zlo - d, nz), gm);
                                if (zhi + d <= nz - 1)
                                    process_range(b0 + zhi + d, b0 + zhi + d, g01 + gap1(qzn, zhi + d, zhi + d, nz), gm);
                            }
                        }
            dl = d;
            bool covers = (z0 == 0) && (z1 == nz - 1);
#pragma unroll
            for (int i = 0; i < 4; i++) covers = covers && (lo[i] == 0) && (hi[i] == rnb[i] - 1);
            if (covers) { full = true; break; }
            if ((fgc_ballot(tau < INFINITY) & gm) == gm) break;
        }
        if (full) continue;

        // -- phase 2: sweep the bins that intersect the balls of radius sqrt(tau) --
        const bool ing = (gm >> lane) & 1ull;
        const float R = sqrtf(tau) * (1.0f + 1e-5f) + margin;
        int blo[4], bhi[4], sweep_lo[4], sweep_hi[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            blo[i] = (int)fminf(fmaxf(floorf((qb[i] - R) / bw + 1e-3f), 0.f), (float)(rnb[i] - 1));
            bhi[i] = (int)fminf(fmaxf(floorf((qb[i] + R) / bw + 1e-3f), 0.f), (float)(rnb[i] - 1));
            sweep_lo[i] = rnb[i] - 1;
            sweep_hi[i] = 0;
        }
        int bzlo = (int)fminf(fmaxf(floorf((qzn - R) / bw + 1e-3f), 0.f), (float)(nz - 1));
        int bzhi = (int)fminf(fmaxf(floorf((qzn + R) / bw + 1e-3f), 0.f), (float)(nz - 1));
        int szlo = nz - 1, szhi = 0;
        (void)ing;
        for (unsigned long long mm = gm; mm;) {
            const int q = __ffsll((long long)mm) - 1;
            mm &= mm - 1;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                sweep_lo[i] = min(sweep_lo[i], fgc_readlane_i(blo[i], q));
                sweep_hi[i] = max(sweep_hi[i], fgc_readlane_i(bhi[i], q));
            }
            szlo = min(szlo, fgc_readlane_i(bzlo, q));
            szhi = max(szhi, fgc_readlane_i(bzhi, q));
        }
        const int pz0 = max(zlo - dl, 0), pz1 = min(zhi + dl, nz - 1);
        for (int a0 = sweep_lo[0]; a0 <= sweep_hi[0]; a0++)
            for (int a1 = sweep_lo[1]; a1 <= sweep_hi[1]; a1++)
                for (int a2 = sweep_lo[2]; a2 <= sweep_hi[2]; a2++)
                    for (int a3 = sweep_lo[3]; a3 <= sweep_hi[3]; a3++) {
                        const int cheb = max(max(abs(a0 - c[0]), abs(a1 - c[1])),
                                             max(abs(a2 - c[2]), abs(a3 - c[3])));
                        const float g01 = gap1(qb[0], a0, a0, rnb[0]) + gap1(qb[1], a1, a1, rnb[1]) +
                                          gap1(qb[2], a2, a2, rnb[2]) + gap1(qb[3], a3, a3, rnb[3]);
                        if (!(gm & fgc_ballot(!(g01 > tau)))) continue;
                        const int b0 = (evrow0 + ((a0 * rnb[1] + a1) * rnb[2] + a2) * rnb[3] + a3) * nz;
                        if (cheb <= dl) {
                            if (szlo <= pz0 - 1)
                                process_range(b0 + szlo, b0 + pz0 - 1, g01 + gap1(qzn, szlo, pz0 - 1, nz), gm);
                            if (pz1 + 1 <= szhi)
                                process_range(b0 + pz1 + 1, b0 + szhi, g01 + gap1(qzn, pz1 + 1, szhi, nz), gm);
                        } else {
                            process_range(b0 + szlo, b0 + szhi, g01 + gap1(qzn, szlo, szhi, nz), gm);
                        }
                    }
    }

    // ---- write the rows back in the original point order ----
    for (int q = 0; q < nq; q++) {
        const int self = qbeg + q;
        const long long orig_q = (long long)a.order[self];
        float L[NSEG];
        int I[NSEG];
#pragma unroll
        for (int s = 0; s < NSEG; s++) { L[s] = ld[q * KP + s * 64 + lane]; I[s] = li[q * KP + s * 64 + lane]; }
        int p = K - 1;
        bool found = false;
#pragma unroll
        for (int s = 0; s < NSEG; s++) {
            const unsigned long long mm = fgc_ballot(I[s] == self && (s * 64 + lane) < K);
            if (mm && !found) { p = s * 64 + __ffsll((long long)mm) - 1; found = true; }
        }
#pragma unroll
        for (int s = 0; s < NSEG; s++) {
            const int slot = s * 64 + lane;
            float up = __shfl_up(L[s], 1, 64);
            int upi = __shfl_up(I[s], 1, 64);
            if (s > 0) {
                const float cf = fgc_readlane_f(L[s - 1], 63);
                const int cidx = fgc_readlane_i(I[s - 1], 63);
                if (lane == 0) { up = cf; upi = cidx; }
            }
            int oi;
            float od;
            if (slot == 0) { oi = self; od = 0.f; }
            else if (slot <= p) { oi = upi; od = up; }
            else { oi = I[s]; od = L[s]; }
            if (slot < K) {
                long long gi;
                float gd;
                if (oi >= 0) { gi = (long long)a.order[oi]; gd = od; }
                else { gi = a.tf_compat ? orig_q : -1ll; gd = 0.f; }
                a.out_idx[orig_q * K + slot] = gi;
                a.out_dist[orig_q * K + slot] = gd;
            }
        }
    }
    if (a.stats && lane == 0) {
        atomicAdd(&a.stats[0], nev);
        atomicAdd(&a.stats[1], nchunks);
        atomicAdd(&a.stats[2], nins);
    }
}

template <int DT, int NSEG> static int launch_knn_t(const KnnArgs &a, hipStream_t s)
{
    constexpr int WPB = KnnCfg<NSEG>::WPB;
    const int tiles = (int)fgc_cdiv(a.n, QT);
    const int blocks = (int)fgc_cdiv(tiles, WPB);
    hipLaunchKernelGGL((k_knn<DT, NSEG>), dim3(blocks), dim3(WPB * 64), 0, s, a);
    FGC_LAUNCH_CHECK();
    return FGC_OK;
}

template <int NSEG> static int launch_knn_d(const KnnArgs &a, hipStream_t s)
{
    switch (a.D) {
    case 2: return launch_knn_t<2, NSEG>(a, s);
    case 3: return launch_knn_t<3, NSEG>(a, s);
    case 4: return launch_knn_t<4, NSEG>(a, s);
    case 5: return launch_knn_t<5, NSEG>(a, s);
    case 6: return launch_knn_t<6, NSEG>(a, s);
    case 7: return launch_knn_t<7, NSEG>(a, s);
    case 8: return launch_knn_t<8, NSEG>(a, s);
    default: return launch_knn_t<0, NSEG>(a, s);
    }
}

int fgc_launch_knn(const KnnArgs &a, hipStream_t s)
{
    if (a.n <= 0) return FGC_OK;
    if (a.K < 1 || a.K > FGC_MAX_K || a.D < 1 || a.nbd < 1 || a.nbd > FGC_MAX_BIN_DIMS || a.nbd > a.D)
        return FGC_EINVAL;
    if (a.K <= 64) return launch_knn_d<1>(a, s);
    if (a.K <= 128) return launch_knn_d<2>(a, s);
    return launch_knn_d<4>(a, s);
}
