// Exact k-nearest-neighbour search over bin-sorted points (gfx950, wave64).
//
// Work decomposition: one wavefront owns QT consecutive points of the sorted
// order.  The order is (flat bin, Morton code inside the bin), so the queries of
// a wavefront are spatial neighbours and every 64 consecutive points ("chunk")
// form a compact cluster whose bounding box is precomputed.
//
// Candidates are streamed one chunk at a time, one candidate per lane, with
// coalesced loads from the structure-of-arrays coordinate copy; the wavefront
// then walks over the queries that still need the chunk (query coordinates
// broadcast from the owning lane), so a loaded candidate is reused by up to QT
// queries.  Each query owns an unsorted candidate pool in LDS (K kept + room for
// one more chunk); tau_q, an upper bound of the query's K-th distance, lives in
// lane q of a register.  Lanes that beat tau append themselves to the pool
// (ballot + prefix count, no sorting); when the pool runs full it is pruned: a
// bisection on the distance threshold, counted with wave ballots over the pool
// held one slot per lane, finds a tighter tau and the survivors are compacted.
// The steady-state loop is subtract / multiply / add / compare; exact selection
// of the K best and the sort by distance happen once per query at the end.
//
// Search order for the queries of a wavefront that share a bin row (all binned
// coordinates but the last one):
//   seed   the chunks around the wavefront's own position (spatial neighbours)
//          give every query K candidates and a tight tau straight away;
//   grow   ring by ring over the bin rows around the own row; a row is one
//          contiguous range of the sorted order, limited along the last binned
//          coordinate to the bins the balls of radius sqrt(tau) can reach;
//          the growth stops when those balls lie inside the rows already done.
// Two filters keep the work small: per (query, row) the squared gap between the
// query and the row's bin box, and per (query, chunk) the squared gap between
// the query and the chunk's bounding box, both against tau.  The box test uses
// the same float operations as the distance itself, so it can never reject a
// candidate the distance test would accept: the result is the exact kNN set of
// the reference's shell search (binned_select_knn_cuda_kernel.cu:101-248).
#include "fgc_common.h"
#include "fgc_internal.h"

#ifndef QT
#define QT 8           // queries per wavefront
#endif
#define CULL_MIN 3     // ranges of at least this many chunks get the per-chunk box test

// wavefronts per block, chosen so that a block's pools fit the 64 KB static LDS limit
template <int NSEG> struct KnnCfg { static constexpr int WPB = (NSEG <= 2 ? 2 : 1) * (16 / QT); };

template <int DT, int NSEG>
__global__ __launch_bounds__(KnnCfg<NSEG>::WPB * 64) void k_knn(KnnArgs a)
{
    constexpr int PS = NSEG + 1;      // pool segments of 64 slots per query
    constexpr int CAP = PS * 64;      // pool capacity: K kept + one chunk of new candidates
    constexpr int WPB = KnnCfg<NSEG>::WPB;
    constexpr int DR = DT > 0 ? DT : 1;
    __shared__ float s_d[WPB][QT * CAP];
    __shared__ int s_i[WPB][QT * CAP];

    const int lane = fgc_lane();
    const int wv = threadIdx.x >> 6;
    const int qbeg = (blockIdx.x * WPB + wv) * QT;
    if (qbeg >= a.n) return;  // no block-wide barrier is used below
    const int nq = min(QT, a.n - qbeg);
    float *ld = s_d[wv];
    int *li = s_i[wv];

    const int K = a.K, D = a.D, nbd = a.nbd, ldc = a.ldc, nch = a.n_chunks;
    const float *__restrict__ sc = a.sc;
    const int *__restrict__ bb = a.bb;
    const float *__restrict__ box_lo = a.box_lo;
    const float *__restrict__ box_hi = a.box_hi;

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
    const int key = (int)(a.skeys[qs] >> a.key_shift);
    const int row = key / nz;
    float tau = INFINITY;   // lane q: upper bound of query q's K-th distance
    int cnt = 0;            // lane q: candidates in query q's pool
    bool qactive = isq;
    if (a.sdir && isq) { unsigned char dd = a.sdir[qs]; qactive = !(dd == 0 || dd == 2); }

    unsigned long long nev = 0, nchunks = 0, nins = 0, nevents = 0, ncullq = 0, nrows = 0, nqchunk = 0;

    const int slack = max(K >> 2, 4);   // a prune may keep up to K + slack candidates

    // ---- shrink query q's pool.  Finds a threshold t with at least K pool entries <= t by bisection
    //      (counts via wave ballots, the pool held one slot per lane and segment), keeps the entries
    //      <= t and compacts them.  exact: t is the K-th smallest value itself and exactly K entries
    //      stay (ties at t by slot order); otherwise a few bisection steps that stop as soon as at most
    //      K + slack entries remain.  tau_q = t afterwards. ----
    auto prune = [&](int q, bool exact) {
        const int c = fgc_readlane_i(cnt, q);
        if (c <= K) return;
        unsigned P[PS];
        int PI[PS];
        bool valid[PS];
#pragma unroll
        for (int s = 0; s < PS; s++) {
            valid[s] = (s * 64 + lane) < c;
            P[s] = valid[s] ? __float_as_uint(ld[q * CAP + s * 64 + lane]) : 0xffffffffu;
            PI[s] = valid[s] ? li[q * CAP + s * 64 + lane] : -1;
        }
        auto count_le = [&](unsigned t) -> int {
            int n = 0;
#pragma unroll
            for (int s = 0; s < PS; s++) n += __popcll(fgc_ballot(P[s] <= t));
            return n;
        };
        const float told = fgc_readlane_f(tau, q);
        unsigned hi = (told < INFINITY) ? __float_as_uint(told) : 0x7f7fffffu;   // count_le(hi) >= K
        int chi = c;
        bool converged = false;
        if (!exact && told < INFINITY) {
            // linear bisection on [0, tau_old]; distances are non-negative floats
            float flo = 0.f, fhi = told;
            for (int it = 0; it < 10; it++) {
                const float mid = 0.5f * (flo + fhi);
                const int cm = count_le(__float_as_uint(mid));
                if (cm >= K) { fhi = mid; chi = cm; if (cm <= K + slack) { converged = true; break; } }
                else flo = mid;
            }
            hi = __float_as_uint(fhi);
        }
        bool keep[PS];
        int newc;
        if (converged) {
#pragma unroll
            for (int s = 0; s < PS; s++) keep[s] = P[s] <= hi;
            newc = chi;
        } else {
            // bisection on the bit pattern (monotone for non-negative floats) down to the K-th value itself
            unsigned lo = 0u;
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
            newc = K;
        }
        int base = 0;
#pragma unroll
        for (int s = 0; s < PS; s++) {
            const unsigned long long km = fgc_ballot(keep[s]);
            if (keep[s]) {
                const int pos = base + fgc_mbcnt(km);
                ld[q * CAP + pos] = __uint_as_float(P[s]);
                li[q * CAP + pos] = PI[s];
            }
            base += __popcll(km);
        }
        nins++;
        const float tnew = __uint_as_float(hi);
        tau = (lane == q) ? tnew : tau;
        cnt = (lane == q) ? newc : cnt;
    };

    // ---- append the lanes of `pm` (distances dsq, sorted ids jbase + lane) to query q's pool ----
    auto insert = [&](int q, unsigned long long pm, float dsq, int jbase) {
        nevents++;
        int c = fgc_readlane_i(cnt, q);
        int np = __popcll(pm);
        if (c + np > CAP) {
            prune(q, false);
            c = fgc_readlane_i(cnt, q);
            pm = fgc_ballot(dsq < fgc_readlane_f(tau, q));
            np = __popcll(pm);
            if (c + np > CAP) {   // K + slack + a full chunk can exceed the pool: cut back to exactly K
                prune(q, true);
                c = fgc_readlane_i(cnt, q);
                pm = fgc_ballot(dsq < fgc_readlane_f(tau, q));
                np = __popcll(pm);
            }
            if (!pm) return;
        }
        if ((pm >> lane) & 1ull) {
            const int pos = c + fgc_mbcnt(pm);
            ld[q * CAP + pos] = dsq;
            li[q * CAP + pos] = jbase + lane;
        }
        c += np;
        cnt = (lane == q) ? c : cnt;
        // keep tau tight: prune as soon as a quarter-chunk more than K candidates are pooled
        if (c >= K + 32 || (c > K && !(fgc_readlane_f(tau, q) < INFINITY))) prune(q, false);
    };

    // ---- the candidates of chunk c inside [j0, j1) against the queries in `act` ----
    auto process_chunk = [&](int c, int j0, int j1, unsigned long long act) {
        const int base = c << 6;
        const int j = base + lane;
        const bool v = (j >= j0) && (j < j1);
        float cx[DR];
        if (DT > 0) {
#pragma unroll
            for (int d = 0; d < DR; d++) cx[d] = v ? sc[(size_t)d * ldc + j] : 0.f;
        }
        bool cand_ok = v;
        if (a.sdir && v) { unsigned char dd = a.sdir[j]; if (dd == 1 || dd == 2) cand_ok = false; }
        if (DT > 0 && !cand_ok) cx[0] = INFINITY;
        nev += (unsigned long long)__popcll(act) * (unsigned)(min(j1, base + 64) - max(j0, base));
        nchunks++;
        nqchunk += __popcll(act);
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
    };

    // ---- all candidates in sorted positions [j0, j1) against the queries in `act`;
    //      chunks seed_c0..seed_c1 were handled before and are skipped ----
    auto process_span = [&](int j0, int j1, unsigned long long act, int seed_c0, int seed_c1) {
        if (j0 >= j1 || !act) return;
        const int c0 = j0 >> 6, c1 = (j1 - 1) >> 6;
        if (DT == 0 || c1 - c0 + 1 < CULL_MIN) {
            for (int c = c0; c <= c1; c++)
                if (c < seed_c0 || c > seed_c1) process_chunk(c, j0, j1, act);
            return;
        }
        // per-chunk bounding-box test, 64 chunks at a time (lane = chunk)
        for (int cb = c0; cb <= c1; cb += 64) {
            const int c = cb + lane;
            const bool cv = (c <= c1) && (c < seed_c0 || c > seed_c1);
            float blo[DR], bhi[DR];
#pragma unroll
            for (int d = 0; d < DR; d++) {
                blo[d] = cv ? box_lo[(size_t)d * nch + c] : 0.f;
                bhi[d] = cv ? box_hi[(size_t)d * nch + c] : 0.f;
            }
            unsigned mymask = 0;
            unsigned long long m = act;
            ncullq += __popcll(act);
            while (m) {
                const int q = __ffsll((long long)m) - 1;
                m &= m - 1;
                const float t = fgc_readlane_f(tau, q);
                // same operation order as the distance: a candidate inside the box is never closer than this
                float x = fgc_readlane_f(qx[0], q);
                float g = fmaxf(fmaxf(blo[0] - x, x - bhi[0]), 0.f);
                float g2 = g * g;
#pragma unroll
                for (int d = 1; d < DR; d++) {
                    x = fgc_readlane_f(qx[d], q);
                    g = fmaxf(fmaxf(blo[d] - x, x - bhi[d]), 0.f);
                    g2 += g * g;
                }
                if (cv && !(g2 > t)) mymask |= 1u << q;
            }
            unsigned long long any = fgc_ballot(mymask != 0u);
            while (any) {
                const int l = __ffsll((long long)any) - 1;
                any &= any - 1;
                const unsigned long long cact = (unsigned long long)(unsigned)fgc_readlane_i((int)mymask, l);
                process_chunk(cb + l, j0, j1, cact);
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
        const int ev = grow / rows_per_event;
        int rr = grow - ev * rows_per_event;
        int c[4];
        c[3] = rr % rnb[3]; rr /= rnb[3];
        c[2] = rr % rnb[2]; rr /= rnb[2];
        c[1] = rr % rnb[1]; rr /= rnb[1];
        c[0] = rr;
        const int evrow0 = ev * rows_per_event;
        const int ev_j0 = bb[evrow0 * nz], ev_j1 = bb[(evrow0 + rows_per_event) * nz];

        // -- seed: the chunks around the wavefront's own position, inside the event --
        const int own = qbeg >> 6;
        const int seed_c0 = max(own - NSEG, ev_j0 >> 6);
        const int seed_c1 = min(own + NSEG, (ev_j1 - 1) >> 6);
        process_chunk(own, ev_j0, ev_j1, gm);
        for (int cc = seed_c0; cc <= seed_c1; cc++)
            if (cc != own) process_chunk(cc, ev_j0, ev_j1, gm);

        // -- grow ring by ring over the bin rows --
        for (int d = 0;; d++) {
            // bins the balls of radius sqrt(tau) reach (whole grid while a query is not filled)
            const bool filled = (fgc_ballot(tau < INFINITY) & gm) == gm;
            int need_lo[4], need_hi[4], zlo = 0, zhi = nz - 1;
#pragma unroll
            for (int i = 0; i < 4; i++) { need_lo[i] = 0; need_hi[i] = rnb[i] - 1; }
            if (filled) {
                const float R = sqrtf(tau) * (1.0f + 1e-5f) + margin;
                int blo[4], bhi[4];
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    blo[i] = (int)fminf(fmaxf(floorf((qb[i] - R) / bw + 1e-3f), 0.f), (float)(rnb[i] - 1));
                    bhi[i] = (int)fminf(fmaxf(floorf((qb[i] + R) / bw + 1e-3f), 0.f), (float)(rnb[i] - 1));
                    need_lo[i] = rnb[i] - 1;
                    need_hi[i] = 0;
                }
                const int bzlo = (int)fminf(fmaxf(floorf((qzn - R) / bw + 1e-3f), 0.f), (float)(nz - 1));
                const int bzhi = (int)fminf(fmaxf(floorf((qzn + R) / bw + 1e-3f), 0.f), (float)(nz - 1));
                zlo = nz - 1;
                zhi = 0;
                for (unsigned long long mm = gm; mm;) {
                    const int q = __ffsll((long long)mm) - 1;
                    mm &= mm - 1;
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        need_lo[i] = min(need_lo[i], fgc_readlane_i(blo[i], q));
                        need_hi[i] = max(need_hi[i], fgc_readlane_i(bhi[i], q));
                    }
                    zlo = min(zlo, fgc_readlane_i(bzlo, q));
                    zhi = max(zhi, fgc_readlane_i(bzhi, q));
                }
            }
            // rings 0..d-1 are done: stop when nothing outside them is needed
            bool done = d > 0;
#pragma unroll
            for (int i = 0; i < 4; i++) done = done && (need_lo[i] >= c[i] - (d - 1)) && (need_hi[i] <= c[i] + (d - 1));
            if (done) break;
            int lo[4], hi[4];
            bool any_row = false;
#pragma unroll
            for (int i = 0; i < 4; i++) { lo[i] = max(c[i] - d, 0); hi[i] = min(c[i] + d, rnb[i] - 1); }
            for (int a0 = lo[0]; a0 <= hi[0]; a0++)
                for (int a1 = lo[1]; a1 <= hi[1]; a1++)
                    for (int a2 = lo[2]; a2 <= hi[2]; a2++)
                        for (int a3 = lo[3]; a3 <= hi[3]; a3++) {
                            const int cheb = max(max(abs(a0 - c[0]), abs(a1 - c[1])),
                                                 max(abs(a2 - c[2]), abs(a3 - c[3])));
                            if (cheb != d) continue;
                            any_row = true;
                            nrows++;
                            const float g2 = gap1(qb[0], a0, a0, rnb[0]) + gap1(qb[1], a1, a1, rnb[1]) +
                                             gap1(qb[2], a2, a2, rnb[2]) + gap1(qb[3], a3, a3, rnb[3]) +
                                             gap1(qzn, zlo, zhi, nz);
                            const unsigned long long act = gm & fgc_ballot(!(g2 > tau));
                            if (!act) continue;
                            const int b0 = (evrow0 + ((a0 * rnb[1] + a1) * rnb[2] + a2) * rnb[3] + a3) * nz;
                            process_span(bb[b0 + zlo], bb[b0 + zhi + 1], act, seed_c0, seed_c1);
                        }
            if (!any_row) break;  // the ring lies outside the grid: everything has been visited
        }
    }

    // ---- per query: cut the pool to exactly K, sort by distance, write the row at the query's
    //      original position (slot 0 = the query itself) ----
    for (int q = 0; q < nq; q++) {
        const int self = qbeg + q;
        const long long orig_q = (long long)a.order[self];
        prune(q, true);
        const int c = fgc_readlane_i(cnt, q);     // <= K entries now, compacted in slots 0..c-1
        float L[NSEG];
        int I[NSEG], rank[NSEG];
        bool valid[NSEG];
#pragma unroll
        for (int s = 0; s < NSEG; s++) {
            valid[s] = (s * 64 + lane) < c;
            L[s] = valid[s] ? ld[q * CAP + s * 64 + lane] : INFINITY;
            I[s] = valid[s] ? li[q * CAP + s * 64 + lane] : -1;
            if (valid[s] && I[s] == self) L[s] = -1.f;   // the query itself sorts first
            rank[s] = 0;
        }
        bool has_self = false;
#pragma unroll
        for (int s = 0; s < NSEG; s++) has_self = has_self || (fgc_ballot(valid[s] && I[s] == self) != 0ull);
        // rank sort: position = number of entries that precede (by distance, then slot)
        for (int e = 0; e < c; e++) {
            float v = 0.f;
#pragma unroll
            for (int s = 0; s < NSEG; s++)
                if ((e >> 6) == s) v = fgc_readlane_f(L[s], e & 63);
#pragma unroll
            for (int s = 0; s < NSEG; s++) rank[s] += ((v < L[s]) || (v == L[s] && e < s * 64 + lane)) ? 1 : 0;
        }
        const int shift = has_self ? 0 : 1;       // without the query in the pool its slot 0 is added here
        const int n_out = min(c + shift, K);
#pragma unroll
        for (int s = 0; s < NSEG; s++) {
            const int slot = rank[s] + shift;
            if (valid[s] && slot < K) {
                const bool is_self = I[s] == self;
                a.out_idx[orig_q * K + slot] = is_self ? orig_q : (long long)a.order[I[s]];
                a.out_dist[orig_q * K + slot] = is_self ? 0.f : L[s];
            }
            const int pslot = s * 64 + lane;      // padding slots and, if needed, the query's own slot 0
            if (pslot < K && pslot >= n_out) {
                a.out_idx[orig_q * K + pslot] = a.tf_compat ? orig_q : -1ll;
                a.out_dist[orig_q * K + pslot] = 0.f;
            }
            if (!has_self && pslot == 0) {
                a.out_idx[orig_q * K] = orig_q;
                a.out_dist[orig_q * K] = 0.f;
            }
        }
    }
    if (a.stats && lane == 0) {
        atomicAdd(&a.stats[0], nev);
        atomicAdd(&a.stats[1], nchunks);
        atomicAdd(&a.stats[2], nins);
        atomicAdd(&a.stats[3], nevents);
        atomicAdd(&a.stats[4], ncullq);
        atomicAdd(&a.stats[5], nrows);
        atomicAdd(&a.stats[6], nqchunk);
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
