// Exact k-nearest-neighbour search over bin-sorted points (gfx950, wave64).
//
// Work decomposition: one wavefront owns QT consecutive points of the sorted
// order.  The order is (flat bin, Hilbert index inside the bin), so the queries of
// a wavefront are spatial neighbours and every 64 consecutive points ("chunk")
// form a compact cluster whose bounding box is precomputed.
//
// Candidates are streamed one chunk at a time, one candidate per lane, with
// coalesced loads from the structure-of-arrays coordinate copy; the wavefront
// then walks over the queries that still need the chunk (the queries' coordinates,
// bounds and pool counts are held as wave-uniform values in scalar registers, the
// walk is unrolled over them), so a loaded candidate is reused by up to QT
// queries.  Each query owns an unsorted candidate pool in LDS (K kept + room for
// one more chunk); tau_q, an upper bound of the query's K-th distance, lives in
// lane q of a register (and in a scalar copy).  Lanes that beat tau append themselves to the pool
// (ballot + prefix count, no sorting); when the pool runs full it is pruned: a
// bisection on the distance threshold, counted with wave ballots over the pool
// held one slot per lane, finds a tighter tau and the survivors are compacted.
// The steady-state loop is subtract / multiply / add / compare; exact selection
// of the K best happens once per query at the end, followed by a sort by distance
// only when the caller asks for ordered rows (the reference's rows have no order).
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
//
// The whole search of a group is one loop over "spans" (seed spans first, then
// one span per bin row) with a single copy of the chunk / pool code inside: the
// kernel stays small in registers and instructions, which is what bounds its
// occupancy.
#include "fgc_common.h"
#include "fgc_internal.h"
#include "fgc_knn_sort.h"

// This file is compiled twice: as it is, and with -DFGC_KNN_STATS for the variant that also counts distance
// evaluations, candidate chunks and prunes (fgc_launch_knn_stats, kernels k_knn_stats): the counters cost scalar
// registers and instructions in the inner loops (3-5 % of the search), so calls that do not ask for them get
// kernels without.
#ifdef FGC_KNN_STATS
#define k_knn k_knn_stats
#define fgc_launch_knn fgc_launch_knn_stats
#elif defined(FGC_KNN_COUNTERS)
#undef FGC_KNN_COUNTERS        // the debug counters exist in the statistics build only
#endif

#ifndef QT_DEFAULT
#define QT_DEFAULT 6   // queries per wavefront (6 x 128 pool slots x 8 B = 6 KB of LDS at K = 64: 26 wavefronts per CU)
#endif
#ifndef QT_SMALL
#define QT_SMALL 3     // for inputs too small to fill the GPU with wavefronts of 6 queries: twice the wavefronts, each with
#endif                 // half the serial work (search of 10 000 points, D = 3, K = 40: 45 -> 33 us; 40 000: 88 -> 82; 80 000: 142 -> 147)
#ifndef KNN_SMALL_N
#define KNN_SMALL_N 49152
#endif
#ifndef POOL_EXTRA
#define POOL_EXTRA 48  // pool slots beyond K (rounded up to 16); LDS per wavefront = QT * pool slots * 8 B
#endif
#ifndef POOL_EXTRA_SMALL_K
#define POOL_EXTRA_SMALL_K 64
#endif
#ifndef PRUNE_MARGIN
#define PRUNE_MARGIN 24 // a pool is pruned when fewer than this many slots are free
#endif
#ifndef SEED_K
#define SEED_K 40    // one seed chunk on either side of the wavefront's own chunk per this many neighbours asked for
#endif
#ifndef CULL_MIN
#define CULL_MIN 5     // spans of at least this many chunks get the per-chunk box test
#endif

// wavefronts per block, chosen so that a block's pools fit the 64 KB static LDS limit
// one wavefront per block: no block-level cooperation is used, and small blocks pack the LDS of a CU best
template <int NSEG> struct KnnCfg { static constexpr int WPB = 1; };

// DT: coordinates per point held in registers (0 = any number, read from memory)
// NSEG: ceil(K / 64);  RD: bin-row dimensions (binned dimensions - 1, padded);  QT: queries per wavefront
template <int DT, int NSEG, int RD, int QT>
__global__ __launch_bounds__(KnnCfg<NSEG>::WPB * 64) void k_knn(KnnArgs a)
{
    constexpr int PS = NSEG + 1;          // pool segments (lanes x PS cover the pool)
    constexpr int WPB = KnnCfg<NSEG>::WPB;
    constexpr int DR = DT > 0 ? DT : 1;
    extern __shared__ uint2 s_pool[];     // [WPB][QT * CAP] (distance bits, sorted position): one 8-byte LDS access per entry
    const int CAP = a.pool_cap;           // pool capacity per query: K kept + room for new candidates

    const int lane = fgc_lane();
    // wave index made explicitly uniform: everything derived from it (tile start, seed chunks, spans)
    // then stays in scalar registers and scalar control flow
    const int wv = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int qbeg = (blockIdx.x * WPB + wv) * QT;
    if (qbeg >= a.n) return;  // no block-wide barrier is used below
    const int nq = min(QT, a.n - qbeg);
    uint2 *pool = s_pool + (size_t)wv * QT * CAP;

    const int K = a.K, ldc = a.ldc, nch = a.n_chunks;
    const int nbd = RD >= 2 ? RD + 1 : a.nbd;     // binned dimensions: RD + 1 except for the smallest instantiation (1 or 2)
    // coordinates per point: a compile-time constant where the kernel is built for exactly that many (2 .. 8), so
    // that the per-coordinate guards of the loads fold away
    const int Dn = (DT >= 2 && DT <= 8) ? DT : a.D;
    const float *__restrict__ sc = a.sc;
    const int *__restrict__ bb = a.bb;

    // ---- geometry (wave-uniform) ----
    const float bw = a.geom[FGC_GEOM_BW];
    const float margin = 1e-4f * bw;
    int rnb[RD];  // bins of the row dimensions (all binned dimensions but the last), padded with 1
    int rows_per_event = 1;
#pragma unroll
    for (int i = 0; i < RD; i++) {
        rnb[i] = (i < nbd - 1) ? __float_as_int(a.geom[FGC_GEOM_NB + i]) : 1;
        rows_per_event *= rnb[i];
    }
    const int nz = __float_as_int(a.geom[FGC_GEOM_NB + nbd - 1]);

    // ---- per-lane query state (lane q < nq holds query qbeg + q) ----
    const bool isq = lane < nq;
    const int qs = qbeg + (isq ? lane : 0);
    float qx[DR];
    if (DT > 0) {
#pragma unroll
        for (int d = 0; d < DR; d++) qx[d] = (d < Dn) ? sc[(size_t)d * ldc + qs] : 0.f;   // padded dimensions: 0
    }
    float qb[RD];  // normalised row-dimension coordinates
#pragma unroll
    for (int i = 0; i < RD; i++) qb[i] = (i < nbd - 1) ? sc[(size_t)i * ldc + qs] - a.geom[FGC_GEOM_MIN + i] : 0.f;
    const float qzn = sc[(size_t)(nbd - 1) * ldc + qs] - a.geom[FGC_GEOM_MIN + nbd - 1];
    const int row = (int)(a.skeys[qs] >> a.key_shift) / nz;
    float tau = a.tau0;     // lane q: upper bound of query q's K-th distance (starts at the radius bound, if any)
    int cnt = 0;            // lane q: candidates in query q's pool
    bool qactive = isq;
    if (a.sdir && isq) { unsigned char dd = a.sdir[qs]; qactive = !(dd == 0 || dd == 2); }
    // With few coordinates the queries' coordinates and bounds are also kept as wave-uniform values (scalar registers):
    // the loops over the queries of a chunk are unrolled and the subtractions take them as scalar operands, instead
    // of one v_readlane per coordinate and (query, chunk).  st[q] mirrors lane q of tau and is refreshed wherever tau
    // changes (seeds, prunes).
    //    sn[q] likewise stands for lane q of cnt while the spans of a group are searched: the common pool append then
    //    touches no per-lane state at all; cnt is brought up to date before anything else reads it (a prune, the epilogue).
    constexpr bool SQ = DT >= 2;
    float sq[SQ ? QT : 1][DR], st[SQ ? QT : 1];
    int sn[SQ ? QT : 1];
    if (SQ) {
#pragma unroll
        for (int q = 0; q < QT; q++) {
#pragma unroll
            for (int dd = 0; dd < DR; dd++) sq[q][dd] = fgc_readlane_f(qx[dd], q);
            st[q] = a.tau0;
            sn[q] = 0;
        }
    }
    // second launch behind the matrix-core search: only the queries it flagged
    const bool redo_q = !a.redo || (isq && a.redo[qs] != 0);
    if (a.redo) {
        if (!fgc_ballot(redo_q)) return;
        qactive = qactive && redo_q;
    }

#ifdef FGC_KNN_STATS
    unsigned long long nev = 0;
    unsigned nchunks = 0, nprunes = 0;
#endif
#ifdef FGC_KNN_COUNTERS
    unsigned n_cullq = 0, n_app = 0, n_span = 0, n_bis = 0, n_bisx = 0;
#define CNT(x) x
#else
#define CNT(x)
#endif
#ifndef SLACK_SHIFT
#define SLACK_SHIFT 3
#endif
    const int slack = max(K >> SLACK_SHIFT, 4);   // a prune may keep up to K + slack candidates

    // ---- shrink query q's pool.  Finds a threshold t with at least K pool entries <= t by bisection
    //      (counts via wave ballots, the pool held one slot per lane and segment), keeps the entries
    //      <= t and compacts them.  exact: exactly K entries stay (ties at the K-th value are cut by
    //      slot order); otherwise the bisection stops as soon as at most K + slack entries remain.
    //      tau_q = t afterwards. ----
    auto prune = [&](int q, bool exact) {
        const int c = fgc_readlane_i(cnt, q);
        if (c <= K) return;
        unsigned P[PS];
        int PI[PS];
#pragma unroll
        for (int s = 0; s < PS; s++) {
            const bool valid = (s * 64 + lane) < c;
            const uint2 e = valid ? pool[q * CAP + s * 64 + lane] : make_uint2(0xffffffffu, 0xffffffffu);
            P[s] = e.x;
            PI[s] = (int)e.y;
        }
        auto count_le = [&](unsigned t) -> int {
            int n = 0;
#pragma unroll
            for (int s = 0; s < PS; s++) n += __popcll(fgc_ballot(P[s] <= t));
            return n;
        };
        float told = fgc_readlane_f(tau, q);
        if (!(told < INFINITY)) {              // first fill: bracket by the largest distance in the pool
            int mx = 0;
#pragma unroll
            for (int s = 0; s < PS; s++) mx = max(mx, P[s] == 0xffffffffu ? 0 : (int)P[s]);
            told = __int_as_float(fgc_wave_max_i(mx));
        }
        unsigned hi = (told < INFINITY) ? __float_as_uint(told) : 0x7f7fffffu;   // count_le(hi) >= K
        int chi = c;
        bool converged = false;
        if (told < INFINITY) {
            // linear bisection on [0, tau_old] (distances are non-negative); stops as soon as the count is
            // inside [K, K + slack] - for an exact cut only at exactly K
            const int accept = exact ? K : K + slack;
            const int iters = exact ? 20 : 10;
            float flo = 0.f, fhi = told;
            for (int it = 0; it < iters; it++) {
                const float mid = 0.5f * (flo + fhi);
                const int cm = count_le(__float_as_uint(mid));
                CNT(if (exact) n_bisx++; else n_bis++);
                if (cm >= K) { fhi = mid; chi = cm; if (cm <= accept) { converged = true; break; } }
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
            // bisection on the bit pattern (monotone for non-negative floats) down to the K-th value itself;
            // ties at that value are cut by slot order
            unsigned lo = 0u;
            while (lo < hi) {
                const unsigned mid = lo + ((hi - lo) >> 1);
                CNT(n_bisx++);
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
                pool[q * CAP + pos] = make_uint2(P[s], (unsigned)PI[s]);
            }
            base += __popcll(km);
        }
#ifdef FGC_KNN_STATS
        nprunes++;
#endif
        const float tnew = __uint_as_float(hi);
        tau = (lane == q) ? tnew : tau;
        cnt = (lane == q) ? newc : cnt;
    };

    // squared gap (with safety margin) of this lane's query to a bin interval [b0, b1] of extent nbn
    auto gap1 = [&](float x, int b0, int b1, int nbn) -> float {
        const float lo = (b0 <= 0) ? -INFINITY : ((float)b0 - 1e-3f) * bw;
        const float hi = (b1 >= nbn - 1) ? INFINITY : ((float)(b1 + 1) - 1e-3f) * bw;
        float g = fmaxf(fmaxf(lo - x, x - hi) - margin, 0.f);
        return g * g;
    };

    // ---- append the lanes in `want` (candidate j at squared distance dsq, one per lane) to query q's pool; when
    //      it overflows or runs nearly full (tau should stay tight) prune it: first to a tighter threshold, then,
    //      if lanes are still waiting, down to exactly K ----
    //      Returns true when the query's bound may have changed (a prune ran).
    auto push = [&](int q, float dsq, int j, bool want) -> bool {
        unsigned long long pm = fgc_ballot(want);
        if (!pm) return false;
        CNT(n_app++);
        int pc = fgc_readlane_i(cnt, q);
        {
            // the common case on a short path of its own: everything fits with room to spare and the query has
            // a bound already (what the loop below does in its first pass when it ends there)
            const int pn = pc + __popcll(pm);
            if (pn <= CAP - PRUNE_MARGIN && (pn <= K || ((fgc_ballot(tau < INFINITY) >> q) & 1ull))) {
                if (want) pool[q * CAP + pc + fgc_mbcnt(pm)] = make_uint2(__float_as_uint(dsq), (unsigned)j);
                cnt = (lane == q) ? pn : cnt;
                return false;
            }
        }
        for (int attempt = 0;; attempt++) {
            const int room = CAP - pc;
            const int rnk = fgc_mbcnt(pm);
            const bool put = want && rnk < room;
            if (put) pool[q * CAP + pc + rnk] = make_uint2(__float_as_uint(dsq), (unsigned)j);
            const int npm = __popcll(pm);
            pc += min(npm, room);
            cnt = (lane == q) ? pc : cnt;
            const bool left = npm > room;          // lanes of rank >= room are still waiting
            if (!left && pc <= CAP - PRUNE_MARGIN && (pc <= K || fgc_readlane_f(tau, q) < INFINITY)) break;
            prune(q, attempt > 0);
            if (!left) break;
            pc = fgc_readlane_i(cnt, q);
            want = want && rnk >= room && dsq < fgc_readlane_f(tau, q);
            pm = fgc_ballot(want);
            if (!pm) break;
        }
        return true;
    };
    // the same with the query's count and bound held as wave-uniform values (sc = sn[q], stq = st[q])
    auto push_s = [&](int q, float dsq, int j, bool want, int &sc, float &stq) {
        const unsigned long long pm = fgc_ballot(want);
        if (!pm) return;
        CNT(n_app++);
        const int pn = sc + __popcll(pm);
        if (pn <= CAP - PRUNE_MARGIN && (pn <= K || stq < INFINITY)) {
            if (want) pool[q * CAP + sc + fgc_mbcnt(pm)] = make_uint2(__float_as_uint(dsq), (unsigned)j);
            sc = pn;
            return;
        }
        CNT(n_app--);
        cnt = (lane == q) ? sc : cnt;
        push(q, dsq, j, want);
        sc = fgc_readlane_i(cnt, q);
        stq = fgc_readlane_f(tau, q);
    };

    // ---- groups of queries sharing a bin row ----
    unsigned long long todo = fgc_ballot(qactive);
    while (todo) {
        const int first = __ffsll((long long)todo) - 1;
        const int grow = fgc_readlane_i(row, first);
        const unsigned long long gm = fgc_ballot(qactive && row == grow);
        todo &= ~gm;
        const int ev = grow / rows_per_event;
        int cr[RD];   // the group's own bin row
        {
            int rr = grow - ev * rows_per_event;
#pragma unroll
            for (int i = RD - 1; i >= 0; i--) { cr[i] = rr % rnb[i]; rr /= rnb[i]; }
        }
        const int evrow0 = ev * rows_per_event;
        const int ev_j0 = bb[evrow0 * nz], ev_j1 = bb[(evrow0 + rows_per_event) * nz];
        const int own = qbeg >> 6;
        const int seed_w = (K + SEED_K - 1) / SEED_K;
        const int seed_c0 = max(own - seed_w, ev_j0 >> 6);
        const int seed_c1 = min(own + seed_w, (ev_j1 - 1) >> 6);

        // ---- seeds in registers.  Up to SMAX chunks around the own one are held one candidate per lane; per query
        //      their distances stay in registers, a bisection on ballot counts finds a bound with K .. K + slack of
        //      them below it, and only those go into the pool - the query starts with a finite tau and a pool that
        //      needs no pruning, instead of pushing every seed candidate through the pool and cutting it down two
        //      or three times. ----
        constexpr int SMAX = DT == 0 ? 0 : (16 / DR >= 5 ? 5 : (16 / DR >= 1 ? 16 / DR : 1));
        int ra = own, rb = own - 1;             // register seeds: chunks ra..rb (none for DT == 0)
        if (SMAX > 0) {
            ra = max(seed_c0, own - (SMAX - 1) / 2);
            rb = min(seed_c1, ra + SMAX - 1);
            ra = max(seed_c0, rb - SMAX + 1);
            float sx[SMAX > 0 ? SMAX : 1][DR];
            bool sv[SMAX > 0 ? SMAX : 1];
#pragma unroll
            for (int s = 0; s < SMAX; s++) {
                const int j = ((ra + s) << 6) + lane;
                sv[s] = (ra + s <= rb) && j >= ev_j0 && j < ev_j1;
                if (a.sdir && sv[s]) { unsigned char dd = a.sdir[j]; if (dd == 1 || dd == 2) sv[s] = false; }
#pragma unroll
                for (int dd = 0; dd < DR; dd++) sx[s][dd] = (ra + s <= rb && dd < Dn) ? sc[(size_t)dd * ldc + j] : 0.f;
            }
#ifdef FGC_KNN_STATS
            nchunks += (unsigned)(rb - ra + 1);
#endif
            for (unsigned long long m = gm; m;) {
                const int q = __ffsll((long long)m) - 1;
                m &= m - 1;
                const float t0 = fgc_readlane_f(tau, q);
                unsigned ds[SMAX > 0 ? SMAX : 1];      // distance bit patterns, 0xffffffff = no candidate
                int total = 0;
                unsigned mx = 0u;
#pragma unroll
                for (int s = 0; s < SMAX; s++) {
                    float df = fgc_readlane_f(qx[0], q) - sx[s][0];
                    float dsq = df * df;
#pragma unroll
                    for (int dd = 1; dd < DR; dd++) { df = fgc_readlane_f(qx[dd], q) - sx[s][dd]; dsq += df * df; }
                    const bool ok = sv[s] && dsq < t0;
                    ds[s] = ok ? __float_as_uint(dsq) : 0xffffffffu;
                    const unsigned long long okm = fgc_ballot(ok);
                    total += __popcll(okm);
#ifdef FGC_KNN_STATS
                    nev += (unsigned long long)__popcll(fgc_ballot(sv[s]));
#endif
                    mx = max(mx, ok ? ds[s] : 0u);
                }
                unsigned sel = 0xfffffffeu;             // candidates <= sel are pushed: everything by default
                if (total > K + slack) {
                    float flo = 0.f, fhi = __int_as_float(fgc_wave_max_i((int)mx));
                    for (int it = 0; it < 12; it++) {
                        const float mid = 0.5f * (flo + fhi);
                        int cm = 0;
#pragma unroll
                        for (int s = 0; s < SMAX; s++) cm += __popcll(fgc_ballot(ds[s] <= __float_as_uint(mid)));
                        CNT(n_bis++);
                        if (cm >= K) {
                            fhi = mid;
                            if (cm <= K + slack) {      // K .. K + slack seeds lie within mid: the first bound
                                sel = __float_as_uint(mid);
                                tau = (lane == q) ? mid : tau;
                                break;
                            }
                        } else flo = mid;
                    }
                }
                if (total <= K + slack || sel != 0xfffffffeu) {
                    // the selected seeds fit the (still empty) pool as they are: one compaction over the registers
                    int base = fgc_readlane_i(cnt, q);
#pragma unroll
                    for (int s = 0; s < SMAX; s++) {
                        const bool want = ds[s] <= sel;
                        const unsigned long long wm = fgc_ballot(want);
                        if (want) pool[q * CAP + base + fgc_mbcnt(wm)] = make_uint2(ds[s], (unsigned)(((ra + s) << 6) + lane));
                        base += __popcll(wm);
                    }
                    cnt = (lane == q) ? base : cnt;
                } else {
                    // no bound with K .. K + slack seeds below it (many equal distances): through the pool
#pragma unroll
                    for (int s = 0; s < SMAX; s++)
                        push(q, __uint_as_float(ds[s]), ((ra + s) << 6) + lane, ds[s] <= sel);
                }
            }
        }

        if (SQ) {
#pragma unroll
            for (int q = 0; q < QT; q++) { st[q] = fgc_readlane_f(tau, q); sn[q] = fgc_readlane_i(cnt, q); }
        }
        // span iteration state: phase 0 = own chunk, 1 = the other seed chunks, 2 = bin rows ring by ring
        int phase = (SMAX > 0) ? ((ra == seed_c0 && rb == seed_c1) ? 2 : 1) : 0, d = 0;
        int ai[RD], lo[RD], hi[RD];
        int zlo = 0, zhi = nz - 1;
        bool ring_open = false, ring_fresh = false, ring_any = false;
#pragma unroll
        for (int i = 0; i < RD; i++) { ai[i] = 0; lo[i] = 0; hi[i] = 0; }

        for (;;) {
            int j0, j1, sk0, sk1;
            unsigned long long act;
            if (phase == 0) {
                j0 = max(ev_j0, own << 6); j1 = min(ev_j1, (own << 6) + 64);
                sk0 = 1; sk1 = 0; act = gm; phase = 1;
            } else if (phase == 1) {
                j0 = max(ev_j0, seed_c0 << 6); j1 = min(ev_j1, (seed_c1 + 1) << 6);
                sk0 = (SMAX > 0) ? ra : own; sk1 = (SMAX > 0) ? rb : own; act = gm; phase = 2;
            } else {
                if (!ring_open) {
                    // start ring d: the bins the balls of radius sqrt(tau) reach (whole grid while a
                    // query of the group has fewer than K candidates)
                    const bool filled = (fgc_ballot(tau < INFINITY) & gm) == gm;
                    int need_lo[RD], need_hi[RD];
                    zlo = 0; zhi = nz - 1;
#pragma unroll
                    for (int i = 0; i < RD; i++) { need_lo[i] = 0; need_hi[i] = rnb[i] - 1; }
                    if (filled) {
                        const float R = sqrtf(tau) * (1.0f + 1e-5f) + margin;
                        int blo[RD], bhi[RD];
#pragma unroll
                        for (int i = 0; i < RD; i++) {
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
                            for (int i = 0; i < RD; i++) {
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
                    for (int i = 0; i < RD; i++)
                        done = done && (need_lo[i] >= cr[i] - (d - 1)) && (need_hi[i] <= cr[i] + (d - 1));
                    if (done) break;
                    // ring d, clipped to the grid and to the bins the balls can reach
#pragma unroll
                    for (int i = 0; i < RD; i++) {
                        lo[i] = max(cr[i] - d, need_lo[i]);
                        hi[i] = min(cr[i] + d, need_hi[i]);
                        ai[i] = lo[i];
                    }
                    ring_open = true; ring_fresh = true; ring_any = false;
                }
                if (ring_fresh) {
                    ring_fresh = false;
                } else {
                    bool carry = true;
#pragma unroll
                    for (int i = RD - 1; i >= 0; i--)
                        if (carry) { if (ai[i] < hi[i]) { ai[i]++; carry = false; } else ai[i] = lo[i]; }
                    if (carry) {             // ring finished
                        ring_open = false;
                        if (!ring_any) break;  // the ring lies outside the grid: everything has been visited
                        d++;
                        continue;
                    }
                }
                int cheb = 0, rf = 0;
#pragma unroll
                for (int i = 0; i < RD; i++) {
                    if (i < RD - 1) cheb = max(cheb, abs(ai[i] - cr[i]));
                    rf = rf * rnb[i] + ai[i];
                }
                if (cheb < d && abs(ai[RD - 1] - cr[RD - 1]) < d) {
                    // interior of the ring's cube: jump to the far face of the last row dimension (or to the
                    // end of this line when that face is clipped away)
                    ai[RD - 1] = (cr[RD - 1] + d <= hi[RD - 1]) ? cr[RD - 1] + d - 1 : hi[RD - 1];
                    continue;
                }
                float g2 = gap1(qzn, zlo, zhi, nz);
#pragma unroll
                for (int i = 0; i < RD; i++) g2 += gap1(qb[i], ai[i], ai[i], rnb[i]);
                ring_any = true;
                act = gm & fgc_ballot(!(g2 > tau));
                if (!act) continue;
                const int b0 = (evrow0 + rf) * nz;
                j0 = bb[b0 + zlo]; j1 = bb[b0 + zhi + 1];
                sk0 = seed_c0; sk1 = seed_c1;
            }
            if (j0 >= j1) continue;

            // ---- one span: sorted positions [j0, j1) against the queries in `act`, chunks sk0..sk1 skipped ----
            const int c0 = j0 >> 6, c1 = (j1 - 1) >> 6;
            const bool cull = (DT > 0) && (c1 - c0 + 1 >= CULL_MIN);
            CNT(n_span++);
            for (int cb = cull ? (c0 & ~63) : c0; cb <= c1; cb += 64) {
                unsigned long long actb = act;
                if (cull) {
                    // the 64 chunks of this step are one aligned group with a bounding box of its own:
                    // drop the queries (lane = query) whose ball does not reach it
                    const int sb = cb >> 6;
                    float g = fmaxf(fmaxf(a.sbox_lo[sb] - qx[0], qx[0] - a.sbox_hi[sb]), 0.f);
                    float g2 = g * g;
#pragma unroll
                    for (int dd = 1; dd < DR; dd++) {
                        if (dd < Dn) {
                            g = fmaxf(fmaxf(a.sbox_lo[(size_t)dd * a.n_super + sb] - qx[dd],
                                            qx[dd] - a.sbox_hi[(size_t)dd * a.n_super + sb]), 0.f);
                            g2 += g * g;
                        }
                    }
                    actb &= fgc_ballot(!(g2 > tau));
                    if (!actb) continue;
                }
                const int c = cb + lane;
                const bool cv = (c >= c0) && (c <= c1) && (c < sk0 || c > sk1);
                unsigned mymask = cv ? (unsigned)actb : 0u;   // queries (bit q) that need chunk c
                if (cull) {
                    // per-chunk bounding-box test, lane = chunk
                    float blo[DR], bhi[DR];
#pragma unroll
                    for (int dd = 0; dd < DR; dd++) {
                        blo[dd] = (cv && dd < Dn) ? a.box_lo[(size_t)dd * nch + c] : 0.f;
                        bhi[dd] = (cv && dd < Dn) ? a.box_hi[(size_t)dd * nch + c] : 0.f;
                    }
                    mymask = 0u;
                    if (SQ) {
#pragma unroll
                        for (int q = 0; q < QT; q++) {
                            if (!((actb >> q) & 1ull)) continue;
                            CNT(n_cullq++);
                            float g = fmaxf(fmaxf(blo[0] - sq[q][0], sq[q][0] - bhi[0]), 0.f);
                            float g2 = g * g;
#pragma unroll
                            for (int dd = 1; dd < DR; dd++) {
                                g = fmaxf(fmaxf(blo[dd] - sq[q][dd], sq[q][dd] - bhi[dd]), 0.f);
                                g2 += g * g;
                            }
                            if (cv && !(g2 > st[q])) mymask |= 1u << q;
                        }
                    } else
                    for (unsigned long long m = actb; m;) {
                        CNT(n_cullq++);
                        const int q = __ffsll((long long)m) - 1;
                        m &= m - 1;
                        const float t = fgc_readlane_f(tau, q);
                        // same operation order as the distance: no candidate inside the box is closer than this
                        float x = fgc_readlane_f(qx[0], q);
                        float g = fmaxf(fmaxf(blo[0] - x, x - bhi[0]), 0.f);
                        float g2 = g * g;
#pragma unroll
                        for (int dd = 1; dd < DR; dd++) {
                            x = fgc_readlane_f(qx[dd], q);
                            g = fmaxf(fmaxf(blo[dd] - x, x - bhi[dd]), 0.f);
                            g2 += g * g;
                        }
                        if (cv && !(g2 > t)) mymask |= 1u << q;
                    }
                }
                // The coordinates of the next surviving chunk are requested before the current one is evaluated
                // (rows are padded to whole chunks, so a whole chunk can always be read).
                unsigned long long any = fgc_ballot(mymask != 0u);
                float nx[DR];
                if (DT > 0 && any) {
                    const int jn = ((cb + __ffsll((long long)any) - 1) << 6) + lane;
#pragma unroll
                    for (int dd = 0; dd < DR; dd++) nx[dd] = (dd < Dn) ? sc[(size_t)dd * ldc + jn] : 0.f;
                }
                while (any) {
                    const int l = __ffsll((long long)any) - 1;
                    any &= any - 1;
                    const unsigned long long cact = (unsigned long long)(unsigned)fgc_readlane_i((int)mymask, l);
                    // ---- chunk cb + l: one candidate per lane ----
                    const int base = (cb + l) << 6;
                    const int j = base + lane;
                    const bool v = (j >= j0) && (j < j1);
                    float cx[DR];
                    if (DT > 0) {
#pragma unroll
                        for (int dd = 0; dd < DR; dd++) cx[dd] = nx[dd];
                        if (any) {
                            const int jn = ((cb + __ffsll((long long)any) - 1) << 6) + lane;
#pragma unroll
                            for (int dd = 0; dd < DR; dd++) nx[dd] = (dd < Dn) ? sc[(size_t)dd * ldc + jn] : 0.f;
                        }
                    }
                    bool cand_ok = v;
                    if (a.sdir && v) { unsigned char dd = a.sdir[j]; if (dd == 1 || dd == 2) cand_ok = false; }
                    if (DT > 0 && !cand_ok) cx[0] = INFINITY;
#ifdef FGC_KNN_STATS
                    nev += (unsigned long long)__popcll(cact) * (unsigned)(min(j1, base + 64) - max(j0, base));
                    nchunks++;
#endif
                    if (SQ) {
#pragma unroll
                        for (int q = 0; q < QT; q++) {
                            if (!((cact >> q) & 1ull)) continue;
                            float df = sq[q][0] - cx[0];
                            float dsq = df * df;
#pragma unroll
                            for (int dd = 1; dd < DR; dd++) { df = sq[q][dd] - cx[dd]; dsq += df * df; }
                            push_s(q, dsq, j, dsq < st[q], sn[q], st[q]);
                        }
                    } else
                    for (unsigned long long m = cact; m;) {
                        const int q = __ffsll((long long)m) - 1;
                        m &= m - 1;
                        const float t = fgc_readlane_f(tau, q);
                        float dsq;
                        if (DT > 0) {
                            float df = fgc_readlane_f(qx[0], q) - cx[0];
                            dsq = df * df;
#pragma unroll
                            for (int dd = 1; dd < DR; dd++) { df = fgc_readlane_f(qx[dd], q) - cx[dd]; dsq += df * df; }
                        } else {
                            dsq = INFINITY;
                            if (cand_ok) {
                                float df = sc[qbeg + q] - sc[j];
                                dsq = df * df;
                                for (int dd = 1; dd < Dn; dd++) {
                                    df = sc[(size_t)dd * ldc + qbeg + q] - sc[(size_t)dd * ldc + j];
                                    dsq += df * df;
                                }
                            }
                        }
                        push(q, dsq, j, dsq < t);
                    }
                }
            }
        }
        if (SQ) {
#pragma unroll
            for (int q = 0; q < QT; q++) cnt = (lane == q) ? sn[q] : cnt;
        }
    }

    // ---- per query: sort the pool by distance, write its first K entries as the row at the query's
    //      original position (slot 0 = the query itself) ----
    for (int q = 0; q < nq; q++) {
        const int self = qbeg + q;
        if (a.redo && !fgc_readlane_i((int)redo_q, q)) continue;
        const long long orig_q = (long long)a.order[self];
        // the sort below takes NSEG * 64 entries: a pool that fits is sorted as it is and its first K entries are
        // written, a larger one is first cut to exactly K
        if (a.any_order) {
            // Rows in pool order: cut the pool to exactly K, move the query itself to slot 0 (its entry trades places
            // with the one in slot 0) and write - no sort.  A pool without the query (direction flags, or more than K
            // points at distance 0) takes the sorting path below, which drops the farthest entry for it.
            if (fgc_readlane_i(cnt, q) > K) prune(q, true);
            const int c = fgc_readlane_i(cnt, q);
            int es = -1;                          // element that holds the query
            unsigned EX[NSEG], EY[NSEG];
#pragma unroll
            for (int s = 0; s < NSEG; s++) {
                const bool valid = (s * 64 + lane) < c;
                const uint2 e = valid ? pool[q * CAP + s * 64 + lane] : make_uint2(0x7f800000u, 0xffffffffu);
                EX[s] = e.x; EY[s] = e.y;
                const unsigned long long sm = fgc_ballot(valid && (int)e.y == self);
                if (sm) es = s * 64 + __ffsll((long long)sm) - 1;
            }
            if (es >= 0) {
#pragma unroll
                for (int s = 0; s < NSEG; s++) {
                    const int e = s * 64 + lane;
                    if (e < c) {
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
        if (fgc_readlane_i(cnt, q) > NSEG * 64) prune(q, true);
        const int c = fgc_readlane_i(cnt, q);     // entries in slots 0..c-1, c <= NSEG * 64
        float L[NSEG];
        int I[NSEG], rank[NSEG];
        bool valid[NSEG];
        bool has_self = false;
#pragma unroll
        for (int s = 0; s < NSEG; s++) {
            valid[s] = (s * 64 + lane) < c;
            const uint2 e = valid[s] ? pool[q * CAP + s * 64 + lane] : make_uint2(0x7f800000u, 0xffffffffu);
            L[s] = __uint_as_float(e.x);
            I[s] = (int)e.y;
            const bool is_self = valid[s] && I[s] == self;
            if (is_self) L[s] = -1.f;             // the query itself sorts first
            has_self = has_self || (fgc_ballot(is_self) != 0ull);
            rank[s] = 0;
        }
        // bitonic sort of the NSEG * 64 (distance, index) pairs, element e = s * 64 + lane; equal keys never swap.
        // Partners less than 64 apart sit in the same register of another lane, the others are two registers of
        // one lane.  The c finite keys end up in elements 0 .. c-1.
        FgcBitonic<2, 1, NSEG>::run(L, I);
#pragma unroll
        for (int s = 0; s < NSEG; s++) { valid[s] = (s * 64 + lane) < c; rank[s] = s * 64 + lane; }
        const int shift = has_self ? 0 : 1;       // without the query in the pool its slot 0 is added here
        const int n_out = min(c + shift, K);
#pragma unroll
        for (int s = 0; s < NSEG; s++) {
            const int slot = rank[s] + shift;
            if (valid[s] && slot < K) {
                const bool is_self = I[s] == self;
                a.out_idx[orig_q * K + slot] = is_self ? orig_q : (long long)a.order[I[s]];
                a.out_dist[orig_q * K + slot] = is_self ? 0.f : L[s];
                if (a.out_sorted) a.out_sorted[(long long)self * K + slot] = I[s];
            }
            const int pslot = s * 64 + lane;      // padding slots and, if needed, the query's own slot 0
            if (pslot < K && pslot >= n_out) {
                a.out_idx[orig_q * K + pslot] = a.tf_compat ? orig_q : -1ll;
                a.out_dist[orig_q * K + pslot] = 0.f;
                if (a.out_sorted) a.out_sorted[(long long)self * K + pslot] = -1;
            }
            if (!has_self && pslot == 0) {
                a.out_idx[orig_q * K] = orig_q;
                a.out_dist[orig_q * K] = 0.f;
                if (a.out_sorted) a.out_sorted[(long long)self * K] = self;
            }
        }
    }
#ifdef FGC_KNN_STATS
    if (a.stats && lane == 0) {
#ifdef FGC_KNN_COUNTERS
        atomicAdd(&a.stats[3], (unsigned long long)n_cullq); atomicAdd(&a.stats[4], (unsigned long long)n_app);
        atomicAdd(&a.stats[5], (unsigned long long)n_span); atomicAdd(&a.stats[6], (unsigned long long)n_bis);
        atomicAdd(&a.stats[7], (unsigned long long)n_bisx);
#endif
        atomicAdd(&a.stats[0], nev);
        atomicAdd(&a.stats[1], (unsigned long long)nchunks);
        atomicAdd(&a.stats[2], (unsigned long long)nprunes);
    }
#endif
}

template <int DT, int NSEG, int RD, int QT = QT_DEFAULT> static int launch_knn_t(const KnnArgs &a, hipStream_t s)
{
    constexpr int WPB = KnnCfg<NSEG>::WPB;
    const int tiles = (int)fgc_cdiv(a.n, QT);
    const int blocks = (int)fgc_cdiv(tiles, WPB);
    const size_t lds = (size_t)WPB * 2 * QT * a.pool_cap * sizeof(float);
    hipLaunchKernelGGL((k_knn<DT, NSEG, RD, QT>), dim3(blocks), dim3(WPB * 64), lds, s, a);
    FGC_LAUNCH_CHECK();
    return FGC_OK;
}

// Kernels with the coordinates in registers are built for the combinations of coordinate count and binned dimensions
// that the two grid rules produce (the library's own grid bins min(D, 5) dimensions, the reference's rule 3 - or 2
// for D = 2); any other combination (a caller's max_bin_dims) runs the variant that reads coordinates from memory.
// up to four coordinates and 64 neighbours: small inputs get wavefronts of QT_SMALL queries
template <int DT, int NSEG, int RD> static int launch_knn_q(const KnnArgs &a, hipStream_t s)
{
    if constexpr (NSEG == 1) {
        if (a.n <= KNN_SMALL_N) return launch_knn_t<DT, NSEG, RD, QT_SMALL>(a, s);
    }
    return launch_knn_t<DT, NSEG, RD>(a, s);
}

template <int NSEG, int RD> static int launch_knn_d(const KnnArgs &a, hipStream_t s)
{
    constexpr bool wide = RD == 2 || RD == 4;      // 3 or 5 binned dimensions
    switch (a.D) {
    case 2: if constexpr (RD == 1) return launch_knn_q<2, NSEG, RD>(a, s); break;
    case 3: if constexpr (RD == 2) return launch_knn_q<3, NSEG, RD>(a, s); break;
    case 4: if constexpr (RD == 2 || RD == 3) return launch_knn_q<4, NSEG, RD>(a, s); break;
    case 5: if constexpr (wide) return launch_knn_t<5, NSEG, RD>(a, s); break;
    case 6: if constexpr (wide) return launch_knn_t<6, NSEG, RD>(a, s); break;
    case 7: if constexpr (wide) return launch_knn_t<7, NSEG, RD>(a, s); break;
    case 8: if constexpr (wide) return launch_knn_t<8, NSEG, RD>(a, s); break;
    default: break;
    }
    // more coordinates: padded up to 12 or 16 registers per point (the padding contributes exact zeros),
    // beyond that read from memory per evaluation
    if constexpr (wide) {
        if (a.D > 8 && a.D <= 12) return launch_knn_t<12, NSEG, RD>(a, s);
        if (a.D > 12 && a.D <= 16) return launch_knn_t<16, NSEG, RD>(a, s);
    }
    return launch_knn_t<0, NSEG, RD>(a, s);
}

template <int NSEG> static int launch_knn_r(const KnnArgs &a, hipStream_t s)
{
    if (a.nbd <= 2) return launch_knn_d<NSEG, 1>(a, s);
    if (a.nbd == 3) return launch_knn_d<NSEG, 2>(a, s);
    if (a.nbd == 4) return launch_knn_d<NSEG, 3>(a, s);
    return launch_knn_d<NSEG, 4>(a, s);
}

template <int NSEG> static int launch_knn_big(const KnnArgs &a, hipStream_t s)
{
    if (a.nbd <= 2) return launch_knn_t<0, NSEG, 1>(a, s);
    if (a.nbd == 3) return launch_knn_t<0, NSEG, 2>(a, s);
    if (a.nbd == 4) return launch_knn_t<0, NSEG, 3>(a, s);
    return launch_knn_t<0, NSEG, 4>(a, s);
}

int fgc_launch_knn(const KnnArgs &a_in, hipStream_t s)
{
    KnnArgs a = a_in;
    if (a.n <= 0) return FGC_OK;
    if (a.K < 1 || a.K > FGC_MAX_K || a.D < 1 || a.nbd < 1 || a.nbd > FGC_MAX_BIN_DIMS || a.nbd > a.D)
        return FGC_EINVAL;
    // K kept + room for new candidates: a whole chunk for K <= 64, where LDS is not yet what limits the number
    // of resident wavefronts, less beyond; always <= 64 * (ceil(K / 64) + 1)
    a.pool_cap = ((a.K + (a.K <= 64 ? POOL_EXTRA_SMALL_K : POOL_EXTRA) + 15) / 16) * 16;
    if (a.K <= 64) return launch_knn_r<1>(a, s);
    if (a.K <= 128) return launch_knn_r<2>(a, s);
    if (a.K <= 256) return launch_knn_r<4>(a, s);
    // Beyond 256 neighbours (rare: the reference's benchmarks stop at 100) only the variant that reads the
    // coordinates from memory per evaluation is built, with pools of up to 1072 entries per query.
    if (a.K <= 512) return launch_knn_big<8>(a, s);
    return launch_knn_big<16>(a, s);
}
