/*
 * CPU restatement of the graph-building path of jkiesele/FastGraphCompute.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker the HIP kernels are
 * compared against and the "port" CPU baseline that the benchmark times.  It
 * is never linked into, imported by, or used as a fallback for the product
 * library; only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline
 * leg may call it.
 *
 * Every function states which part of the reference it follows
 * (paths relative to the reference checkout, fastgraphcompute/extensions/).
 * The arithmetic (operation order, float widths, comparison strictness) is
 * kept identical to the reference's CPU kernels so that bin indices are
 * bit-exact and the number of distance evaluations (C_eval) is the same
 * deterministic function of the input.
 *
 * Build: gcc -O2 -std=c11 -ffp-contract=off -fopenmp -shared -fPIC (see
 * oracle/build_oracle.py).  -ffp-contract=off keeps every float operation a
 * single IEEE-754 binary32 operation, as in the reference's x86-64 -O2 build.
 *
 * Pinning status of each function is listed in oracle/oracle.py's header.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define FGC_MAX_BIN_DIMS 5

/* ------------------------------------------------------------------ */
/* Binning kernel.  Follows `calc`, bin_by_coordinates_cpu.cpp:7-99.
 * coords are the already min-normalised [n_vert, n_dims] floats; the bin of a
 * coordinate is floorf(x / bw + 1e-3f), clamped into [0, n_bins-1]; the flat
 * index is row-major with coordinate 0 most significant, plus
 * event * prod(n_bins).  Returns the number of clamped coordinates (the
 * reference prints a warning for each instead). */
int64_t fgc_oracle_bin_points(const float *coords, const int64_t *row_splits,
                              float bin_width, const int64_t *n_bins,
                              int64_t *assigned, int64_t *flat,
                              int64_t *n_per_bin, int64_t n_vert,
                              int64_t n_dims, int64_t n_rs,
                              int64_t n_total_bins, int calc_n_per_bin)
{
    int64_t clamped = 0;
    const float eps = 1e-3f;
    for (int64_t v = 0; v < n_vert; v++) {
        int64_t stride = 1, f = 0;
        for (int64_t c = n_dims - 1; c >= 0; c--) {
            float q = coords[v * n_dims + c] / bin_width;
            int64_t b = (int64_t)floorf(q + eps);
            if (b < 0) { b = 0; clamped++; }
            else if (b >= n_bins[c]) { b = n_bins[c] - 1; clamped++; }
            assigned[v * (n_dims + 1) + c + 1] = b;
            f += b * stride;
            stride *= n_bins[c];
        }
        int64_t ev = 0;
        for (int64_t r = 1; r < n_rs; r++) {
            if (row_splits[r] > v) break;
            ev++;
        }
        f += ev * stride;
        if (f >= n_total_bins) continue;   /* reference skips the point */
        assigned[v * (n_dims + 1)] = ev;
        flat[v] = f;
        if (calc_n_per_bin) n_per_bin[f] += 1;
    }
    return clamped;
}

/* ------------------------------------------------------------------ */
/* Shell enumeration.  Follows binstepper<N,T>, binstepper.h:22-106: all cells
 * of the (2d+1)^n cube around `centre` in lexicographic order (dimension 0
 * slowest), keeping those with Chebyshev offset exactly d that lie inside the
 * grid; yields the row-major flat bin (dimension n-1 fastest). */
typedef struct {
    int n;
    int64_t d;
    int64_t off[FGC_MAX_BIN_DIMS];      /* current offset in [-d, d] */
    int64_t centre[FGC_MAX_BIN_DIMS];
    int64_t nb[FGC_MAX_BIN_DIMS];
    int started, finished;
} shell_iter;

static void shell_begin(shell_iter *s, int n, const int64_t *nb,
                        const int64_t *centre, int64_t d)
{
    s->n = n; s->d = d; s->started = 0; s->finished = 0;
    for (int i = 0; i < n; i++) {
        s->nb[i] = nb[i]; s->centre[i] = centre[i]; s->off[i] = -d;
    }
}

/* next in-grid surface cell of the current shell, or -1 */
static int64_t shell_next(shell_iter *s)
{
    for (;;) {
        if (s->finished) return -1;
        if (s->started) {
            int i = s->n - 1;
            while (i >= 0) {
                if (s->off[i] < s->d) { s->off[i]++; break; }
                s->off[i] = -s->d; i--;
            }
            if (i < 0) { s->finished = 1; return -1; }
        }
        s->started = 1;
        int surface = 0, inside = 1;
        int64_t f = 0;
        for (int i = 0; i < s->n; i++) {
            int64_t o = s->off[i];
            if (o == s->d || o == -s->d) surface = 1;
            int64_t g = s->centre[i] + o;
            if (g < 0 || g >= s->nb[i]) inside = 0;
            f = f * s->nb[i] + g;
        }
        if (surface && inside) return f;
    }
}

/* ------------------------------------------------------------------ */
/* One query of the shell search.  Follows select_knn_kernel_cpu,
 * binned_select_knn_cpu.cpp:56-208 (distance :10-19, max rescan :22-37).
 * Works in bin-sorted space.  Returns the number of distance evaluations. */
static int64_t knn_one_query(int64_t i, const float *coord,
                             const int64_t *bin_idx, const int64_t *direction,
                             const int64_t *dim_bin_idx,
                             const int64_t *bin_boundaries,
                             const int64_t *n_bins, float bw, int64_t *out_idx,
                             float *out_dist, int64_t n_vert, int64_t K,
                             int64_t n_coords, int n_bin_dims,
                             int64_t n_bboundaries, int use_direction,
                             int64_t *d_stop)
{
    int64_t evals = 0;
    if (use_direction && (direction[i] == 0 || direction[i] == 2)) {
        if (d_stop) *d_stop = -1;
        return 0;
    }
    int64_t cells = 1;
    for (int b = 0; b < n_bin_dims; b++) cells *= n_bins[b];
    const int64_t event_off = cells * (bin_idx[i] / cells);

    int64_t *row_i = out_idx + i * K;
    float *row_d = out_dist + i * K;
    int64_t filled = 1, max_slot = 0;
    float max_d = 0.f;
    const float *xi = coord + i * n_coords;

    shell_iter it;
    int64_t d = 0;
    for (;; d++) {
        shell_begin(&it, n_bin_dims, n_bins,
                    dim_bin_idx + i * (n_bin_dims + 1) + 1, d);
        int any_cell = 0;
        for (;;) {
            int64_t cell = shell_next(&it);
            if (cell < 0) break;
            cell += event_off;
            if (cell < 0 || cell + 1 >= n_bboundaries) continue;
            any_cell = 1;   /* empty bins count as "shell exists" too */
            int64_t lo = bin_boundaries[cell], hi = bin_boundaries[cell + 1];
            if (lo == hi) continue;
            if (lo >= n_vert || hi > n_vert) continue;
            for (int64_t j = lo; j < hi; j++) {
                if (j == i) continue;
                if (use_direction && (direction[j] == 1 || direction[j] == 2))
                    continue;
                const float *xj = coord + j * n_coords;
                float dsq = 0.f;
                for (int64_t c = 0; c < n_coords; c++) {
                    float t = xi[c] - xj[c];
                    dsq += t * t;
                }
                evals++;
                if (filled < K) {
                    row_i[filled] = j; row_d[filled] = dsq;
                    if (dsq > max_d) { max_d = dsq; max_slot = filled; }
                    filled++;
                } else if (dsq < max_d) {
                    row_i[max_slot] = j; row_d[max_slot] = dsq;
                    max_d = 0.f; max_slot = 0;
                    for (int64_t s = 1; s < K; s++)
                        if (row_d[s] > max_d) { max_d = row_d[s]; max_slot = s; }
                }
            }
        }
        if (!any_cell) break;
        /* same expression, same association as the reference's stop test */
        float fd = (float)d;
        if (filled == K && bw * fd * bw * fd > max_d) break;
    }
    if (d_stop) *d_stop = d;
    return evals;
}

/* Whole kNN kernel over bin-sorted inputs: defaults as setDefaults
 * (binned_select_knn_cpu.cpp:40-53), then every query.  n_threads == 1 is the
 * reference's serial loop; n_threads > 1 splits queries over OpenMP threads
 * (queries are independent, results are identical).  Returns C_eval, the total
 * number of distance evaluations; d_stop (optional, [n_vert]) receives the
 * last shell radius visited per query.  query_stride > 1 evaluates only every
 * query_stride-th query starting at query_offset (bounded-sample timing). */
int64_t fgc_oracle_knn_sorted(const float *coord, const int64_t *bin_idx,
                              const int64_t *direction,
                              const int64_t *dim_bin_idx,
                              const int64_t *bin_boundaries,
                              const int64_t *n_bins, const float *bin_width,
                              int64_t *out_idx, float *out_dist,
                              int64_t n_vert, int64_t K, int64_t n_coords,
                              int64_t n_bin_dims, int64_t n_bboundaries,
                              int tf_compat, int use_direction,
                              int64_t *d_stop, int n_threads,
                              int64_t query_stride, int64_t query_offset)
{
    if (n_bin_dims < 2 || n_bin_dims > FGC_MAX_BIN_DIMS) return -1;
    if (query_stride < 1) query_stride = 1;
    for (int64_t v = 0; v < n_vert; v++)
        for (int64_t k = 0; k < K; k++) {
            out_idx[v * K + k] = (k == 0) ? v : (tf_compat ? v : -1);
            out_dist[v * K + k] = 0.f;
        }
    int64_t total = 0;
    const float bw = bin_width[0];
    int64_t n_q = (n_vert - query_offset + query_stride - 1) / query_stride;
    if (n_vert <= query_offset) n_q = 0;
#ifdef _OPENMP
    if (n_threads < 1) n_threads = 1;
#pragma omp parallel for schedule(dynamic, 64) num_threads(n_threads) reduction(+ : total)
#endif
    for (int64_t q = 0; q < n_q; q++) {
        int64_t i = query_offset + q * query_stride;
        total += knn_one_query(i, coord, bin_idx, direction, dim_bin_idx,
                               bin_boundaries, n_bins, bw, out_idx, out_dist,
                               n_vert, K, n_coords, (int)n_bin_dims,
                               n_bboundaries, use_direction,
                               d_stop ? d_stop + i : NULL);
    }
    return total;
}

/* ------------------------------------------------------------------ */
/* Follows index_replacer_cpu_kernel, index_replacer_cpu.cpp:7-26, except that
 * an index >= n_repl is passed through instead of reading repl[i] (an
 * out-of-range read in the reference that the kNN path never reaches). */
void fgc_oracle_index_replacer(const int64_t *in, const int64_t *repl,
                               int64_t *out, int64_t n, int64_t n_repl)
{
    for (int64_t i = 0; i < n; i++) {
        int64_t r = in[i];
        out[i] = (r < 0 || r >= n_repl) ? r : repl[r];
    }
}

/* ------------------------------------------------------------------ */
/* Gradient of distsq wrt coordinates.  Follows
 * select_knn_grad_selfloop_kernel / _neighloop_kernel,
 * binned_select_knn_grad_cpu.cpp:6-47,50-93: the products are formed in
 * double (the reference's `2.` literal) and rounded to float when they are
 * accumulated; the self loop runs first over all points, then the neighbour
 * loop adds in (i, coordinate, k) order. */
void fgc_oracle_knn_grad(const float *grad_dist, const int64_t *idx,
                         const float *coord, float *grad_coord, int64_t n_vert,
                         int64_t K, int64_t n_coords)
{
    for (int64_t i = 0; i < n_vert; i++)
        for (int64_t c = 0; c < n_coords; c++) {
            const float xi = coord[i * n_coords + c];
            float acc = 0.f;
            for (int64_t k = 0; k < K; k++) {
                int64_t m = idx[i * K + k];
                if (m < 0 || m >= n_vert) continue;
                const float g = grad_dist[i * K + k];
                const float xm = coord[m * n_coords + c];
                acc -= 2. * g * (xm - xi);
            }
            grad_coord[i * n_coords + c] = acc;
        }
    for (int64_t i = 0; i < n_vert; i++)
        for (int64_t c = 0; c < n_coords; c++) {
            const float xi = coord[i * n_coords + c];
            for (int64_t k = 0; k < K; k++) {
                int64_t m = idx[i * K + k];
                if (m < 0 || m >= n_vert) continue;
                const float g = grad_dist[i * K + k];
                const float xm = coord[m * n_coords + c];
                float add = 2. * g * (xm - xi);
                grad_coord[m * n_coords + c] += add;
            }
        }
}

/* ------------------------------------------------------------------ */
/* GravNet neighbour aggregation, forward.  Follows gnn_ops.py:90-102 with
 * select_with_default (oc_helper.py:232-271): w = exp(-10 d^2); gathered
 * feature times w (slots with idx -1 contribute 0); mean over all K slots and
 * max over all K slots (first maximal slot recorded in argmax).  float
 * accumulation in slot order. */
void fgc_oracle_gravnet_agg_fwd(const int64_t *idx, const float *distsq,
                                const float *feat, float *fmean, float *fmax,
                                int64_t *argmax, int64_t n_vert, int64_t K,
                                int64_t P)
{
    for (int64_t i = 0; i < n_vert; i++)
        for (int64_t p = 0; p < P; p++) {
            float s = 0.f, mx = 0.f;
            int64_t am = -1;
            for (int64_t k = 0; k < K; k++) {
                int64_t m = idx[i * K + k];
                float w = expf(-10.f * distsq[i * K + k]);
                float v = (m == -1 ? 0.f : feat[m * P + p]) * w;
                s += v;
                if (k == 0 || v > mx) { mx = v; am = k; }
            }
            fmean[i * P + p] = s / (float)K;
            fmax[i * P + p] = mx;
            if (argmax) argmax[i * P + p] = am;
        }
}

/* Brute-force exact kNN inside each event (the mathematical definition the
 * shell search must reproduce).  Used only to pin fgc_oracle_knn_sorted on
 * small inputs.  Rows are written sorted by (distance, index). */
void fgc_oracle_knn_brute(const float *coord, const int64_t *row_splits,
                          int64_t n_rs, int64_t K, int64_t n_coords,
                          int64_t *out_idx, float *out_dist)
{
    for (int64_t e = 0; e + 1 < n_rs; e++) {
        int64_t lo = row_splits[e], hi = row_splits[e + 1];
        for (int64_t i = lo; i < hi; i++) {
            int64_t *ri = out_idx + i * K;
            float *rd = out_dist + i * K;
            int64_t n = 0;
            for (int64_t j = lo; j < hi; j++) {
                float dsq = 0.f;
                if (j != i)
                    for (int64_t c = 0; c < n_coords; c++) {
                        float t = coord[i * n_coords + c] - coord[j * n_coords + c];
                        dsq += t * t;
                    }
                /* self sorts first: give it distance -1 while inserting */
                float key = (j == i) ? -1.f : dsq;
                int64_t pos = n;
                while (pos > 0) {
                    float pk = (ri[pos - 1] == i) ? -1.f : rd[pos - 1];
                    if (pk <= key) break;
                    pos--;
                }
                if (pos >= K) continue;
                int64_t last = (n < K) ? n : K - 1;
                for (int64_t s = last; s > pos; s--) { ri[s] = ri[s - 1]; rd[s] = rd[s - 1]; }
                ri[pos] = j; rd[pos] = dsq;
                if (n < K) n++;
            }
            for (int64_t s = n; s < K; s++) { ri[s] = -1; rd[s] = 0.f; }
        }
    }
}

/* Object/vertex index matrices of the object-condensation helper
 * (calc_m, oc_helper_cpu.cpp:17-82).  For object k = (unique_idx[k], row split
 * unique_rs_asso[k]): M[k, :] lists, in ascending order, the vertices of that
 * row split whose association index equals unique_idx[k]; M_not[k, :] those
 * whose index differs; both padded with -1.  The reference fills transposed
 * buffers and transposes afterwards (oc_helper_cpu.cpp:150-151); the result is
 * the row-major [n_unique, n_max*] layout written here directly.  A row that
 * would overflow its width is cut at the width (the reference warns and stops
 * one element later, outside the buffer).  Returns the number of cut rows. */
int64_t fgc_oracle_oc_calc_m(const int64_t *asso_idx, const int64_t *unique_idx,
                             const int64_t *unique_rs_asso, const int64_t *rs,
                             int64_t *M, int64_t *M_not, int64_t n_vert, int64_t n_unique,
                             int64_t n_maxuq, int64_t n_maxrs, int calc_m_not)
{
    int64_t cut = 0;
    for (int64_t k = 0; k < n_unique; k++) {
        int64_t uq = unique_idx[k];
        int64_t r = unique_rs_asso[k];
        int64_t lo = rs[r], hi = rs[r + 1];
        if (hi > n_vert) hi = n_vert;
        int64_t fill = 0;
        for (int64_t v = lo; v < hi; v++)
            if (asso_idx[v] == uq) {
                if (fill >= n_maxuq) { cut++; break; }
                M[k * n_maxuq + fill++] = v;
            }
        for (; fill < n_maxuq; fill++) M[k * n_maxuq + fill] = -1;
        if (!calc_m_not) continue;
        fill = 0;
        for (int64_t v = lo; v < hi; v++)
            if (asso_idx[v] != uq) {
                if (fill >= n_maxrs) { cut++; break; }
                M_not[k * n_maxrs + fill++] = v;
            }
        for (; fill < n_maxrs; fill++) M_not[k * n_maxrs + fill] = -1;
    }
    return cut;
}

/* Brute-force kNN with a radius limit (select_knn_kernel, select_knn_cpu.cpp:68-126, with set_defaults
 * :49-66 and the radius handling of select_knn_cpu :174-176): per event, slot 0 = the point itself, then up to
 * K-1 (or event size - 1) other points of the event with distsq <= r2 (any when r2 <= 0): slots fill in index
 * order, afterwards a candidate strictly closer than the current largest entry replaces it.  Distances are
 * sequential float sums. */
void fgc_oracle_select_knn(const float *coord, const int64_t *row_splits, int64_t *idx, float *dist,
                           int64_t n_vert, int64_t K, int64_t n_coords, int64_t n_rs, double max_radius)
{
    if (max_radius > 0) max_radius *= max_radius;
    const float r2 = (float)max_radius;
    for (int64_t i = 0; i < n_vert; i++)
        for (int64_t k = 0; k < K; k++) { idx[i * K + k] = k ? -1 : i; dist[i * K + k] = 0.f; }
    for (int64_t e = 0; e + 1 < n_rs; e++) {
        const int64_t lo = row_splits[e], hi = row_splits[e + 1];
        for (int64_t i = lo; i < hi && i < n_vert; i++) {
            int64_t maxn = K < hi - lo ? K : hi - lo;
            int64_t nfilled = 1, maxidx = 0;
            float maxd = 0.f;
            for (int64_t j = lo; j < hi; j++) {
                if (j == i) continue;
                float d = 0.f;
                for (int64_t c = 0; c < n_coords; c++) {
                    float t = coord[i * n_coords + c] - coord[j * n_coords + c];
                    d += t * t;
                }
                if (nfilled < maxn && (r2 <= 0 || r2 >= d)) {
                    idx[i * K + nfilled] = j; dist[i * K + nfilled] = d;
                    if (d > maxd) { maxd = d; maxidx = nfilled; }
                    nfilled++;
                    continue;
                }
                if (d < maxd) {
                    idx[i * K + maxidx] = j; dist[i * K + maxidx] = d;
                    maxd = 0.f; maxidx = 0;
                    for (int64_t n = 1; n < K; n++)
                        if (dist[i * K + n] > maxd) { maxd = dist[i * K + n]; maxidx = n; }
                }
            }
        }
    }
}

int fgc_oracle_max_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
