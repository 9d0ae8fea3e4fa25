/*
 * fgc_hip.h - C ABI of libfgc_hip.so, the MI355X (gfx950) implementation of
 * FastGraphCompute's graph-building path.
 *
 * Conventions
 *   - Every pointer named d_* is device memory on the current HIP device; the
 *     caller owns all of it, including the workspace.  The library allocates
 *     nothing and frees nothing.
 *   - `stream` is a hipStream_t passed as void*.  All work is enqueued on it
 *     and the call returns without synchronising; results are valid once the
 *     stream has reached that point.
 *   - Return value: 0 on success, a negative FGC_E* code for rejected
 *     arguments, a positive hipError_t for a failed launch.  No C++ exception
 *     crosses this boundary and the process is never exit()ed.
 *   - d_status (where present) is an int32[FGC_STATUS_WORDS] device array the
 *     kernels OR anomaly bits into (the reference printf()s from the kernel
 *     instead); the caller reads it whenever it synchronises anyway.
 *   - Citations name the reference interface each entry point replaces, as
 *     fastgraphcompute/extensions/<file>:<line>.
 */
#ifndef FGC_HIP_H_
#define FGC_HIP_H_

#include <stdint.h>
#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FGC_OK 0
#define FGC_EINVAL (-1)      /* bad shape / unsupported size                  */
#define FGC_ENOSPACE (-2)    /* workspace too small                           */
#define FGC_EUNSUPPORTED (-3)/* e.g. number of binned dims outside 1..5       */
#define FGC_ETOOLARGE (-4)   /* input exceeds the fixed scratch of a no-allocation entry point */
#define FGC_ESHAPE (-5)      /* a shape outside what a specialised entry point handles (its comment says which
                                general entry point takes every shape)          */

#define FGC_MAX_BIN_DIMS 5
#define FGC_MAX_K 1024       /* neighbours per query the kNN kernels support; the reference's loops take any
                                K (binned_select_knn_cpu.cpp:211-326), its benchmarks stop at 100.  Up to 256
                                the search runs its register-tiled kernels, beyond that a slower variant  */
#define FGC_MAX_VERTICES ((1ll << 31) - 65) /* points per call of the kNN entry points: sorted positions are 32-bit
                                (FGC_EINVAL beyond); the reference indexes with int64 but its [N, K] int64 output
                                alone is 1 TB at K = 64 there */
/* bits of the kNN entry points' tf_compat argument */
#define FGC_KNN_TF_COMPAT 1  /* padding slots name the query itself instead of -1 (binned_select_knn.py:7-9) */
#define FGC_KNN_ANY_ORDER 2  /* slots 1.. of a row in any order instead of by increasing distance: the reference
                                promises no order either (its kernel replaces the farthest entry in place, its tests
                                sort every row before comparing, tests/test_binned_select_knn.py:90-91); saves the
                                per-query sort */
#define FGC_KNN_NO_MATRIX 4  /* keep the vector-unit search where the library would screen the candidates on the
                                matrix cores (5 to 8 coordinates, K <= 256, events of at most 65535 points and of a
                                size at which bounding boxes thin out little); same neighbours, for comparison runs */
#define FGC_KNN_FORCE_MATRIX 8 /* screen on the matrix cores wherever that search can run (5 to 8 coordinates, K <= 256,
                                events of at most 65535 points), whatever the event sizes; for comparison runs */

#define FGC_STATUS_WORDS 4
/* bits of d_status[0] */
#define FGC_ST_NONFINITE 1   /* a binned coordinate is inf/nan                */
#define FGC_ST_CLAMPED 2     /* a coordinate fell outside the grid (clamped)  */
#define FGC_ST_BAD_RANGE 4   /* range / bin width / n_bins not positive       */
#define FGC_ST_BAD_INDEX 8   /* neighbour index >= n_vert seen (gradient)     */
#define FGC_ST_OC_TRUNCATED 16 /* an object has more vertices than M is wide   */

/* Library version (major*100 + minor) and the text for a return code. */
int fgc_version(void);
const char *fgc_error_string(int code);

/* ---------------------------------------------------------------------------
 * Binning geometry.  Replaces the tensor preprocessing of bin_by_coordinates
 * (bin_by_coordinates.cpp:57-111, same arithmetic as bin_by_coordinates.py:
 * 40-92): global per-dimension minimum, range (+1 where zero, +1e-3), and
 * either the cubic bin width max_d(range_d / n_bins_d) from given n_bins
 * (mode 0) or n_bins_d = int(range_d / bin_width) + 1 from a given width
 * (mode 1).  All in single float32 operations.  Mode 2 is mode 0 with the
 * range padded by a factor 1.001 instead of +1e-3: the grid the kNN search
 * builds for itself (no counterpart in the reference; the neighbours found do
 * not depend on the grid).
 *
 *   d_coords     [n_vert, ld_coords] float32, first n_bin_dims columns binned
 *   d_geom       out, float32[FGC_GEOM_FLOATS]: min[5], bin_width, then the
 *                n_bins[5] as int32 bit patterns and a flags word
 *   n_bins_in    host array [n_bin_dims] (mode 0; mode 1 with given n_bins)
 *   bin_width_in used when mode == 1
 *   pre_normalized != 0: minimum taken as 0 (coordinates used as they are)
 *   d_ws         workspace of fgc_bin_geometry_workspace_bytes(n_vert) bytes
 */
#define FGC_GEOM_FLOATS 16
size_t fgc_bin_geometry_workspace_bytes(int64_t n_vert);
int fgc_bin_geometry_f32(const float *d_coords, int64_t n_vert, int32_t ld_coords,
                         int32_t n_bin_dims, int32_t mode, const int64_t *n_bins_in,
                         int32_t n_bins_given, float bin_width_in, int32_t pre_normalized,
                         float *d_geom, int32_t *d_status, void *d_ws, size_t ws_bytes,
                         void *stream);

/* ---------------------------------------------------------------------------
 * Per-point binning.  Replaces bin_by_coordinates_cuda_fn
 * (bin_by_coordinates_cuda_kernel.cu:119-172; CPU twin
 * bin_by_coordinates_cpu.cpp:7-99): bin of a coordinate =
 * floorf((x - min) / bin_width + 1e-3f) clamped to [0, n_bins-1]; flat index
 * row-major with dimension 0 most significant, plus event * prod(n_bins).
 *
 *   d_geom        as written by fgc_bin_geometry_f32
 *   d_row_splits  int64 [n_rs]
 *   d_assigned    out int64 [n_vert, n_bin_dims+1] (col 0 = event) or NULL
 *   d_flat        out int64 [n_vert] or NULL
 *   d_n_per_bin   out int64 [n_total_bins], must be zeroed by the caller, or NULL
 */
int fgc_bin_points_f32(const float *d_coords, int64_t n_vert, int32_t ld_coords,
                       int32_t n_bin_dims, const float *d_geom, const int64_t *d_row_splits,
                       int32_t n_rs, const int64_t *n_bins_host, int64_t *d_assigned,
                       int64_t *d_flat, int64_t *d_n_per_bin, int32_t *d_status, void *stream);

/* ---------------------------------------------------------------------------
 * Whole forward of binned_select_knn.  Replaces BinnedKNNAutograd::forward
 * (binned_knn_autograd_kernel.cpp:85-209), i.e. bin_by_coordinates on the
 * first n_bin_dims coordinates, the sort by flat bin, binned_select_knn_cuda_fn
 * (binned_select_knn_cuda_kernel.cu:252-384), index_replacer_cuda_fn and the
 * scatter back to the original order, in one call.
 *
 *   d_coords      [n_vert, n_coords] float32 row-major (original order)
 *   d_row_splits  int64 [n_rs] on the device; row_splits_host the same values
 *                 on the host (used to size the launch)
 *   n_bins        host array [n_bin_dims], bins per binned dimension; the caller
 *                 evaluates the reference's heuristic (calculate_optimal_bins,
 *                 :67-82) or passes the user's n_bins
 *   d_direction   int64 [n_vert] or NULL (0: only neighbour, 1: only query,
 *                 2: neither; binned_select_knn_cuda_kernel.cu:120-122,194-196)
 *   tf_compat     bit set of FGC_KNN_TF_COMPAT, FGC_KNN_ANY_ORDER, FGC_KNN_NO_MATRIX and FGC_KNN_FORCE_MATRIX (0 or 1 as before: rows
 *                 by distance)
 *   d_idx         out int64 [n_vert, K]: slot 0 the query itself, then its
 *                 K-1 nearest points of the same event by increasing distance
 *                 (in any order with FGC_KNN_ANY_ORDER), then -1 (or the
 *                 query's index with FGC_KNN_TF_COMPAT) where the event has
 *                 fewer than K points
 *   d_distsq      out float32 [n_vert, K], 0 for slot 0 and for padding
 *   d_stats       optional uint64[8] device counters, accumulated: [0] distance
 *                 evaluations, [1] candidate chunks visited, [2] pool prunes
 *                 ([3..7] only in debug builds with -DFGC_KNN_COUNTERS: box
 *                 tests, appends, spans, bisection steps; when the search ran
 *                 on the matrix cores: [3] queries it handed to the vector
 *                 search, [5] candidates it collected for the others, and
 *                 [0] counts screened pairs); NULL to skip.  A call
 *                 with d_stats runs a second build of the search kernels that carries
 *                 the counters and is slower (time a call without)
 */
size_t fgc_binned_select_knn_workspace_bytes(int64_t n_vert, int32_t n_coords,
                                             int32_t n_bin_dims, const int64_t *n_bins,
                                             int32_t n_rs, int32_t K);
int fgc_binned_select_knn_f32(const float *d_coords, int64_t n_vert, int32_t n_coords,
                              const int64_t *d_row_splits, const int64_t *row_splits_host,
                              int32_t n_rs, int32_t K, int32_t n_bin_dims, const int64_t *n_bins,
                              const int64_t *d_direction, int32_t tf_compat,
                              int64_t *d_idx, float *d_distsq, int32_t *d_status,
                              uint64_t *d_stats, void *d_ws, size_t ws_bytes, void *stream);

/* The whole forward without a workspace argument and without any allocation.
 * No counterpart in the reference (its forward allocates every intermediate
 * with torch::empty, binned_knn_autograd_kernel.cpp:118-139); it is for the
 * callers that cannot allocate device memory or size a workspace: code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
 * Same arguments and results as fgc_binned_select_knn_f32 (no d_stats); the
 * intermediates live in a fixed array of FGC_NOALLOC_SCRATCH_BYTES bytes that
 * is part of the library's device code, one copy per GPU, held until the
 * process ends.  The call allocates and frees nothing.
 *   - An input whose workspace (fgc_binned_select_knn_workspace_bytes) exceeds
 *     FGC_NOALLOC_SCRATCH_BYTES is rejected with FGC_ETOOLARGE (about one
 *     million points with three coordinates fit).
 *   - All calls on one GPU share that GPU's array: calls that overlap on one
 *     GPU (two streams, two host threads) race.  Calls on one stream are safe.
 *   - The current device at the call must be the one the pointers belong to.
 */
#define FGC_NOALLOC_SCRATCH_BYTES (32u << 20)
/* Optional, once per device with that device current: looks up the device address of the scratch array (a symbol
 * lookup, which may load the library's code object) so that the entry point itself does neither on its first call.
 * Call it before capturing fgc_binned_select_knn_noalloc_f32 into a HIP graph; without it the first call per device
 * does the lookup itself and must therefore happen outside a capture.  No counterpart in the reference. */
int fgc_noalloc_init(void);
int fgc_binned_select_knn_noalloc_f32(const float *d_coords, int64_t n_vert, int32_t n_coords,
                                      const int64_t *d_row_splits, const int64_t *row_splits_host,
                                      int32_t n_rs, int32_t K, int32_t n_bin_dims, const int64_t *n_bins,
                                      const int64_t *d_direction, int32_t tf_compat,
                                      int64_t *d_idx, float *d_distsq, int32_t *d_status, void *stream);

/* The same forward in two stages sharing one workspace, for callers that
 * search one prepared point set more than once or time the stages apart:
 * prepare = geometry + binning + sort + bin boundaries + sorted coordinate
 * copy (binned_knn_autograd_kernel.cpp:100-139); search = the neighbour
 * search with the un-sort fused (:157-195).  Both take the same shape
 * arguments; the workspace must not be touched in between.  d_nbr_sorted
 * (optional, int32 [n_vert, K]) receives the neighbour rows once more in the
 * search's own sorted order - row r belongs to the r-th point of that order and
 * holds positions in it, -1 padding - which is the layout
 * fgc_binned_select_knn_grad_sorted_f32 reads. */
int fgc_binned_knn_prepare_f32(const float *d_coords, int64_t n_vert, int32_t n_coords,
                               const int64_t *d_row_splits, const int64_t *row_splits_host,
                               int32_t n_rs, int32_t K, int32_t n_bin_dims, const int64_t *n_bins,
                               const int64_t *d_direction, int32_t *d_status, void *d_ws,
                               size_t ws_bytes, void *stream);
/* fgc_binned_knn_prepare_f32 for coordinates that are the first n_coords columns of a wider row-major matrix
 * (ld_coords floats per row), e.g. the learned coordinates inside the joint projection of a GravNet layer
 * (gnn_ops.py:79-87 computes them as a matrix of their own). */
int fgc_binned_knn_prepare_ld_f32(const float *d_coords, int64_t n_vert, int32_t n_coords, int32_t ld_coords,
                                  const int64_t *d_row_splits, const int64_t *row_splits_host, int32_t n_rs,
                                  int32_t K, int32_t n_bin_dims, const int64_t *n_bins,
                                  const int64_t *d_direction, int32_t *d_status, void *d_ws, size_t ws_bytes,
                                  void *stream);
int fgc_binned_knn_search_f32(int64_t n_vert, int32_t n_coords, const int64_t *row_splits_host,
                              int32_t n_rs, int32_t K, int32_t n_bin_dims, const int64_t *n_bins,
                              int32_t with_direction, int32_t tf_compat, int64_t *d_idx,
                              float *d_distsq, int32_t *d_nbr_sorted, uint64_t *d_stats, void *d_ws,
                              size_t ws_bytes, void *stream);

/* ---------------------------------------------------------------------------
 * k nearest neighbours inside a radius.  Replaces select_knn_cuda_fn
 * (select_knn_cuda_kernel.cu:136-212; CPU twin select_knn_cpu.cpp:68-205), the
 * reference's brute-force search per event: slot 0 the query itself, then its
 * at most K-1 nearest points of the same event whose squared distance is
 * <= (float)(max_radius * max_radius), by increasing distance, -1 / 0 padding.
 * max_radius <= 0 means no limit.  The reference's mask / mask_mode arguments
 * are read by neither of its implementations and have no counterpart here.
 * Runs the binned search of fgc_binned_select_knn_f32 with the radius as the
 * initial bound; workspace and grid arguments as there.
 */
int fgc_select_knn_f32(const float *d_coords, int64_t n_vert, int32_t n_coords,
                       const int64_t *d_row_splits, const int64_t *row_splits_host, int32_t n_rs,
                       int32_t K, double max_radius, int32_t n_bin_dims, const int64_t *n_bins,
                       int64_t *d_idx, float *d_distsq, int32_t *d_status, void *d_ws, size_t ws_bytes,
                       void *stream);

/* ---------------------------------------------------------------------------
 * Replaces index_replacer_cuda_fn (index_replacer_cuda_kernel.cu:30-59):
 * out[i] = in[i] if in[i] < 0 or in[i] >= n_repl, else repl[in[i]].
 */
int fgc_index_replacer_i64(const int64_t *d_in, const int64_t *d_repl, int64_t *d_out,
                           int64_t n, int64_t n_repl, void *stream);

/* ---------------------------------------------------------------------------
 * Replaces binned_select_knn_grad_cuda_fn
 * (binned_select_knn_grad_cuda_kernel.cu:90-164; CPU twin
 * binned_select_knn_grad_cpu.cpp:96-165):
 *   g[i,c]      = -2 sum_k gd[i,k] (x[n_ik,c] - x[i,c])
 *   g[n_ik,c]  +=  2 gd[i,k] (x[n_ik,c] - x[i,c])          (n_ik < 0 skipped)
 * d_grad_coords [n_vert, n_coords] is fully overwritten.
 * d_order (optional, int32 [n_vert]): a permutation of the points in which
 * consecutive entries are spatial neighbours (the bin-sorted order of the
 * forward, see fgc_binned_knn_export_order_i32).  It only changes the order in
 * which queries are processed, so that contributions to the same point are
 * combined on chip before they reach memory; NULL = original order.
 */
int fgc_binned_select_knn_grad_f32(const float *d_grad_distsq, const int64_t *d_idx,
                                   const float *d_coords, float *d_grad_coords,
                                   int64_t n_vert, int32_t K, int32_t n_coords,
                                   const int32_t *d_order, int32_t *d_status, void *stream);

/* Copies the bin-sorted order (sorted position -> original row) out of a
 * workspace that fgc_binned_knn_prepare_f32 / fgc_binned_select_knn_f32 filled
 * with the same shape arguments.  No counterpart in the reference (its sort
 * order, binned_knn_autograd_kernel.cpp:118-120, never leaves the forward). */
int fgc_binned_knn_export_order_i32(int64_t n_vert, int32_t n_coords, const int64_t *row_splits_host,
                                    int32_t n_rs, int32_t K, int32_t n_bin_dims, const int64_t *n_bins,
                                    int32_t with_direction, const void *d_ws, size_t ws_bytes,
                                    int32_t *d_order_out, void *stream);

/* The same gradient from the neighbour rows in the search's sorted order (d_nbr_sorted as written by
 * fgc_binned_knn_search_f32, d_order as exported by fgc_binned_knn_export_order_i32): neighbours are then memory
 * neighbours, which is what makes the coordinate gathers cheap.  d_grad_distsq, d_coords and d_grad_coords stay
 * in the original order.  d_ws: fgc_binned_select_knn_grad_sorted_workspace_bytes(n_vert, n_coords) bytes. */
size_t fgc_binned_select_knn_grad_sorted_workspace_bytes(int64_t n_vert, int32_t n_coords);
int fgc_binned_select_knn_grad_sorted_f32(const float *d_grad_distsq, const int32_t *d_nbr_sorted,
                                          const float *d_coords, const int32_t *d_order, float *d_grad_coords,
                                          int64_t n_vert, int32_t K, int32_t n_coords, int32_t *d_status,
                                          void *d_ws, size_t ws_bytes, void *stream);

/* The same with leading dimensions: d_coords and d_grad_coords are the first n_coords columns of row-major
 * matrices with ld_coords / ld_grad_coords floats per row (the other columns of d_grad_coords are not touched). */
int fgc_binned_select_knn_grad_sorted_ld_f32(const float *d_grad_distsq, const int32_t *d_nbr_sorted,
                                             const float *d_coords, int32_t ld_coords, const int32_t *d_order,
                                             float *d_grad_coords, int32_t ld_grad_coords, int64_t n_vert,
                                             int32_t K, int32_t n_coords, int32_t *d_status, void *d_ws,
                                             size_t ws_bytes, void *stream);

/* ---------------------------------------------------------------------------
 * Replaces select_with_default (oc_helper.py:232-271) for float32 features:
 * out[v,k,:] = feat[idx[v,k],:], or default_value where idx[v,k] == -1.
 */
int fgc_select_with_default_f32(const int64_t *d_idx, const float *d_feat, float *d_out,
                                int64_t n_vert, int32_t K, int32_t n_feat, int64_t n_feat_rows,
                                float default_value, void *stream);
/* The same for 8-byte elements (int64 or float64 features, as the object-condensation loss selects point
 * indices and per-event counts, object_condensation.py:148,312); default_bits is the default value's bit
 * pattern in the element type. */
int fgc_select_with_default_b64(const int64_t *d_idx, const void *d_feat, void *d_out, int64_t n_vert,
                                int32_t K, int32_t n_feat, int64_t n_feat_rows, uint64_t default_bits,
                                void *stream);

/* ---------------------------------------------------------------------------
 * GravNet neighbour aggregation, fused.  Replaces the tensor ops of
 * GravNetOp.forward, gnn_ops.py:90-102 (exp(-10 d^2) weights, gather with
 * default 0, multiply, mean and max over the K slots) without materialising the
 * [n_vert, K, P] tensor.
 *   d_fmean, d_fmax  out float32 [n_vert, P]
 *   d_argmax         out int32 [n_vert, P]: slot of the (first) maximum
 * Backward: given d(loss)/d(fmean), d(loss)/d(fmax) it accumulates
 *   d_grad_feat   [n_feat_rows, P], must be zeroed by the caller
 *   d_grad_distsq [n_vert, K], fully overwritten
 */
int fgc_gravnet_aggregate_fwd_f32(const int64_t *d_idx, const float *d_distsq,
                                  const float *d_feat, float *d_fmean, float *d_fmax,
                                  int32_t *d_argmax, int64_t n_vert, int32_t K, int32_t P,
                                  void *stream);
int fgc_gravnet_aggregate_bwd_f32(const int64_t *d_idx, const float *d_distsq,
                                  const float *d_feat, const int32_t *d_argmax,
                                  const float *d_grad_fmean, const float *d_grad_fmax,
                                  float *d_grad_feat, float *d_grad_distsq, int64_t n_vert,
                                  int32_t K, int32_t P, void *stream);

/* The same with leading dimensions, so that the layer around the aggregation needs no copies: the features may
 * be columns of a wider matrix (ld_feat floats per row, n_feat_rows rows; gnn_ops.py:83 computes them as a matrix
 * of their own), d_fmean / d_fmax may point into one [n_vert, 2P] matrix that feeds the output layer directly
 * (ld_out; replaces the torch.cat of gnn_ops.py:105), the gradients come from and go to such matrices likewise.
 * A neighbour index >= n_feat_rows sets FGC_ST_BAD_INDEX in d_status (optional) and counts as padding. */
int fgc_gravnet_aggregate_fwd_ld_f32(const int64_t *d_idx, const float *d_distsq, const float *d_feat,
                                     int32_t ld_feat, int64_t n_feat_rows, float *d_fmean, float *d_fmax,
                                     int32_t ld_out, int32_t *d_argmax, int64_t n_vert, int32_t K, int32_t P,
                                     int32_t *d_status, void *stream);
int fgc_gravnet_aggregate_bwd_ld_f32(const int64_t *d_idx, const float *d_distsq, const float *d_feat,
                                     int32_t ld_feat, int64_t n_feat_rows, const int32_t *d_argmax,
                                     const float *d_grad_fmean, const float *d_grad_fmax, int32_t ld_grad,
                                     float *d_grad_feat, int32_t ld_grad_feat, float *d_grad_distsq,
                                     int64_t n_vert, int32_t K, int32_t P, int32_t *d_status, void *stream);

/* The backward for callers that hold the neighbour rows in the search's sorted order (d_nbr_sorted and d_order as
 * for fgc_binned_select_knn_grad_sorted_f32; everything else - d_distsq, d_feat, d_argmax, the gradients - stays in
 * the original order): the feature gradients of 16 consecutive sorted rows, which share most of their neighbours,
 * are combined on chip, so that one row update per distinct target of the tile reaches memory instead of one per
 * (point, slot) pair.  Same results as fgc_gravnet_aggregate_bwd_ld_f32 up to the order of the float sums.
 * Supports K <= 64, 8 < P <= 64, fewer than 2^24 points, rows of fewer than 2^22 floats and matrices of less than
 * 4 GiB (24-bit row arithmetic, 32-bit byte offsets); FGC_ESHAPE otherwise: fgc_gravnet_aggregate_bwd_ld_f32 takes
 * every shape.  fgc_gravnet_aggregate_bwd_sorted_supported returns 1 for exactly the shapes this entry point takes,
 * so that a caller can choose without trying. */
int fgc_gravnet_aggregate_bwd_sorted_supported(int64_t n_vert, int32_t K, int32_t P, int32_t ld_feat,
                                               int32_t ld_grad_feat);
int fgc_gravnet_aggregate_bwd_sorted_f32(const int32_t *d_nbr_sorted, const int32_t *d_order, const float *d_distsq,
                                         const float *d_feat, int32_t ld_feat, const int32_t *d_argmax,
                                         const float *d_grad_fmean, const float *d_grad_fmax, int32_t ld_grad,
                                         float *d_grad_feat, int32_t ld_grad_feat, float *d_grad_distsq,
                                         int64_t n_vert, int32_t K, int32_t P, int32_t *d_status, void *stream);

/* ---------------------------------------------------------------------------
 * Weight and bias gradient of a dense layer y = x W^T + b over n points:
 *   d_grad_weight [n_out, n_in] = grad_out^T x,  d_grad_bias [n_out] = column sums
 * of grad_out (NULL to skip).  Replaces the weight-gradient GEMMs that autograd
 * issues for the three nn.Linear layers of GravNetOp (gnn_ops.py:48-62,79-80,
 * 105): with n ~ 10^5..10^6 and n_out, n_in <= a few hundred a tiled library
 * GEMM runs one workgroup per output tile; this splits the points over the
 * chip (MFMA fp32, fixed summation order).
 *   d_grad_out [n, n_out], d_input [n, n_in] float32 row-major
 *   d_ws       fgc_linear_wgrad_workspace_bytes(n, n_out, n_in) bytes
 */
size_t fgc_linear_wgrad_workspace_bytes(int64_t n, int32_t n_out, int32_t n_in);
int fgc_linear_wgrad_f32(const float *d_grad_out, const float *d_input, int64_t n, int32_t n_out,
                         int32_t n_in, float *d_grad_weight, float *d_grad_bias, void *d_ws,
                         size_t ws_bytes, void *stream);

/* ---------------------------------------------------------------------------
 * Object-condensation helper matrices.  Two calls with one host read between
 * them (the output shapes depend on the data):
 *
 * fgc_oc_helper_objects_i64 replaces the input analysis of oc_helper_matrices,
 * i.e. _helper_inputs (oc_helper.py:18-149: torch.unique over (value, row
 * split) pairs) and max_same_valued_entries_per_row_split
 * (oc_helper_helper.cpp:30-94).  An object is a distinct (association index,
 * row split) pair; with filter_negative != 0 negative indices form no object.
 *   d_asso               int64 [n_vert] association (truth) index per vertex
 *   d_row_splits         int64 [n_rs] on the device
 *   wide_keys            0: sort on 32-bit keys (row split beside value + 1);
 *                        summary[2] bit 0 is set when a value does not fit and
 *                        the call must be repeated with wide_keys = 1 (full
 *                        64-bit values, three sorts).  Forced when
 *                        filter_negative == 0.
 *   d_max_per_split      out int64 [n_rs-1] vertices of the largest object
 *   d_objects_per_split  out int64 [n_rs-1] number of objects
 *   d_summary            out int64 [FGC_OC_SUMMARY_WORDS]: [0] number of objects
 *                        (rows of M), [1] vertices of the largest object
 *                        (columns of M), [2] flags
 *   d_ws                 fgc_oc_helper_workspace_bytes(n_vert) bytes; holds the
 *                        object table (ordered by row split, then value) that
 *                        fgc_oc_helper_fill_i64 reads
 *
 * fgc_oc_helper_fill_i64 replaces oc_helper_cuda_fn
 * (oc_helper_cuda_kernel.cu:154-203, kernel calc_m :19-116; CPU twin
 * oc_helper_cpu.cpp:17-82) including its transposes: row k of M [n_rows,
 * n_maxuq] lists the vertices of object k in ascending order, row k of M_not
 * [n_rows, n_maxrs] the other vertices of the object's row split in ascending
 * order, both padded with -1.
 *   d_unique_idx, d_unique_rs  NULL: rows follow the library's object table
 *                        (n_rows = summary[0]); else int64 [n_rows] objects in
 *                        the caller's order as the reference's op takes them
 *                        (a pair without vertices gives an all -1 row of M and
 *                        the whole row split in M_not); d_summary is then read
 *                        on the device
 *   d_M_not              NULL to skip (calc_m_not = False)
 *   d_obj_idx_out, d_obj_rs_out  optional int64 [n_rows]: value and row split
 *                        of each object of the library's table
 *   d_status             optional int32[FGC_STATUS_WORDS]; FGC_ST_OC_TRUNCATED
 *                        when n_maxuq is smaller than an object (the reference
 *                        prints and stops filling, oc_helper_cuda_kernel.cu:59-63)
 * Row splits longer than n_maxrs are cut to n_maxrs vertices as in
 * oc_helper_cuda_kernel.cu:49-52.
 */
#define FGC_OC_SUMMARY_WORDS 4
size_t fgc_oc_helper_workspace_bytes(int64_t n_vert);
int fgc_oc_helper_objects_i64(const int64_t *d_asso, int64_t n_vert, const int64_t *d_row_splits, int32_t n_rs,
                              int32_t filter_negative, int32_t wide_keys, int64_t *d_max_per_split,
                              int64_t *d_objects_per_split, int64_t *d_summary, void *d_ws, size_t ws_bytes,
                              void *stream);
int fgc_oc_helper_fill_i64(int64_t n_vert, const int64_t *d_row_splits, int32_t n_rs, int64_t n_rows,
                           int64_t n_maxuq, int64_t n_maxrs, const int64_t *d_unique_idx,
                           const int64_t *d_unique_rs, const int64_t *d_summary, int64_t *d_M, int64_t *d_M_not,
                           int64_t *d_obj_idx_out, int64_t *d_obj_rs_out, int32_t *d_status, const void *d_ws,
                           size_t ws_bytes, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* FGC_HIP_H_ */
