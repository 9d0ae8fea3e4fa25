// Whole-call entry points and bookkeeping of libfgc_hip.so.
#include "fgc_common.h"
#include "fgc_internal.h"
#include <algorithm>
#include <cstdlib>
#include <mutex>

extern "C" int fgc_version(void) { return 101; }

extern "C" const char *fgc_error_string(int code)
{
    switch (code) {
    case FGC_OK: return "success";
    case FGC_EINVAL: return "invalid argument (shape, size or row splits)";
    case FGC_ENOSPACE: return "workspace too small";
    case FGC_EUNSUPPORTED: return "Unsupported number of binning dimensions.";
    case FGC_ESHAPE:
        return "shape outside what this specialised entry point handles; the general entry point takes every shape";
    case FGC_ETOOLARGE:
        return "input needs more scratch memory than the fixed area of the no-allocation entry point "
               "(FGC_NOALLOC_SCRATCH_BYTES); use fgc_binned_select_knn_f32 with a workspace of the caller";
    default: break;
    }
    if (code > 0) return hipGetErrorString((hipError_t)code);
    return "unknown error";
}

namespace {
struct KnnWorkspace {
    size_t geom, partial, keys, vals, sort, sort_alt_vals, bb, sc, sp, spa, grp, mfstat, redo, sdir, box_lo, box_hi, sbox_lo, sbox_hi, total;
    bool with_sp;
    int ldc;
};

int64_t total_bins(int n_bin_dims, const int64_t *n_bins, int n_rs)
{
    int64_t b = n_rs - 1;
    for (int d = 0; d < n_bin_dims; d++) {
        if (n_bins[d] < 1 || n_bins[d] > (1ll << 31)) return -1;
        if (b > (1ll << 31) / n_bins[d]) return -1;
        b *= n_bins[d];
    }
    return b;
}

KnnWorkspace plan(int64_t n, int D, int K, int nbd, const int64_t *n_bins, int n_rs, bool with_dir)
{
    KnnWorkspace w;
    size_t off = 0;
    auto take = [&](size_t bytes) { size_t o = off; off += fgc_align(bytes); return o; };
    int64_t B = total_bins(nbd, n_bins, n_rs);
    if (B < 0) B = 0;
    w.ldc = (int)((n + 63) & ~63ll);
    w.geom = take(FGC_GEOM_FLOATS * sizeof(float));
    w.partial = take(fgc_bin_geometry_workspace_bytes(n));
    w.keys = take((size_t)n * 4);
    w.vals = take((size_t)n * 4);
    w.sort = take(fgc_sort_workspace_bytes(n));
    w.sort_alt_vals = fgc_align((size_t)n * 4);  // offset of the alternate value buffer inside the sort area
    w.bb = take((size_t)(B + 1) * 4);
    w.sc = take((size_t)w.ldc * D * 4);
    w.with_sp = fgc_knn_uses_mfma(D, K);     // rows of 8 floats for the matrix-core search
    w.sp = take(w.with_sp ? (size_t)w.ldc * 32 : 0);
    w.spa = take(w.with_sp ? (size_t)w.ldc * 32 : 0);    // float16 operands of the same points
    w.grp = take(w.with_sp ? (size_t)((w.ldc / 64 + FGC_MF_GROUP_CHUNKS - 1) / FGC_MF_GROUP_CHUNKS) * FGC_MF_GRP_FLOATS * 4 : 0);
    w.mfstat = take(w.with_sp ? 8 : 0);
    w.redo = take(w.with_sp ? (size_t)w.ldc : 0);   // flags of the queries the matrix-core search leaves to the vector search
    w.sdir = take(with_dir ? (size_t)n : 0);
    w.box_lo = take((size_t)(w.ldc / 64) * D * 4);
    w.box_hi = take((size_t)(w.ldc / 64) * D * 4);
    w.sbox_lo = take((size_t)((w.ldc / 64 + 63) / 64) * D * 4);
    w.sbox_hi = take((size_t)((w.ldc / 64 + 63) / 64) * D * 4);
    w.total = off;
    return w;
}
}  // namespace

extern "C" size_t fgc_binned_select_knn_workspace_bytes(int64_t n_vert, int32_t n_coords, int32_t n_bin_dims,
                                                        const int64_t *n_bins, int32_t n_rs, int32_t K)
{
    if (n_vert <= 0 || !n_bins || n_bin_dims < 1 || n_bin_dims > FGC_MAX_BIN_DIMS) return 256;
    return plan(n_vert, n_coords, K, n_bin_dims, n_bins, n_rs, true).total;
}

namespace {
struct KnnCall {
    KnnWorkspace w;
    int64_t B;
    int sub_bits;   // sub-cell bits per binned dimension appended to the flat bin in the sort key
    int key_bits;   // total significant bits of the sort key
};

// bits per binned dimension for the order inside a bin (sub-cells along a Hilbert curve): five if they fit into
// the 32-bit key, and beyond that as many as the radix sort takes without another 8-bit pass (dense bins, e.g. a
// cluster of 10^5 points in one bin, need the finer cells; sparse ones lose nothing)
int choose_sub_bits(int bin_bits, int nbd)
{
    int sb = (32 - bin_bits) / nbd;
    if (sb > 5) {
        const int passes5 = (bin_bits + 5 * nbd + 7) / 8;
        int s = 5;
        while (s < 8 && s < sb && (bin_bits + (s + 1) * nbd + 7) / 8 == passes5) s++;
        sb = s;
    }
    if (sb < 0) sb = 0;
    return sb;
}

// argument validation shared by the staged and the whole-call entry points
int knn_validate(int64_t n_vert, int32_t n_coords, const int64_t *row_splits_host, int32_t n_rs, int32_t K,
                 int32_t n_bin_dims, const int64_t *n_bins, bool with_dir, const void *d_ws, size_t ws_bytes,
                 KnnCall *c)
{
    if (n_vert < 0 || n_coords < 1 || n_rs < 2 || !row_splits_host || !n_bins) return FGC_EINVAL;
    if (K < 1 || K > FGC_MAX_K) return FGC_EINVAL;
    if (n_bin_dims < 2 || n_bin_dims > FGC_MAX_BIN_DIMS || n_bin_dims > n_coords) return FGC_EUNSUPPORTED;
    if (n_vert >= (1ll << 31) - 64) return FGC_EINVAL;
    // "Bin boundaries do not match row splits" of the reference, checked up front
    if (row_splits_host[0] != 0 || row_splits_host[n_rs - 1] != n_vert) return FGC_EINVAL;
    for (int r = 1; r < n_rs; r++)
        if (row_splits_host[r] < row_splits_host[r - 1]) return FGC_EINVAL;
    c->B = total_bins(n_bin_dims, n_bins, n_rs);
    if (c->B < 0 || c->B >= (1ll << 31)) return FGC_EINVAL;
    c->w = plan(n_vert > 0 ? n_vert : 1, n_coords, K, n_bin_dims, n_bins, n_rs, with_dir);
    int bin_bits = 1;
    while ((1ll << bin_bits) < c->B) bin_bits++;
    c->sub_bits = choose_sub_bits(bin_bits, n_bin_dims);
    c->key_bits = bin_bits + c->sub_bits * n_bin_dims;
    if (n_vert > 0 && (!d_ws || ws_bytes < c->w.total)) return d_ws ? FGC_ENOSPACE : FGC_EINVAL;
    return FGC_OK;
}

// where the sorted keys / order end up after the ping-pong passes of the sort
void sorted_buffers(const KnnCall &c, char *ws, uint32_t **skeys, uint32_t **order)
{
    const int passes = (c.key_bits + 7) / 8;
    const bool in_alt = (passes & 1) != 0;
    char *sortws = ws + c.w.sort;
    *skeys = in_alt ? (uint32_t *)sortws : (uint32_t *)(ws + c.w.keys);
    *order = in_alt ? (uint32_t *)(sortws + c.w.sort_alt_vals) : (uint32_t *)(ws + c.w.vals);
}
}  // namespace

extern "C" int fgc_binned_knn_prepare_f32(const float *d_coords, int64_t n_vert, int32_t n_coords,
                                          const int64_t *d_row_splits, const int64_t *row_splits_host,
                                          int32_t n_rs, int32_t K, int32_t n_bin_dims, const int64_t *n_bins,
                                          const int64_t *d_direction, int32_t *d_status, void *d_ws,
                                          size_t ws_bytes, void *stream)
{
    return fgc_binned_knn_prepare_ld_f32(d_coords, n_vert, n_coords, n_coords, d_row_splits, row_splits_host, n_rs, K,
                                         n_bin_dims, n_bins, d_direction, d_status, d_ws, ws_bytes, stream);
}

extern "C" int fgc_binned_knn_prepare_ld_f32(const float *d_coords, int64_t n_vert, int32_t n_coords,
                                             int32_t ld_coords, const int64_t *d_row_splits,
                                             const int64_t *row_splits_host, int32_t n_rs, int32_t K,
                                             int32_t n_bin_dims, const int64_t *n_bins,
                                             const int64_t *d_direction, int32_t *d_status, void *d_ws,
                                             size_t ws_bytes, void *stream)
{
    if (ld_coords < n_coords) return FGC_EINVAL;
    KnnCall c;
    int rc = knn_validate(n_vert, n_coords, row_splits_host, n_rs, K, n_bin_dims, n_bins, d_direction != nullptr,
                          d_ws, ws_bytes, &c);
    if (rc) return rc;
    if (n_vert == 0) return FGC_OK;
    if (!d_coords || !d_row_splits) return FGC_EINVAL;
    const KnnWorkspace &w = c.w;
    hipStream_t s = (hipStream_t)stream;
    char *ws = (char *)d_ws;
    float *geom = (float *)(ws + w.geom);
    uint32_t *keys = (uint32_t *)(ws + w.keys), *vals = (uint32_t *)(ws + w.vals);
    int *bb = (int *)(ws + w.bb);
    float *sc = (float *)(ws + w.sc);
    unsigned char *sdir = d_direction ? (unsigned char *)(ws + w.sdir) : nullptr;

    float *spp = w.with_sp ? (float *)(ws + w.sp) : nullptr;
    uint32_t *skeys = nullptr, *order = nullptr;
    if (fgc_sort_fused_fits(n_vert)) {
        // up to a few hundred thousand points: one launch per sort pass, the geometry record derived by the key kernel
        rc = fgc_keys_and_sort_fused(d_coords, (int)n_vert, ld_coords, n_bin_dims, n_bins, c.sub_bits, c.key_bits,
                                     d_row_splits, n_rs, (float *)(ws + w.partial), geom, keys, vals, ws + w.sort,
                                     d_status, s, &skeys, &order);
        if (rc) return rc;
    } else {
        rc = fgc_bin_geometry_f32(d_coords, n_vert, ld_coords, n_bin_dims, 2, n_bins, 1, 0.f, 0, geom, d_status,
                                  ws + w.partial, fgc_bin_geometry_workspace_bytes(n_vert), stream);
        if (rc) return rc;
        rc = fgc_launch_bin_keys(d_coords, (int)n_vert, ld_coords, n_bin_dims, c.sub_bits, geom, d_row_splits, n_rs,
                                 keys, d_status, s);
        if (rc) return rc;
        rc = fgc_sort_keys(keys, vals, n_vert, c.key_bits, ws + w.sort, s, &skeys, &order);
        if (rc) return rc;
    }
    {
        uint32_t *skeys2, *order2;
        sorted_buffers(c, ws, &skeys2, &order2);
        if (skeys2 != skeys || order2 != order) return FGC_EINVAL;  // internal layout mismatch
    }
    rc = fgc_launch_prepare_tail(d_coords, ld_coords, order, skeys, (int)n_vert, n_coords, w.ldc, sc, d_direction, sdir,
                                 spp, fgc_knn_sp_half(n_coords), (float *)(ws + w.box_lo), (float *)(ws + w.box_hi),
                                 (float *)(ws + w.sbox_lo), (float *)(ws + w.sbox_hi), c.sub_bits * n_bin_dims,
                                 (int)c.B, bb, w.with_sp ? (unsigned *)(ws + w.mfstat) : nullptr, s);
    if (rc || !w.with_sp) return rc;
    return fgc_launch_mf_operands((const float *)(ws + w.sp), (const float *)(ws + w.box_lo),
                                  (const float *)(ws + w.box_hi), (int)n_vert, n_coords, w.ldc, (float *)(ws + w.grp),
                                  ws + w.spa, (unsigned *)(ws + w.mfstat), s);
}

namespace {
int knn_search(float tau0, int32_t *d_nbr_sorted, int64_t n_vert, int32_t n_coords, const int64_t *row_splits_host,
                                         int32_t n_rs, int32_t K, int32_t n_bin_dims, const int64_t *n_bins,
                                         int32_t with_direction, int32_t tf_compat, int64_t *d_idx,
                                         float *d_distsq, uint64_t *d_stats, void *d_ws, size_t ws_bytes,
                                         void *stream)
{
    KnnCall c;
    int rc = knn_validate(n_vert, n_coords, row_splits_host, n_rs, K, n_bin_dims, n_bins, with_direction != 0,
                          d_ws, ws_bytes, &c);
    if (rc) return rc;
    if (n_vert == 0) return FGC_OK;
    if (!d_idx || !d_distsq) return FGC_EINVAL;
    char *ws = (char *)d_ws;
    KnnArgs a;
    uint32_t *skeys, *order;
    sorted_buffers(c, ws, &skeys, &order);
    a.sc = (const float *)(ws + c.w.sc); a.ldc = c.w.ldc; a.skeys = skeys; a.order = order;
    a.key_shift = c.sub_bits * n_bin_dims;
    a.box_lo = (const float *)(ws + c.w.box_lo); a.box_hi = (const float *)(ws + c.w.box_hi);
    a.n_chunks = c.w.ldc / 64;
    a.sbox_lo = (const float *)(ws + c.w.sbox_lo); a.sbox_hi = (const float *)(ws + c.w.sbox_hi);
    a.n_super = (a.n_chunks + 63) / 64;
    a.bb = (const int *)(ws + c.w.bb); a.geom = (const float *)(ws + c.w.geom);
    a.sdir = with_direction ? (const unsigned char *)(ws + c.w.sdir) : nullptr;
    a.n = (int)n_vert; a.D = n_coords; a.nbd = n_bin_dims; a.K = K;
    a.tf_compat = (tf_compat & FGC_KNN_TF_COMPAT) != 0; a.any_order = (tf_compat & FGC_KNN_ANY_ORDER) != 0;
    a.tau0 = tau0;
    a.out_sorted = d_nbr_sorted;
    a.out_idx = d_idx; a.out_dist = d_distsq; a.stats = (unsigned long long *)d_stats;
    a.sp = c.w.with_sp ? (const float *)(ws + c.w.sp) : nullptr;
    a.spa = c.w.with_sp ? (const void *)(ws + c.w.spa) : nullptr;
    a.grp = c.w.with_sp ? (const float *)(ws + c.w.grp) : nullptr;
    a.mfstat = c.w.with_sp ? (const unsigned *)(ws + c.w.mfstat) : nullptr;
    a.redo = nullptr;
    // Many coordinates and events that the bounding boxes cannot thin out: the matrix-core search.  Measured on
    // uniform and clustered points with 1 000 to 65 000 points per event: it wins up to about 1536 * 3^(D - 5)
    // points per event (half as many again from K = 64 on), where the size is the one a typical point sees,
    // sum n_e^2 / n.
    // It stores candidates as 16-bit positions inside their event, so no event may exceed 65535 points.  A search
    // with a radius bound keeps the vector search, which culls by the bound from the first bin row on.
    int64_t largest_event = 0;
    double sum_sq = 0;
    for (int r = 1; r < n_rs; r++) {
        const int64_t ne = row_splits_host[r] - row_splits_host[r - 1];
        largest_event = std::max(largest_event, ne);
        sum_sq += (double)ne * (double)ne;
    }
    const double typical_event = n_vert > 0 ? sum_sq / (double)n_vert : 0.0;
    double limit = 1536.0;
    for (int d = 5; d < n_coords; d++) limit *= 3.0;
    if (K >= 64) limit *= 1.5;
    limit = std::min(limit, 32768.0);
    const bool force = (tf_compat & FGC_KNN_FORCE_MATRIX) != 0;
    if (a.sp && !(tf_compat & FGC_KNN_NO_MATRIX) && !(tau0 < INFINITY) && largest_event <= 65535 &&
        (typical_event <= limit || force)) {
        a.redo = (unsigned char *)(ws + c.w.redo);
        return a.stats ? fgc_launch_knn_mfma_stats(a, (hipStream_t)stream) : fgc_launch_knn_mfma(a, (hipStream_t)stream);
    }
    return a.stats ? fgc_launch_knn_stats(a, (hipStream_t)stream) : fgc_launch_knn(a, (hipStream_t)stream);
}

}  // namespace

extern "C" int fgc_binned_knn_export_order_i32(int64_t n_vert, int32_t n_coords, const int64_t *row_splits_host,
                                               int32_t n_rs, int32_t K, int32_t n_bin_dims,
                                               const int64_t *n_bins, int32_t with_direction, const void *d_ws,
                                               size_t ws_bytes, int32_t *d_order_out, void *stream)
{
    KnnCall c;
    int rc = knn_validate(n_vert, n_coords, row_splits_host, n_rs, K, n_bin_dims, n_bins, with_direction != 0,
                          d_ws, ws_bytes, &c);
    if (rc) return rc;
    if (n_vert == 0) return FGC_OK;
    if (!d_order_out) return FGC_EINVAL;
    uint32_t *skeys, *order;
    sorted_buffers(c, (char *)const_cast<void *>(d_ws), &skeys, &order);
    return fgc_copy_u32(d_order_out, order, n_vert, (hipStream_t)stream);
}

extern "C" int fgc_binned_knn_search_f32(int64_t n_vert, int32_t n_coords, const int64_t *row_splits_host,
                                         int32_t n_rs, int32_t K, int32_t n_bin_dims, const int64_t *n_bins,
                                         int32_t with_direction, int32_t tf_compat, int64_t *d_idx,
                                         float *d_distsq, int32_t *d_nbr_sorted, uint64_t *d_stats, void *d_ws,
                                         size_t ws_bytes, void *stream)
{
    return knn_search(INFINITY, d_nbr_sorted, n_vert, n_coords, row_splits_host, n_rs, K, n_bin_dims, n_bins, with_direction,
                      tf_compat, d_idx, d_distsq, d_stats, d_ws, ws_bytes, stream);
}

extern "C" int fgc_select_knn_f32(const float *d_coords, int64_t n_vert, int32_t n_coords,
                                  const int64_t *d_row_splits, const int64_t *row_splits_host, int32_t n_rs,
                                  int32_t K, double max_radius, int32_t n_bin_dims, const int64_t *n_bins,
                                  int64_t *d_idx, float *d_distsq, int32_t *d_status, void *d_ws,
                                  size_t ws_bytes, void *stream)
{
    int rc = fgc_binned_knn_prepare_f32(d_coords, n_vert, n_coords, d_row_splits, row_splits_host, n_rs, K,
                                        n_bin_dims, n_bins, nullptr, d_status, d_ws, ws_bytes, stream);
    if (rc) return rc;
    float tau0 = INFINITY;
    if (max_radius > 0) {
        // the reference squares the radius in double, narrows it to float and accepts distsq <= that
        // (select_knn_cpu.cpp:174-176,110); the search keeps candidates strictly below its bound
        const float r2 = (float)(max_radius * max_radius);
        tau0 = nextafterf(r2, INFINITY);
    }
    return knn_search(tau0, nullptr, n_vert, n_coords, row_splits_host, n_rs, K, n_bin_dims, n_bins, 0, 0, d_idx,
                      d_distsq, nullptr, d_ws, ws_bytes, stream);
}

extern "C" int fgc_binned_select_knn_f32(const float *d_coords, int64_t n_vert, int32_t n_coords,
                                         const int64_t *d_row_splits, const int64_t *row_splits_host,
                                         int32_t n_rs, int32_t K, int32_t n_bin_dims, const int64_t *n_bins,
                                         const int64_t *d_direction, int32_t tf_compat, int64_t *d_idx,
                                         float *d_distsq, int32_t *d_status, uint64_t *d_stats, void *d_ws,
                                         size_t ws_bytes, void *stream)
{
    int rc = fgc_binned_knn_prepare_f32(d_coords, n_vert, n_coords, d_row_splits, row_splits_host, n_rs, K,
                                        n_bin_dims, n_bins, d_direction, d_status, d_ws, ws_bytes, stream);
    if (rc) return rc;
    return fgc_binned_knn_search_f32(n_vert, n_coords, row_splits_host, n_rs, K, n_bin_dims, n_bins,
                                     d_direction != nullptr, tf_compat, d_idx, d_distsq, nullptr, d_stats, d_ws,
                                     ws_bytes, stream);
}

// ---------------------------------------------------------------------------
// The whole forward for callers that cannot allocate (code under HIP graph capture, tight serving loops): the
// workspace is a fixed array in the code object's own device memory.  Every GPU the library runs on holds one
// copy of it at its own address until the process ends; that address is looked up once per device.
// ---------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[FGC_NOALLOC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void *g_scratch_ptr[kMaxDevices];    // device address of `scratch` on each device, 0 = not looked up yet

// address of this device's copy of `scratch` (the array's name is only a host-side handle for the lookup)
int scratch_address(void **out)
{
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= kMaxDevices) return FGC_EINVAL;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (!p) return FGC_EINVAL;
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return FGC_OK;
}
}  // namespace

// Looks the scratch address of the current device up ahead of time, so that the first
// fgc_binned_select_knn_noalloc_f32 on that device does no symbol lookup (and no lazy load of the code object): a
// caller that captures the entry point into a HIP graph calls this once per device before it starts capturing.
extern "C" int fgc_noalloc_init(void)
{
    void *ws = nullptr;
    return scratch_address(&ws);
}

extern "C" int fgc_binned_select_knn_noalloc_f32(const float *d_coords, int64_t n_vert, int32_t n_coords,
                                                 const int64_t *d_row_splits, const int64_t *row_splits_host,
                                                 int32_t n_rs, int32_t K, int32_t n_bin_dims,
                                                 const int64_t *n_bins, const int64_t *d_direction,
                                                 int32_t tf_compat, int64_t *d_idx, float *d_distsq,
                                                 int32_t *d_status, void *stream)
{
    if (n_vert < 0 || n_coords < 1 || n_rs < 2 || !n_bins || n_bin_dims < 1 || n_bin_dims > FGC_MAX_BIN_DIMS)
        return FGC_EINVAL;
    const size_t need = n_vert > 0 ? plan(n_vert, n_coords, K, n_bin_dims, n_bins, n_rs, d_direction != nullptr).total : 0;
    if (need > (size_t)FGC_NOALLOC_SCRATCH_BYTES) return FGC_ETOOLARGE;
    void *ws = nullptr;
    int rc = scratch_address(&ws);
    if (rc) return rc;
    // every stage writes what it later reads (the workspace of the other entry points is uninitialised memory
    // too), so nothing of the previous call's contents has to be cleared
    return fgc_binned_select_knn_f32(d_coords, n_vert, n_coords, d_row_splits, row_splits_host, n_rs, K, n_bin_dims,
                                     n_bins, d_direction, tf_compat, d_idx, d_distsq, d_status, nullptr, ws,
                                     (size_t)FGC_NOALLOC_SCRATCH_BYTES, stream);
}
