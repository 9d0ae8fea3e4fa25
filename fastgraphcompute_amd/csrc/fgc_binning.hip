// Binning geometry, per-point binning, and the stable LSD radix sort that puts
// points into bin order (keys = flat bin index, 8-bit digits, LDS histograms,
// wave-ballot ranking).  gfx950, wave64.
#include "fgc_common.h"
#include "fgc_internal.h"

// ---------------------------------------------------------------------------
// small utilities
// ---------------------------------------------------------------------------
__global__ void k_fill_u32(uint32_t *p, uint32_t v, int64_t n)
{
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) p[i] = v;
}

int fgc_fill_u32(void *d, uint32_t v, int64_t n_words, hipStream_t s)
{
    if (n_words <= 0) return FGC_OK;
    int64_t blocks = fgc_cdiv(n_words, 256 * 8);
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(k_fill_u32, dim3((unsigned)blocks), dim3(256), 0, s, (uint32_t *)d, v, n_words);
    FGC_LAUNCH_CHECK();
    return FGC_OK;
}

__global__ void k_copy_u32(uint32_t *__restrict__ dst, const uint32_t *__restrict__ src, int64_t n)
{
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) dst[i] = src[i];
}

int fgc_copy_u32(void *dst, const void *src, int64_t n_words, hipStream_t s)
{
    if (n_words <= 0) return FGC_OK;
    int64_t blocks = fgc_cdiv(n_words, 256 * 8);
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(k_copy_u32, dim3((unsigned)blocks), dim3(256), 0, s, (uint32_t *)dst, (const uint32_t *)src,
                       n_words);
    FGC_LAUNCH_CHECK();
    return FGC_OK;
}

// minimum / maximum over the 64 lanes, in every lane: four DPP steps inside each row of 16 lanes, then the four
// rows through scalar reads
__device__ __forceinline__ float wave_min_f(float v)
{
    v = fminf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xf, 0xf, true)));
    v = fminf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xf, 0xf, true)));
    v = fminf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xf, 0xf, true)));
    v = fminf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xf, 0xf, true)));
    return fminf(fminf(fgc_readlane_f(v, 0), fgc_readlane_f(v, 16)), fminf(fgc_readlane_f(v, 32), fgc_readlane_f(v, 48)));
}
__device__ __forceinline__ float wave_max_f(float v)
{
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xf, 0xf, true)));
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xf, 0xf, true)));
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xf, 0xf, true)));
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xf, 0xf, true)));
    return fmaxf(fmaxf(fgc_readlane_f(v, 0), fgc_readlane_f(v, 16)), fmaxf(fgc_readlane_f(v, 32), fgc_readlane_f(v, 48)));
}

// ---------------------------------------------------------------------------
// geometry: per-dimension min / max of the binned coordinates
// ---------------------------------------------------------------------------
#define RANGE_BLOCKS_MAX 1024

// partial[blk][0..4] = min, [5..9] = max, [10] = non-finite seen (as float 0/1)
// (also clears `zero_words` words at `zero`: the digit tables of the sort that follows on a small input)
__global__ __launch_bounds__(256) void k_range_partial(const float *__restrict__ coords, int64_t n,
                                                       int ld, int nbd, float *__restrict__ partial,
                                                       uint32_t *__restrict__ zero, int zero_words)
{
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < zero_words; i += gridDim.x * blockDim.x) zero[i] = 0u;
    float mn[FGC_MAX_BIN_DIMS], mx[FGC_MAX_BIN_DIMS];
    int bad = 0;
#pragma unroll
    for (int d = 0; d < FGC_MAX_BIN_DIMS; d++) { mn[d] = INFINITY; mx[d] = -INFINITY; }
    int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
#pragma unroll
        for (int d = 0; d < FGC_MAX_BIN_DIMS; d++)
            if (d < nbd) {
                float x = coords[i * ld + d];
                bad |= !isfinite(x);
                mn[d] = fminf(mn[d], x);
                mx[d] = fmaxf(mx[d], x);
            }
    }
    __shared__ float s_red[4][11];
    const int lane = fgc_lane(), wv = threadIdx.x >> 6;
#pragma unroll
    for (int d = 0; d < FGC_MAX_BIN_DIMS; d++) {
        float a = wave_min_f(mn[d]), b = wave_max_f(mx[d]);
        if (lane == 0) { s_red[wv][d] = a; s_red[wv][5 + d] = b; }
    }
    unsigned long long anybad = fgc_ballot(bad != 0);
    if (lane == 0) s_red[wv][10] = anybad ? 1.f : 0.f;
    __syncthreads();
    if (threadIdx.x < 11) {
        int t = threadIdx.x;
        float v = s_red[0][t];
        for (int w = 1; w < 4; w++) {
            float o = s_red[w][t];
            v = (t < 5) ? fminf(v, o) : fmaxf(v, o);
        }
        partial[blockIdx.x * 11 + t] = v;
    }
}

// The geometry record from the per-dimension range (one thread).  Arithmetic order as the reference's tensor ops:
// (max - min), +1 where the range is zero, +1e-3, width = max_d(range_d / n_bins_d)  [or n_bins from a width].
__device__ inline void geometry_record(const float (&mn)[FGC_MAX_BIN_DIMS], const float (&mx)[FGC_MAX_BIN_DIMS], bool bad,
                                       int nbd, int mode, int nb_given, float bw_in, int pre_norm,
                                       const int (&nb_in)[FGC_MAX_BIN_DIMS], float *__restrict__ geom,
                                       int *__restrict__ status)
{
    int flags = bad ? FGC_ST_NONFINITE : 0;
    float rng[FGC_MAX_BIN_DIMS];
    float bw = bw_in;
    for (int d = 0; d < FGC_MAX_BIN_DIMS; d++) {
        if (d >= nbd) { geom[FGC_GEOM_MIN + d] = 0.f; continue; }
        float sub = pre_norm ? 0.f : mn[d];
        float lo = pre_norm ? mn[d] : (mn[d] - sub);
        float hi = pre_norm ? mx[d] : (mx[d] - sub);
        if (lo == hi) hi = hi + 1.0f;
        // mode 2 (the kNN search's own grid) pads the range relatively: point clouds that are tiny in absolute
        // terms still spread over all bins
        hi = (mode == 2) ? lo + (hi - lo) * 1.001f : hi + 1e-3f;
        if (!isfinite(hi)) hi = 1.0f;
        if (!(hi > 0.f)) flags |= FGC_ST_BAD_RANGE;
        rng[d] = hi;
        geom[FGC_GEOM_MIN + d] = sub;
    }
    int nbo[FGC_MAX_BIN_DIMS] = {1, 1, 1, 1, 1};
    if (mode == 0 || mode == 2) {
        float w = -INFINITY;
        for (int d = 0; d < nbd; d++) {
            nbo[d] = nb_in[d];
            w = fmaxf(w, rng[d] / (float)nb_in[d]);
        }
        bw = w;
    } else {
        for (int d = 0; d < nbd; d++)
            nbo[d] = nb_given ? nb_in[d] : (int)(long long)(rng[d] / bw) + 1;
    }
    for (int d = 0; d < nbd; d++)
        if (nbo[d] <= 0) flags |= FGC_ST_BAD_RANGE;
    if (!(bw > 0.f)) flags |= FGC_ST_BAD_RANGE;
    geom[FGC_GEOM_BW] = bw;
    for (int d = 0; d < FGC_MAX_BIN_DIMS; d++) geom[FGC_GEOM_NB + d] = __int_as_float(nbo[d]);
    geom[FGC_GEOM_FLAGS] = __int_as_float(flags);
    for (int d = 12; d < FGC_GEOM_FLOATS; d++) geom[d] = 0.f;
    if (status && flags) atomicOr(&status[0], flags);
}

// One block: reduce the partials and derive the geometry record.
__global__ __launch_bounds__(256) void k_geometry(const float *__restrict__ partial, int nblk, int nbd,
                                                  int mode, int nb_given, float bw_in, int pre_norm,
                                                  int nb0, int nb1, int nb2, int nb3, int nb4,
                                                  float *__restrict__ geom, int *__restrict__ status)
{
    __shared__ float s_red[4][11];
    const int lane = fgc_lane(), wv = threadIdx.x >> 6;
    float mn[FGC_MAX_BIN_DIMS], mx[FGC_MAX_BIN_DIMS];
    float bad = 0.f;
#pragma unroll
    for (int d = 0; d < FGC_MAX_BIN_DIMS; d++) { mn[d] = INFINITY; mx[d] = -INFINITY; }
    for (int b = threadIdx.x; b < nblk; b += 256) {
#pragma unroll
        for (int d = 0; d < FGC_MAX_BIN_DIMS; d++) {
            mn[d] = fminf(mn[d], partial[b * 11 + d]);
            mx[d] = fmaxf(mx[d], partial[b * 11 + 5 + d]);
        }
        bad = fmaxf(bad, partial[b * 11 + 10]);
    }
#pragma unroll
    for (int d = 0; d < FGC_MAX_BIN_DIMS; d++) {
        const float a = wave_min_f(mn[d]), b = wave_max_f(mx[d]);
        if (lane == 0) { s_red[wv][d] = a; s_red[wv][5 + d] = b; }
    }
    bad = wave_max_f(bad);
    if (lane == 0) s_red[wv][10] = bad;
    __syncthreads();
    if (threadIdx.x != 0) return;
#pragma unroll
    for (int d = 0; d < FGC_MAX_BIN_DIMS; d++) {
        mn[d] = fminf(fminf(s_red[0][d], s_red[1][d]), fminf(s_red[2][d], s_red[3][d]));
        mx[d] = fmaxf(fmaxf(s_red[0][5 + d], s_red[1][5 + d]), fmaxf(s_red[2][5 + d], s_red[3][5 + d]));
    }
    bad = fmaxf(fmaxf(s_red[0][10], s_red[1][10]), fmaxf(s_red[2][10], s_red[3][10]));
    const int nb_in[FGC_MAX_BIN_DIMS] = {nb0, nb1, nb2, nb3, nb4};
    geometry_record(mn, mx, bad > 0.f, nbd, mode, nb_given, bw_in, pre_norm, nb_in, geom, status);
}

extern "C" size_t fgc_bin_geometry_workspace_bytes(int64_t n_vert)
{
    (void)n_vert;
    return fgc_align((size_t)RANGE_BLOCKS_MAX * 11 * sizeof(float));
}

extern "C" int fgc_bin_geometry_f32(const float *d_coords, int64_t n_vert, int32_t ld_coords,
                                    int32_t n_bin_dims, int32_t mode, const int64_t *n_bins_in,
                                    int32_t n_bins_given, float bin_width_in, int32_t pre_normalized,
                                    float *d_geom, int32_t *d_status, void *d_ws, size_t ws_bytes,
                                    void *stream)
{
    if (n_vert <= 0 || n_bin_dims < 1 || n_bin_dims > FGC_MAX_BIN_DIMS || ld_coords < n_bin_dims)
        return FGC_EINVAL;
    if (!d_coords || !d_geom || !d_ws) return FGC_EINVAL;
    if (ws_bytes < fgc_bin_geometry_workspace_bytes(n_vert)) return FGC_ENOSPACE;
    if (mode < 0 || mode > 2) return FGC_EINVAL;
    if (mode != 1 && (!n_bins_in || !n_bins_given)) return FGC_EINVAL;
    int nb[FGC_MAX_BIN_DIMS] = {1, 1, 1, 1, 1};
    if (n_bins_in && n_bins_given)
        for (int d = 0; d < n_bin_dims; d++) {
            if (n_bins_in[d] > 0x7fffffff) return FGC_EINVAL;
            nb[d] = (int)n_bins_in[d];
        }
    hipStream_t s = (hipStream_t)stream;
    int nblk = (int)fgc_cdiv(n_vert, 256 * 4);
    if (nblk > RANGE_BLOCKS_MAX) nblk = RANGE_BLOCKS_MAX;
    hipLaunchKernelGGL(k_range_partial, dim3(nblk), dim3(256), 0, s, d_coords, n_vert, (int)ld_coords,
                       (int)n_bin_dims, (float *)d_ws, (uint32_t *)nullptr, 0);
    FGC_LAUNCH_CHECK();
    hipLaunchKernelGGL(k_geometry, dim3(1), dim3(256), 0, s, (const float *)d_ws, nblk, (int)n_bin_dims,
                       (int)mode, (int)n_bins_given, bin_width_in, (int)pre_normalized, nb[0], nb[1],
                       nb[2], nb[3], nb[4], d_geom, d_status);
    FGC_LAUNCH_CHECK();
    return FGC_OK;
}

// ---------------------------------------------------------------------------
// per-point binning
// ---------------------------------------------------------------------------
struct BinGeom {
    float mn[FGC_MAX_BIN_DIMS];
    float bw;
    int nb[FGC_MAX_BIN_DIMS];
};

__device__ __forceinline__ BinGeom load_geom(const float *__restrict__ geom)
{
    BinGeom g;
#pragma unroll
    for (int d = 0; d < FGC_MAX_BIN_DIMS; d++) {
        g.mn[d] = geom[FGC_GEOM_MIN + d];
        g.nb[d] = __float_as_int(geom[FGC_GEOM_NB + d]);
    }
    g.bw = geom[FGC_GEOM_BW];
    return g;
}

// number of row-split entries rs[1..n_rs-1] that are <= v  (the event of point v)
__device__ __forceinline__ int event_of(const int64_t *__restrict__ rs, int n_rs, int64_t v)
{
    int lo = 1, hi = n_rs;  // first r in [1, n_rs) with rs[r] > v
    while (lo < hi) {
        int mid = (lo + hi) >> 1;
        if (rs[mid] > v) hi = mid; else lo = mid + 1;
    }
    return lo - 1;
}

// bin index of one coordinate: floorf((x - min) / bw + 1e-3f), clamped
__device__ __forceinline__ int bin_of(float x, float mn, float bw, int nb, int &clamped)
{
    float q = (x - mn) / bw;
    long long b = (long long)floorf(q + 1e-3f);
    if (b < 0) { b = 0; clamped = 1; }
    else if (b >= nb) { b = nb - 1; clamped = 1; }
    return (int)b;
}

__global__ __launch_bounds__(256) void k_bin_points(const float *__restrict__ coords, int64_t n, int ld,
                                                    int nbd, const float *__restrict__ geom,
                                                    const int64_t *__restrict__ rs, int n_rs,
                                                    int64_t n_total_bins,
                                                    int64_t *__restrict__ assigned,
                                                    int64_t *__restrict__ flat,
                                                    unsigned long long *__restrict__ n_per_bin,
                                                    int *__restrict__ status)
{
    int64_t v = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (v >= n) return;
    BinGeom g = load_geom(geom);
    int clamped = 0;
    int64_t f = 0, stride = 1;
    int b[FGC_MAX_BIN_DIMS];
#pragma unroll
    for (int d = FGC_MAX_BIN_DIMS - 1; d >= 0; d--)
        if (d < nbd) {
            b[d] = bin_of(coords[v * ld + d], g.mn[d], g.bw, g.nb[d], clamped);
            f += (int64_t)b[d] * stride;
            stride *= g.nb[d];
        }
    int ev = event_of(rs, n_rs, v);
    f += (int64_t)ev * stride;
    if (clamped && status) atomicOr(&status[0], FGC_ST_CLAMPED);
    if (assigned) {
#pragma unroll
        for (int d = 0; d < FGC_MAX_BIN_DIMS; d++)
            if (d < nbd) assigned[v * (nbd + 1) + 1 + d] = b[d];
    }
    if (f >= n_total_bins) return;  // point beyond the last row split: left out, as the reference does
    if (assigned) assigned[v * (nbd + 1)] = ev;
    if (flat) flat[v] = f;
    if (n_per_bin) atomicAdd(&n_per_bin[f], 1ull);
}

extern "C" int fgc_bin_points_f32(const float *d_coords, int64_t n_vert, int32_t ld_coords,
                                  int32_t n_bin_dims, const float *d_geom, const int64_t *d_row_splits,
                                  int32_t n_rs, const int64_t *n_bins_host, int64_t *d_assigned,
                                  int64_t *d_flat, int64_t *d_n_per_bin, int32_t *d_status, void *stream)
{
    if (n_vert < 0 || n_bin_dims < 1 || n_bin_dims > FGC_MAX_BIN_DIMS || n_rs < 2 || !n_bins_host)
        return FGC_EINVAL;
    if (n_vert == 0) return FGC_OK;
    int64_t total = n_rs - 1;
    for (int d = 0; d < n_bin_dims; d++) {
        if (n_bins_host[d] <= 0) return FGC_EINVAL;
        if (total > INT64_MAX / n_bins_host[d]) return FGC_EINVAL;
        total *= n_bins_host[d];
    }
    hipStream_t s = (hipStream_t)stream;
    hipLaunchKernelGGL(k_bin_points, dim3((unsigned)fgc_cdiv(n_vert, 256)), dim3(256), 0, s, d_coords,
                       n_vert, (int)ld_coords, (int)n_bin_dims, d_geom, d_row_splits, (int)n_rs, total,
                       d_assigned, d_flat, (unsigned long long *)d_n_per_bin, d_status);
    FGC_LAUNCH_CHECK();
    return FGC_OK;
}

// ---------------------------------------------------------------------------
// sort keys for the kNN pipeline: key = (flat bin << sub_bits*nbd) | Hilbert index
// of the point's sub-cell inside its bin (sub_bits per binned dimension).  The
// low part only orders points inside a bin so that consecutive points are
// spatially compact (consecutive sub-cells of a Hilbert curve share a face, so a
// run of 64 points has a tight bounding box wherever it starts); it never changes
// which bin a point belongs to.
// ---------------------------------------------------------------------------
// key of point v (its coordinates at `row`, its event `ev`)
__device__ inline uint32_t knn_sort_key(const float *__restrict__ row, const BinGeom &g, int nbd, int sub_bits, int ev,
                                        int &clamped)
{
    uint32_t f = 0, stride = 1;
    int sub[FGC_MAX_BIN_DIMS];
    const int smax = (1 << sub_bits) - 1;
#pragma unroll
    for (int d = FGC_MAX_BIN_DIMS - 1; d >= 0; d--) {
        sub[d] = 0;
        if (d < nbd) {
            const float x = row[d];
            int b = bin_of(x, g.mn[d], g.bw, g.nb[d], clamped);
            f += (uint32_t)b * stride;
            stride *= (uint32_t)g.nb[d];
            const float t = (x - g.mn[d]) / g.bw + 1e-3f;
            const float fr = t - (float)b;  // position inside the bin, [0, 1) unless the point was clamped
            sub[d] = min(max((int)(fr * (float)(smax + 1)), 0), smax);
        }
    }
    f += (uint32_t)ev * stride;
#ifndef FGC_MORTON_KEYS
    // sub-cell coordinates -> transposed Hilbert index (Skilling's in-place transform: undo the excess work of
    // the Gray code from the most significant level down, then Gray-encode), so that interleaving the bits
    // below yields the position along a Hilbert curve through the bin's sub-cells
    if (sub_bits > 1) {
        const int top = 1 << (sub_bits - 1);
        for (int q = top; q > 1; q >>= 1) {
            const int p = q - 1;
#pragma unroll
            for (int d = 0; d < FGC_MAX_BIN_DIMS; d++) {
                if (d < nbd) {
                    if (sub[d] & q) sub[0] ^= p;
                    else { const int t = (sub[0] ^ sub[d]) & p; sub[0] ^= t; sub[d] ^= t; }
                }
            }
        }
#pragma unroll
        for (int d = 1; d < FGC_MAX_BIN_DIMS; d++)
            if (d < nbd) sub[d] ^= sub[d - 1];
        int last = sub[0];
#pragma unroll
        for (int d = 1; d < FGC_MAX_BIN_DIMS; d++)
            if (d < nbd) last = sub[d];
        int t = 0;
        for (int q = top; q > 1; q >>= 1)
            if (last & q) t ^= q - 1;
#pragma unroll
        for (int d = 0; d < FGC_MAX_BIN_DIMS; d++)
            if (d < nbd) sub[d] ^= t;
    }
#endif
    uint32_t code = 0;
    for (int l = sub_bits - 1; l >= 0; l--)
#pragma unroll
        for (int d = 0; d < FGC_MAX_BIN_DIMS; d++)
            if (d < nbd) code = (code << 1) | (uint32_t)((sub[d] >> l) & 1);
    return (f << (sub_bits * nbd)) | code;
}

__global__ __launch_bounds__(256) void k_bin_keys(const float *__restrict__ coords, int n, int ld, int nbd,
                                                  int sub_bits, const float *__restrict__ geom,
                                                  const int64_t *__restrict__ rs, int n_rs,
                                                  uint32_t *__restrict__ keys, int *__restrict__ status)
{
    int v = blockIdx.x * blockDim.x + threadIdx.x;
    if (v >= n) return;
    BinGeom g = load_geom(geom);
    int clamped = 0;
    keys[v] = knn_sort_key(coords + (int64_t)v * ld, g, nbd, sub_bits, event_of(rs, n_rs, v), clamped);
    if (clamped && status) atomicOr(&status[0], FGC_ST_CLAMPED);
}

// ---------------------------------------------------------------------------
// LSD radix sort, 8-bit digits, stable.  Tile = 4 waves x CH chunks x 64 keys; the passes are short and bound by
// latency, so small tiles (many blocks in flight) win: CH = 4 up to RS_SMALL_N keys, 8 beyond (1 M keys: 16 chunks
// 0.209 ms for the whole preparation stage, 8 chunks 0.193, 4 chunks 0.202; 200 k keys: 0.124 / 0.094 / 0.082;
// with the tile put into digit order in LDS before it is written: 8 chunks 0.179, 16 chunks 0.211).
// ---------------------------------------------------------------------------
#define RS_MIN_TILE (256 * 4)
#define RS_SMALL_N 700000
#ifndef RS_BIG_CH
#define RS_BIG_CH 8
#endif

// lanes of this wave holding the same digit (valid lanes only)
__device__ __forceinline__ unsigned long long match_digit(int digit, bool valid)
{
    unsigned long long m = fgc_ballot(valid);
#pragma unroll
    for (int b = 0; b < 8; b++) {
        unsigned long long s = fgc_ballot(valid && ((digit >> b) & 1));
        m &= ((digit >> b) & 1) ? s : ~s;
    }
    return m;
}

// block_hist is digit-major: block_hist[digit * nblk + blk]
template <int RS_CHUNKS>
__global__ __launch_bounds__(256) void k_rs_hist(const uint32_t *__restrict__ keys, int n, int shift,
                                                 int nblk, uint32_t *__restrict__ block_hist)
{
    constexpr int RS_TILE = 256 * RS_CHUNKS;
    __shared__ uint32_t s_h[256];
    s_h[threadIdx.x] = 0;
    __syncthreads();
    const int base = blockIdx.x * RS_TILE;
#pragma unroll 4
    for (int c = 0; c < RS_CHUNKS; c++) {
        int i = base + c * 256 + threadIdx.x;
        if (i < n) atomicAdd(&s_h[(keys[i] >> shift) & 255u], 1u);
    }
    __syncthreads();
    block_hist[threadIdx.x * nblk + blockIdx.x] = s_h[threadIdx.x];
}

// exclusive scan of every digit's row of per-block counts (one block per digit, in place);
// digit_total[digit] receives the row sum
__global__ __launch_bounds__(256) void k_rs_scan_rows(uint32_t *__restrict__ block_hist, int nblk,
                                                      uint32_t *__restrict__ digit_total)
{
    __shared__ uint32_t s_w[4];
    __shared__ uint32_t s_carry;
    uint32_t *row = block_hist + (size_t)blockIdx.x * nblk;
    const int t = threadIdx.x, lane = t & 63, wv = t >> 6;
    if (t == 0) s_carry = 0;
    __syncthreads();
    for (int base = 0; base < nblk; base += 256) {
        const int i = base + t;
        const uint32_t v = (i < nblk) ? row[i] : 0u;
        uint32_t incl = v;
        for (int o = 1; o < 64; o <<= 1) {
            uint32_t u = __shfl_up(incl, o, 64);
            if (lane >= o) incl += u;
        }
        if (lane == 63) s_w[wv] = incl;
        __syncthreads();
        uint32_t off = s_carry;
        for (int w = 0; w < wv; w++) off += s_w[w];
        if (i < nblk) row[i] = off + incl - v;
        __syncthreads();
        if (t == 255) s_carry = off + incl;
        __syncthreads();
    }
    if (t == 0) digit_total[blockIdx.x] = s_carry;
}

template <int RS_CHUNKS>
__global__ __launch_bounds__(256) void k_rs_scatter(const uint32_t *__restrict__ keys_in,
                                                    const uint32_t *__restrict__ vals_in,
                                                    uint32_t *__restrict__ keys_out,
                                                    uint32_t *__restrict__ vals_out, int n, int shift,
                                                    int nblk, const uint32_t *__restrict__ block_hist,
                                                    const uint32_t *__restrict__ digit_total)
{
    constexpr int RS_TILE = 256 * RS_CHUNKS;
    __shared__ uint32_t s_cnt[4][256];
    __shared__ uint32_t s_dig[256];   // exclusive scan of the digit totals
    {
        __shared__ uint32_t s_ws[4];
        const int t = threadIdx.x, ln = t & 63, w = t >> 6;
        const uint32_t v = digit_total[t];
        uint32_t incl = v;
        for (int o = 1; o < 64; o <<= 1) {
            uint32_t u = __shfl_up(incl, o, 64);
            if (ln >= o) incl += u;
        }
        __shared__ int s_const;
        if (t == 0) s_const = 0;
        if (ln == 63) s_ws[w] = incl;
        __syncthreads();
        uint32_t off = 0;
        for (int k = 0; k < w; k++) off += s_ws[k];
        s_dig[t] = off + incl - v;
        if (v == (uint32_t)n) s_const = 1;      // every key has this digit: the pass is the identity
        __syncthreads();
        if (s_const) {
            for (int i = blockIdx.x * RS_TILE + t; i < min(n, (int)(blockIdx.x + 1) * RS_TILE); i += 256) {
                keys_out[i] = keys_in[i];
                vals_out[i] = vals_in ? vals_in[i] : (uint32_t)i;
            }
            return;
        }
    }
    const int lane = fgc_lane(), wv = threadIdx.x >> 6;
    volatile uint32_t *cnt = s_cnt[wv];
    for (int i = lane; i < 256; i += 64) cnt[i] = 0;
    const int base = blockIdx.x * RS_TILE + wv * (RS_TILE / 4);
    uint32_t key[RS_CHUNKS];
    // pass 1: per-wave digit counts
#pragma unroll
    for (int c = 0; c < RS_CHUNKS; c++) {
        int i = base + c * 64 + lane;
        bool valid = i < n;
        key[c] = valid ? keys_in[i] : 0u;
        int digit = (int)((key[c] >> shift) & 255u);
        unsigned long long m = match_digit(digit, valid);
        if (valid && fgc_mbcnt(m) == 0) cnt[digit] = cnt[digit] + (uint32_t)__popcll(m);
    }
    __syncthreads();
    // The tile is first put into digit order inside LDS and then written out position by position: keys of one digit
    // leave as one contiguous run instead of one scattered 4-byte write each.  Per digit: its start inside the
    // tile (exclusive scan of the block's digit counts), the running offsets of the four waves on top of that, and
    // the global position of its first key minus that start.
    __shared__ uint32_t s_key[RS_TILE], s_val[RS_TILE];
    __shared__ uint32_t s_gbase[256];
    {
        __shared__ uint32_t s_ws2[4];
        const int t = threadIdx.x;
        const uint32_t c0 = s_cnt[0][t], c1 = s_cnt[1][t], c2 = s_cnt[2][t], c3 = s_cnt[3][t];
        const uint32_t tot = c0 + c1 + c2 + c3;
        uint32_t incl = tot;
        for (int o = 1; o < 64; o <<= 1) {
            uint32_t u = __shfl_up(incl, o, 64);
            if (lane >= o) incl += u;
        }
        if (lane == 63) s_ws2[wv] = incl;
        __syncthreads();
        uint32_t loc = incl - tot;
        for (int k = 0; k < wv; k++) loc += s_ws2[k];
        s_gbase[t] = s_dig[t] + block_hist[t * nblk + blockIdx.x] - loc;
        s_cnt[0][t] = loc; s_cnt[1][t] = loc + c0; s_cnt[2][t] = loc + c0 + c1; s_cnt[3][t] = loc + c0 + c1 + c2;
    }
    __syncthreads();
    // pass 2: same order, running offsets -> stable
#pragma unroll
    for (int c = 0; c < RS_CHUNKS; c++) {
        int i = base + c * 64 + lane;
        bool valid = i < n;
        int digit = (int)((key[c] >> shift) & 255u);
        unsigned long long m = match_digit(digit, valid);
        int rank = fgc_mbcnt(m);
        uint32_t off = valid ? cnt[digit] : 0u;
        if (valid && rank == 0) cnt[digit] = off + (uint32_t)__popcll(m);
        if (valid) {
            s_key[off + (uint32_t)rank] = key[c];
            s_val[off + (uint32_t)rank] = vals_in ? vals_in[i] : (uint32_t)i;
        }
    }
    __syncthreads();
    const int n_tile = min(RS_TILE, n - (int)blockIdx.x * RS_TILE);
    for (int i = threadIdx.x; i < n_tile; i += 256) {
        const uint32_t k = s_key[i];
        const uint32_t pos = s_gbase[(k >> shift) & 255u] + (uint32_t)i;
        keys_out[pos] = k;
        vals_out[pos] = s_val[i];
    }
}

size_t fgc_sort_workspace_bytes(int64_t n)
{
    int64_t nblk = fgc_cdiv(n > 0 ? n : 1, RS_MIN_TILE);   // the smallest tile has the most blocks
    if (n <= 32768) nblk *= 3;                             // three digit tables of the one-launch passes
    return fgc_align((size_t)n * 4) * 2 /* ping-pong keys / vals */ + fgc_align((size_t)nblk * 256 * 4) +
           fgc_align(256 * 4) /* digit totals */;
}

// Sorts (keys, vals) stably by the low `key_bits` bits; vals start as the identity unless
// `vals_given`.  On return *keys_sorted / *vals_sorted point at the buffers holding the result
// (either the caller's primary pair or the alternates inside the workspace).
int fgc_sort_keys(uint32_t *keys, uint32_t *vals, int64_t n, int key_bits, void *d_ws, hipStream_t s,
                  uint32_t **keys_sorted, uint32_t **vals_sorted, bool vals_given)
{
    if (n >= (1ll << 31)) return FGC_EINVAL;
    char *w = (char *)d_ws;
    uint32_t *k_alt = (uint32_t *)w; w += fgc_align((size_t)n * 4);
    uint32_t *v_alt = (uint32_t *)w; w += fgc_align((size_t)n * 4);
    uint32_t *hist = (uint32_t *)w;
    const bool small = n <= RS_SMALL_N;
    const int nblk = (int)fgc_cdiv(n, small ? 256 * 4 : 256 * RS_BIG_CH);
    uint32_t *digit_total = (uint32_t *)(w + fgc_align((size_t)fgc_cdiv(n > 0 ? n : 1, RS_MIN_TILE) * 256 * 4));
    if ((int64_t)fgc_cdiv(n, RS_MIN_TILE) * 256 >= (1ll << 31)) return FGC_EINVAL;
    uint32_t *kin = keys, *vin = vals_given ? vals : nullptr, *kout = k_alt, *vout = v_alt;
    int passes = (key_bits + 7) / 8;
    if (passes < 1) passes = 1;
    for (int p = 0; p < passes; p++) {
        int shift = p * 8;
        if (small) hipLaunchKernelGGL(k_rs_hist<4>, dim3(nblk), dim3(256), 0, s, kin, (int)n, shift, nblk, hist);
        else hipLaunchKernelGGL(k_rs_hist<RS_BIG_CH>, dim3(nblk), dim3(256), 0, s, kin, (int)n, shift, nblk, hist);
        FGC_LAUNCH_CHECK();
        hipLaunchKernelGGL(k_rs_scan_rows, dim3(256), dim3(256), 0, s, hist, nblk, digit_total);
        FGC_LAUNCH_CHECK();
        if (small)
            hipLaunchKernelGGL(k_rs_scatter<4>, dim3(nblk), dim3(256), 0, s, kin, vin, kout, vout, (int)n, shift,
                               nblk, hist, digit_total);
        else
            hipLaunchKernelGGL(k_rs_scatter<RS_BIG_CH>, dim3(nblk), dim3(256), 0, s, kin, vin, kout, vout, (int)n, shift,
                               nblk, hist, digit_total);
        FGC_LAUNCH_CHECK();
        kin = kout; vin = vout;
        if (kout == k_alt) { kout = keys; vout = vals; } else { kout = k_alt; vout = v_alt; }
    }
    *keys_sorted = kin;
    *vals_sorted = vin;
    return FGC_OK;
}

int fgc_launch_bin_keys(const float *d_coords, int n, int ld, int nbd, int sub_bits, const float *d_geom,
                        const int64_t *d_rs, int n_rs, uint32_t *d_keys, int *d_status, hipStream_t s)
{
    hipLaunchKernelGGL(k_bin_keys, dim3((unsigned)fgc_cdiv(n, 256)), dim3(256), 0, s, d_coords, n, ld, nbd,
                       sub_bits, d_geom, d_rs, n_rs, d_keys, d_status);
    FGC_LAUNCH_CHECK();
    return FGC_OK;
}

// ---------------------------------------------------------------------------
// Up to FS_MAX_N points (a few dozen tiles) the sort needs ONE launch per pass instead of three, and the geometry record none of its
// own: launches of a few microseconds each otherwise dominate the preparation of a few thousand points - the
// typical event of the reference's tests.
//   * k_bin_keys_geom: every block reduces the range partials itself (a few hundred records) and derives the
//     geometry record in LDS (block 0 also stores it); it adds its keys' lowest digits to the first digit table.
//   * k_rs_pass: a digit table holds, tile by tile, how many keys of the tile have each digit (table[tile][digit]).
//     Every block sums the table's rows itself - the rows before its own tile and all of them - instead of reading
//     a scan another launch made; while it writes a key to its sorted position it adds the key's NEXT digit to
//     the next pass's table at the tile that position lies in; and it clears its row of a third table for the pass
//     after that.  Integer atomic adds only: the tables, hence the order, do not depend on timing.
// No block waits for another inside a launch.
// ---------------------------------------------------------------------------
#define FS_MAX_N 32768
#define FS_CH 4
#define FS_TILE (256 * FS_CH)
#define FS_TILE_SHIFT 10

__global__ __launch_bounds__(256) void k_bin_keys_geom(const float *__restrict__ coords, int n, int ld, int nbd,
                                                       int sub_bits, const float *__restrict__ partial, int npart,
                                                       int nb0, int nb1, int nb2, int nb3, int nb4,
                                                       float *__restrict__ geom_out, const int64_t *__restrict__ rs,
                                                       int n_rs, uint32_t *__restrict__ keys,
                                                       int *__restrict__ status, uint32_t *__restrict__ table0)
{
    __shared__ float s_red[4][11];
    __shared__ float s_geom[FGC_GEOM_FLOATS];
    __shared__ uint32_t s_h[256];
    const int t = threadIdx.x, lane = fgc_lane(), wv = t >> 6;
    // this thread's point and its event first: the loads travel while the geometry record is made
    const int v = blockIdx.x * 256 + t;
    float x[FGC_MAX_BIN_DIMS];
#pragma unroll
    for (int d = 0; d < FGC_MAX_BIN_DIMS; d++) x[d] = (v < n && d < nbd) ? coords[(int64_t)v * ld + d] : 0.f;
    const int ev = v < n ? event_of(rs, n_rs, v) : 0;
    {
        float mn[FGC_MAX_BIN_DIMS], mx[FGC_MAX_BIN_DIMS];
        float bad = 0.f;
#pragma unroll
        for (int d = 0; d < FGC_MAX_BIN_DIMS; d++) { mn[d] = INFINITY; mx[d] = -INFINITY; }
        for (int b = t; b < npart; b += 256) {
#pragma unroll
            for (int d = 0; d < FGC_MAX_BIN_DIMS; d++) {
                mn[d] = fminf(mn[d], partial[b * 11 + d]);
                mx[d] = fmaxf(mx[d], partial[b * 11 + 5 + d]);
            }
            bad = fmaxf(bad, partial[b * 11 + 10]);
        }
#pragma unroll
        for (int d = 0; d < FGC_MAX_BIN_DIMS; d++) {
            const float a = wave_min_f(mn[d]), b = wave_max_f(mx[d]);
            if (lane == 0) { s_red[wv][d] = a; s_red[wv][5 + d] = b; }
        }
        bad = wave_max_f(bad);
        if (lane == 0) s_red[wv][10] = bad;
        s_h[t] = 0;
        __syncthreads();
        if (t == 0) {
#pragma unroll
            for (int d = 0; d < FGC_MAX_BIN_DIMS; d++) {
                mn[d] = fminf(fminf(s_red[0][d], s_red[1][d]), fminf(s_red[2][d], s_red[3][d]));
                mx[d] = fmaxf(fmaxf(s_red[0][5 + d], s_red[1][5 + d]), fmaxf(s_red[2][5 + d], s_red[3][5 + d]));
            }
            bad = fmaxf(fmaxf(s_red[0][10], s_red[1][10]), fmaxf(s_red[2][10], s_red[3][10]));
            const int nb_in[FGC_MAX_BIN_DIMS] = {nb0, nb1, nb2, nb3, nb4};
            geometry_record(mn, mx, bad > 0.f, nbd, 2, 1, 0.f, 0, nb_in, s_geom, blockIdx.x == 0 ? status : nullptr);
            if (blockIdx.x == 0)
                for (int d = 0; d < FGC_GEOM_FLOATS; d++) geom_out[d] = s_geom[d];
        }
        __syncthreads();
    }
    if (v < n) {
        const BinGeom g = load_geom(s_geom);
        int clamped = 0;
        const uint32_t key = knn_sort_key(x, g, nbd, sub_bits, ev, clamped);
        keys[v] = key;
        if (clamped && status) atomicOr(&status[0], FGC_ST_CLAMPED);
        atomicAdd(&s_h[key & 255u], 1u);
    }
    __syncthreads();
    // the 256 keys of a block lie in one tile of the sort
    if (s_h[t]) atomicAdd(&table0[(size_t)((blockIdx.x * 256) >> FS_TILE_SHIFT) * 256 + t], s_h[t]);
}

__global__ __launch_bounds__(256) void k_rs_pass(const uint32_t *__restrict__ keys_in,
                                                 const uint32_t *__restrict__ vals_in, uint32_t *__restrict__ keys_out,
                                                 uint32_t *__restrict__ vals_out, int n, int shift, int nblk,
                                                 const uint32_t *__restrict__ table, uint32_t *__restrict__ table_next,
                                                 uint32_t *__restrict__ table_clear)
{
    __shared__ uint32_t s_cnt[4][256];
    __shared__ uint32_t s_gbase[256];
    __shared__ uint32_t s_ws[4], s_ws2[4];
    __shared__ int s_const;
    __shared__ uint32_t s_key[FS_TILE], s_val[FS_TILE];
    const int t = threadIdx.x, lane = fgc_lane(), wv = t >> 6, blk = blockIdx.x;
    if (table_clear) table_clear[(size_t)blk * 256 + t] = 0u;
    const int tile0 = blk * FS_TILE;
    const int n_tile = min(FS_TILE, n - tile0);
    const int next_shift = shift + 8;
    const int base = tile0 + wv * (FS_TILE / 4);
    uint32_t key[FS_CH], val[FS_CH];
#pragma unroll
    for (int c = 0; c < FS_CH; c++) {
        const int i = base + c * 64 + lane;
        key[c] = i < n ? keys_in[i] : 0u;
        val[c] = i < n ? (vals_in ? vals_in[i] : (uint32_t)i) : 0u;
    }
    // digit t: keys in the tiles before this one, keys in all tiles
    uint32_t before = 0, total = 0;
    {
        int b = 0;
        for (; b + 16 <= nblk; b += 16) {
            uint32_t c[16];
#pragma unroll
            for (int k = 0; k < 16; k++) c[k] = table[(size_t)(b + k) * 256 + t];
#pragma unroll
            for (int k = 0; k < 16; k++) { total += c[k]; before += (b + k < blk) ? c[k] : 0u; }
        }
        uint32_t c[16];
#pragma unroll
        for (int k = 0; k < 16; k++) c[k] = b + k < nblk ? table[(size_t)(b + k) * 256 + t] : 0u;
#pragma unroll
        for (int k = 0; k < 16; k++) { total += c[k]; before += (b + k < blk) ? c[k] : 0u; }
    }
    uint32_t incl = total;
    for (int o = 1; o < 64; o <<= 1) {
        const uint32_t u = __shfl_up(incl, o, 64);
        if (lane >= o) incl += u;
    }
    if (t == 0) s_const = 0;
    if (lane == 63) s_ws[wv] = incl;
    __syncthreads();
    uint32_t first = incl - total;                 // sorted position of the first key with digit t
    for (int k = 0; k < wv; k++) first += s_ws[k];
    if (total == (uint32_t)n) s_const = 1;         // every key has this digit: the pass is the identity
    volatile uint32_t *cnt = s_cnt[wv];
    for (int i = lane; i < 256; i += 64) cnt[i] = 0;
    __syncthreads();
    if (s_const) {
        for (int c = 0; c < FS_CH; c++) {
            const int i = base + c * 64 + lane;
            const bool valid = i < n;
            if (valid) { keys_out[i] = key[c]; vals_out[i] = val[c]; }
            if (table_next) {
                const int nd = (int)((key[c] >> next_shift) & 255u);
                const unsigned long long m = match_digit(nd, valid);
                if (valid && fgc_mbcnt(m) == 0) atomicAdd(&table_next[(size_t)blk * 256 + nd], (uint32_t)__popcll(m));
            }
        }
        return;
    }
    // per-wavefront digit counts
#pragma unroll
    for (int c = 0; c < FS_CH; c++) {
        const bool valid = base + c * 64 + lane < n;
        const int digit = (int)((key[c] >> shift) & 255u);
        const unsigned long long m = match_digit(digit, valid);
        if (valid && fgc_mbcnt(m) == 0) cnt[digit] = cnt[digit] + (uint32_t)__popcll(m);
    }
    __syncthreads();
    // the tile in digit order inside LDS: start of every digit inside the tile, the running offsets of the four
    // wavefronts on top of that, and the sorted position of the digit's first key of this tile minus that start
    {
        const uint32_t c0 = s_cnt[0][t], c1 = s_cnt[1][t], c2 = s_cnt[2][t], c3 = s_cnt[3][t];
        const uint32_t tot = c0 + c1 + c2 + c3;
        uint32_t in2 = tot;
        for (int o = 1; o < 64; o <<= 1) {
            const uint32_t u = __shfl_up(in2, o, 64);
            if (lane >= o) in2 += u;
        }
        if (lane == 63) s_ws2[wv] = in2;
        __syncthreads();
        uint32_t loc = in2 - tot;
        for (int k = 0; k < wv; k++) loc += s_ws2[k];
        s_gbase[t] = first + before - loc;
        s_cnt[0][t] = loc; s_cnt[1][t] = loc + c0; s_cnt[2][t] = loc + c0 + c1; s_cnt[3][t] = loc + c0 + c1 + c2;
    }
    __syncthreads();
#pragma unroll
    for (int c = 0; c < FS_CH; c++) {
        const bool valid = base + c * 64 + lane < n;
        const int digit = (int)((key[c] >> shift) & 255u);
        const unsigned long long m = match_digit(digit, valid);
        const int rank = fgc_mbcnt(m);
        const uint32_t off = valid ? cnt[digit] : 0u;
        if (valid && rank == 0) cnt[digit] = off + (uint32_t)__popcll(m);
        if (valid) { s_key[off + (uint32_t)rank] = key[c]; s_val[off + (uint32_t)rank] = val[c]; }
    }
    __syncthreads();
    for (int i = t; i < FS_TILE; i += 256) {
        const bool valid = i < n_tile;
        const uint32_t k = valid ? s_key[i] : 0u;
        const uint32_t pos = valid ? s_gbase[(k >> shift) & 255u] + (uint32_t)i : 0u;
        if (valid) { keys_out[pos] = k; vals_out[pos] = s_val[i]; }
        if (table_next) {
            // one add per (tile, digit) of the wavefront where its keys land in one tile (the usual case: a run of
            // one digit), one per key otherwise
            const int nd = (int)((k >> next_shift) & 255u);
            const uint32_t dst = pos >> FS_TILE_SHIFT;
            const bool mine = valid && dst == (uint32_t)__builtin_amdgcn_readfirstlane((int)dst);
            const unsigned long long m = match_digit(nd, mine);
            if (mine) {
                if (fgc_mbcnt(m) == 0) atomicAdd(&table_next[(size_t)dst * 256 + nd], (uint32_t)__popcll(m));
            } else if (valid) atomicAdd(&table_next[(size_t)dst * 256 + nd], 1u);
        }
    }
}

bool fgc_sort_fused_fits(int64_t n) { return n > 0 && n <= FS_MAX_N; }

// range + geometry + keys + sort of a small input: 2 + passes launches.  `partial` as in fgc_bin_geometry_f32's
// workspace, `d_sort_ws` as for fgc_sort_keys.
int fgc_keys_and_sort_fused(const float *coords, int n, int ld, int nbd, const int64_t *n_bins, int sub_bits,
                            int key_bits, const int64_t *rs, int n_rs, float *partial, float *geom, uint32_t *keys,
                            uint32_t *vals, void *d_sort_ws, int *status, hipStream_t s, uint32_t **keys_sorted,
                            uint32_t **vals_sorted)
{
    int nb[FGC_MAX_BIN_DIMS] = {1, 1, 1, 1, 1};
    for (int d = 0; d < nbd; d++) {
        if (n_bins[d] > 0x7fffffff) return FGC_EINVAL;
        nb[d] = (int)n_bins[d];
    }
    char *w = (char *)d_sort_ws;
    uint32_t *k_alt = (uint32_t *)w; w += fgc_align((size_t)n * 4);
    uint32_t *v_alt = (uint32_t *)w; w += fgc_align((size_t)n * 4);
    const int nblk = (int)fgc_cdiv(n, FS_TILE);
    uint32_t *tab[3] = {(uint32_t *)w, (uint32_t *)w + (size_t)nblk * 256, (uint32_t *)w + (size_t)nblk * 512};
    int npart = (int)fgc_cdiv(n, 256 * 4);
    if (npart > RANGE_BLOCKS_MAX) npart = RANGE_BLOCKS_MAX;
    hipLaunchKernelGGL(k_range_partial, dim3(npart), dim3(256), 0, s, coords, (int64_t)n, ld, nbd, partial, tab[0],
                       nblk * 512);
    FGC_LAUNCH_CHECK();
    hipLaunchKernelGGL(k_bin_keys_geom, dim3((unsigned)fgc_cdiv(n, 256)), dim3(256), 0, s, coords, n, ld, nbd, sub_bits,
                       partial, npart, nb[0], nb[1], nb[2], nb[3], nb[4], geom, rs, n_rs, keys, status, tab[0]);
    FGC_LAUNCH_CHECK();
    uint32_t *kin = keys, *vin = nullptr, *kout = k_alt, *vout = v_alt;
    int passes = (key_bits + 7) / 8;
    if (passes < 1) passes = 1;
    for (int p = 0; p < passes; p++) {
        hipLaunchKernelGGL(k_rs_pass, dim3(nblk), dim3(256), 0, s, kin, vin, kout, vout, n, p * 8, nblk, tab[p % 3],
                           p + 1 < passes ? tab[(p + 1) % 3] : (uint32_t *)nullptr,
                           p + 2 < passes ? tab[(p + 2) % 3] : (uint32_t *)nullptr);
        FGC_LAUNCH_CHECK();
        kin = kout; vin = vout;
        if (kout == k_alt) { kout = keys; vout = vals; } else { kout = k_alt; vout = v_alt; }
    }
    *keys_sorted = kin;
    *vals_sorted = vin;
    return FGC_OK;
}

// ---------------------------------------------------------------------------
// The tail of the preparation in one launch: sorted coordinates (structure of arrays, optionally also as rows of 8
// floats), direction flags, the bounding boxes of the chunks and of the groups of 64 chunks, and the bin
// boundaries.  One block of 16 wavefronts per group of 64 chunks: wavefront w gathers chunks 4 w .. 4 w + 3 of the
// group (lane = point; the loads of all four requested before the first is used) and reduces their boxes, the block
// combines them into the group's box through LDS.  Bin boundaries (bb[b] = first sorted position whose bin is
// >= b) from the same positions: where the bin changes between positions i - 1 and i, position i is the boundary
// of every bin in between.
// ---------------------------------------------------------------------------
template <int DT>   // DT = D where the gather is unrolled for it, 0 = any D
__global__ __launch_bounds__(1024) void k_prepare_tail(const float *__restrict__ coords, int ld_in,
                                                       const uint32_t *__restrict__ order,
                                                       const uint32_t *__restrict__ skeys, int n, int D_rt, int ldc,
                                                       float *__restrict__ sc, const int64_t *__restrict__ direction,
                                                       unsigned char *__restrict__ sdir, float4 *__restrict__ sp,
                                                       int sp_half, float *__restrict__ box_lo,
                                                       float *__restrict__ box_hi, float *__restrict__ sbox_lo,
                                                       float *__restrict__ sbox_hi, int key_shift, int n_bins_total,
                                                       int *__restrict__ bb, unsigned *__restrict__ zero2)
{
    __shared__ float s_lo[16][16], s_hi[16][16];
    if (zero2 && blockIdx.x == 0 && threadIdx.x < 2) zero2[threadIdx.x] = 0u;   // counters of the kernel that follows
    const int D = DT ? DT : D_rt;
    const int lane = fgc_lane(), wv = threadIdx.x >> 6;
    const int n_chunks = ldc / 64, n_super = (n_chunks + 63) / 64;
    const int g = blockIdx.x;                 // group of 64 chunks
    const int c0 = g * 64 + wv * 4;
    uint32_t o[4], key[4], keyp[4];
    int64_t dirv[4];
#pragma unroll
    for (int cc = 0; cc < 4; cc++) {
        const int i = (c0 + cc) * 64 + lane;
        o[cc] = i < n ? order[i] : 0u;
        key[cc] = i < n ? skeys[i] : 0u;
        keyp[cc] = (i <= n && i > 0) ? skeys[i - 1] : 0u;
    }
    if (sdir) {
#pragma unroll
        for (int cc = 0; cc < 4; cc++) dirv[cc] = (c0 + cc) * 64 + lane < n ? direction[o[cc]] : 0;
    }
    float glo[16], ghi[16];                   // this wavefront's share of the group's box, coordinate d in slot d (d < 16)
#pragma unroll
    for (int d = 0; d < 16; d++) { glo[d] = INFINITY; ghi[d] = -INFINITY; }
    if (DT) {
        float x[4][DT ? DT : 1];
#pragma unroll
        for (int cc = 0; cc < 4; cc++)
#pragma unroll
            for (int d = 0; d < DT; d++) x[cc][d] = (c0 + cc) * 64 + lane < n ? coords[(int64_t)o[cc] * ld_in + d] : 0.f;
#pragma unroll
        for (int cc = 0; cc < 4; cc++) {
            const int c = c0 + cc, i = c * 64 + lane;
            if (c >= n_chunks) break;
            const bool in = i < n;
            float r[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int d = 0; d < DT; d++) {
                if (in) sc[(int64_t)d * ldc + i] = x[cc][d];
                if (d < 2 * sp_half) r[d < sp_half ? d : 4 + d - sp_half] = x[cc][d];
                const float lo = wave_min_f(in ? x[cc][d] : INFINITY), hi = wave_max_f(in ? x[cc][d] : -INFINITY);
                if (lane == 0) { box_lo[(size_t)d * n_chunks + c] = lo; box_hi[(size_t)d * n_chunks + c] = hi; }
                if (d < 16) { glo[d] = fminf(glo[d], lo); ghi[d] = fmaxf(ghi[d], hi); }
            }
            if (sp) {
                sp[(int64_t)i * 2] = make_float4(r[0], r[1], r[2], r[3]);
                sp[(int64_t)i * 2 + 1] = make_float4(r[4], r[5], r[6], r[7]);
            }
        }
    } else {
        for (int cc = 0; cc < 4; cc++) {
            const int c = c0 + cc, i = c * 64 + lane;
            if (c >= n_chunks) break;
            const bool in = i < n;
            float r[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
            for (int d = 0; d < D; d++) {
                const float x = in ? coords[(int64_t)o[cc] * ld_in + d] : 0.f;
                if (in) sc[(int64_t)d * ldc + i] = x;
                if (d < 2 * sp_half) r[d < sp_half ? d : 4 + d - sp_half] = x;
                const float lo = wave_min_f(in ? x : INFINITY), hi = wave_max_f(in ? x : -INFINITY);
                if (lane == 0) { box_lo[(size_t)d * n_chunks + c] = lo; box_hi[(size_t)d * n_chunks + c] = hi; }
                if (d < 16) { glo[d] = fminf(glo[d], lo); ghi[d] = fmaxf(ghi[d], hi); }   // (coordinates 16 and up: below)
            }
            if (sp) {
                sp[(int64_t)i * 2] = make_float4(r[0], r[1], r[2], r[3]);
                sp[(int64_t)i * 2 + 1] = make_float4(r[4], r[5], r[6], r[7]);
            }
        }
    }
#pragma unroll
    for (int cc = 0; cc < 4; cc++) {
        const int i = (c0 + cc) * 64 + lane;
        if (sdir && i < n) sdir[i] = (unsigned char)((dirv[cc] >= 0 && dirv[cc] <= 2) ? dirv[cc] : 3);
        // bin boundaries
        int b_from = 1, b_to = 0;                    // bins b_from .. b_to get the boundary `at`
        int at = i;
        if (i < n) {
            b_from = i > 0 ? (int)(keyp[cc] >> key_shift) + 1 : 0;
            b_to = (int)(key[cc] >> key_shift);
        }
        if (i == n) { b_from = n > 0 ? (int)(keyp[cc] >> key_shift) + 1 : 0; b_to = n_bins_total; at = n; }
        if (b_to > n_bins_total) b_to = n_bins_total;    // (keys are made of valid bins; guards the store all the same)
        // short runs by the lane itself, long ones (empty regions of the grid) by the whole wavefront
        const bool longrun = b_to - b_from >= 8;
        if (!longrun) for (int b = b_from; b <= b_to; b++) bb[b] = at;
        unsigned long long m = fgc_ballot(longrun);
        while (m) {
            const int l = __builtin_ctzll(m);
            m &= m - 1;
            const int f = fgc_readlane_i(b_from, l), t2 = fgc_readlane_i(b_to, l), a = fgc_readlane_i(at, l);
            for (int b = f + lane; b <= t2; b += 64) bb[b] = a;
        }
    }
    if (lane < 16) {
        float lo = INFINITY, hi = -INFINITY;
#pragma unroll
        for (int d = 0; d < 16; d++) if (lane == d) { lo = glo[d]; hi = ghi[d]; }
        s_lo[wv][lane] = lo; s_hi[wv][lane] = hi;
    }
    __syncthreads();
    if (g < n_super && (int)threadIdx.x < min(D, 16)) {
        float lo = INFINITY, hi = -INFINITY;
        for (int w = 0; w < 16; w++) { lo = fminf(lo, s_lo[w][threadIdx.x]); hi = fmaxf(hi, s_hi[w][threadIdx.x]); }
        sbox_lo[(size_t)threadIdx.x * n_super + g] = lo;
        sbox_hi[(size_t)threadIdx.x * n_super + g] = hi;
    }
    if (D > 16 && g < n_super) {
        // coordinates 16 and up (rare): from the chunk boxes this block has just written
        for (int d = 16 + wv; d < D; d += 16) {
            const int c = g * 64 + lane;
            const float lo = wave_min_f(c < n_chunks ? box_lo[(size_t)d * n_chunks + c] : INFINITY);
            const float hi = wave_max_f(c < n_chunks ? box_hi[(size_t)d * n_chunks + c] : -INFINITY);
            if (lane == 0) { sbox_lo[(size_t)d * n_super + g] = lo; sbox_hi[(size_t)d * n_super + g] = hi; }
        }
    }
}

int fgc_launch_prepare_tail(const float *coords, int ld_in, const uint32_t *order, const uint32_t *skeys, int n, int D,
                            int ldc, float *sc, const int64_t *direction, unsigned char *sdir, float *sp, int sp_half,
                            float *box_lo, float *box_hi, float *sbox_lo, float *sbox_hi, int key_shift,
                            int n_bins_total, int *bb, unsigned *zero2, hipStream_t s)
{
    // position n (the end of the last bin's run) must belong to a chunk some wavefront visits
    const int n_super = ((n + 1 + 63) / 64 + 63) / 64;
#define FGC_TAIL(DT)                                                                                                    \
    hipLaunchKernelGGL(k_prepare_tail<DT>, dim3((unsigned)n_super), dim3(1024), 0, s, coords, ld_in, order, skeys, n, D, \
                       ldc, sc, direction, sdir, (float4 *)sp, sp_half, box_lo, box_hi, sbox_lo, sbox_hi, key_shift,   \
                       n_bins_total, bb, zero2)
    switch (D) {
    case 2: FGC_TAIL(2); break;
    case 3: FGC_TAIL(3); break;
    case 4: FGC_TAIL(4); break;
    case 5: FGC_TAIL(5); break;
    case 6: FGC_TAIL(6); break;
    case 8: FGC_TAIL(8); break;
    default: FGC_TAIL(0); break;
    }
#undef FGC_TAIL
    FGC_LAUNCH_CHECK();
    return FGC_OK;
}


