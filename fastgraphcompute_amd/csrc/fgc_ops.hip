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

// ---------------------------------------------------------------------------
// gradient of distsq wrt the coordinates
// ---------------------------------------------------------------------------
// A group of W = 2^w lanes (W >= min(K, 64)) owns one query; lane k of the
// group owns neighbour slot k (K > 64: slots k, k + 64, ...).  The neighbour
// receives +2 g (x_m - x_i) through a float atomic; the query's own
// -2 sum_k g (x_m - x_i) is reduced inside the group first and added with one
// atomic per coordinate.
template <int W>
__global__ __launch_bounds__(256) void k_knn_grad(const float *__restrict__ gd, const int64_t *__restrict__ idx,
                                                  const float *__restrict__ x, float *__restrict__ gx,
                                                  int64_t n, int K, int D, int *__restrict__ status)
{
    constexpr int QPW = 64 / W;  // queries per wave
    const int lane = fgc_lane();
    const int sub = lane / W, kl = lane % W;
    const int64_t wave = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int64_t i = wave * QPW + sub;
    const bool qv = i < n;
    bool bad = false;
    for (int c = 0; c < D; c++) {
        const float xi = qv ? x[i * D + c] : 0.f;
        float self = 0.f;
        for (int k = kl; k < K; k += W) {
            if (!qv) continue;
            const int64_t m = idx[i * K + k];
            if (m < 0) continue;
            if (m >= n) { bad = true; continue; }
            const float g = gd[i * K + k];
            const float add = 2.f * g * (x[m * D + c] - xi);
            self -= add;
            atomicAdd(&gx[m * D + c], add);
        }
#pragma unroll
        for (int o = W / 2; o > 0; o >>= 1) self += __shfl_xor(self, o, 64);
        if (qv && kl == 0) atomicAdd(&gx[i * D + c], self);
    }
    if (bad && status) atomicOr(&status[0], FGC_ST_BAD_INDEX);
}

extern "C" int fgc_binned_select_knn_grad_f32(const float *d_grad_distsq, const int64_t *d_idx,
                                              const float *d_coords, float *d_grad_coords, int64_t n_vert,
                                              int32_t K, int32_t n_coords, int32_t *d_status, void *stream)
{
    if (n_vert < 0 || K < 1 || n_coords < 1) return FGC_EINVAL;
    if (n_vert == 0) return FGC_OK;
    hipStream_t s = (hipStream_t)stream;
    int rc = fgc_fill_u32(d_grad_coords, 0u, n_vert * n_coords, s);
    if (rc) return rc;
    int W = 64;
    while (W > 8 && (W >> 1) >= K) W >>= 1;
    const int qpw = 64 / W;
    const int64_t waves = fgc_cdiv(n_vert, qpw);
    const unsigned blocks = (unsigned)fgc_cdiv(waves, 4);
#define FGC_GRAD_LAUNCH(WW)                                                                              \
    hipLaunchKernelGGL((k_knn_grad<WW>), dim3(blocks), dim3(256), 0, s, d_grad_distsq, d_idx, d_coords, \
                       d_grad_coords, n_vert, (int)K, (int)n_coords, d_status)
    switch (W) {
    case 8: FGC_GRAD_LAUNCH(8); break;
    case 16: FGC_GRAD_LAUNCH(16); break;
    case 32: FGC_GRAD_LAUNCH(32); break;
    default: FGC_GRAD_LAUNCH(64); break;
    }
#undef FGC_GRAD_LAUNCH
    FGC_LAUNCH_CHECK();
    return FGC_OK;
}

// ---------------------------------------------------------------------------
// select_with_default
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void k_select_with_default(const int64_t *__restrict__ idx,
                                                             const float *__restrict__ feat,
                                                             float *__restrict__ out, int64_t n_pairs, int F,
                                                             int64_t n_rows, float dflt)
{
    int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int64_t total = n_pairs * F;
    if (t >= total) return;
    int64_t p = t / F;
    int f = (int)(t - p * F);
    int64_t m = idx[p];
    if (m < 0) m += n_rows;  // torch advanced indexing wraps negative indices other than the -1 default
    out[t] = (idx[p] == -1 || m < 0 || m >= n_rows) ? dflt : feat[m * F + f];
}

extern "C" int fgc_select_with_default_f32(const int64_t *d_idx, const float *d_feat, float *d_out,
                                           int64_t n_vert, int32_t K, int32_t n_feat, int64_t n_feat_rows,
                                           float default_value, void *stream)
{
    if (n_vert < 0 || K < 0 || n_feat < 0) return FGC_EINVAL;
    int64_t total = n_vert * K * n_feat;
    if (total == 0) return FGC_OK;
    hipLaunchKernelGGL(k_select_with_default, dim3((unsigned)fgc_cdiv(total, 256)), dim3(256), 0,
                       (hipStream_t)stream, d_idx, d_feat, d_out, n_vert * K, (int)n_feat, n_feat_rows,
                       default_value);
    FGC_LAUNCH_CHECK();
    return FGC_OK;
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
                                                     const float *__restrict__ feat, float *__restrict__ fmean,
                                                     float *__restrict__ fmax, int *__restrict__ argmax,
                                                     int64_t n, int K, int P)
{
    constexpr int QPW = 64 / PW;
    const int lane = fgc_lane();
    const int sub = lane / PW, pl = lane % PW;
    const int64_t wave = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int64_t i = wave * QPW + sub;
    if (i >= n) return;
    for (int p = pl; p < P; p += PW) {
        float s = 0.f, mx = 0.f;
        int am = 0;
        for (int k = 0; k < K; k++) {
            const int64_t m = idx[i * K + k];
            const float w = expf(-10.f * dsq[i * K + k]);
            const float v = (m == -1 ? 0.f : feat[m * P + p]) * w;
            s += v;
            if (k == 0 || v > mx) { mx = v; am = k; }
        }
        fmean[i * P + p] = s / (float)K;
        fmax[i * P + p] = mx;
        if (argmax) argmax[i * P + p] = am;
    }
}

template <int PW>
__global__ __launch_bounds__(256) void k_gravnet_bwd(const int64_t *__restrict__ idx,
                                                     const float *__restrict__ dsq,
                                                     const float *__restrict__ feat,
                                                     const int *__restrict__ argmax,
                                                     const float *__restrict__ gmean,
                                                     const float *__restrict__ gmax, float *__restrict__ gfeat,
                                                     float *__restrict__ gdsq, int64_t n, int K, int P)
{
    constexpr int QPW = 64 / PW;
    const int lane = fgc_lane();
    const int sub = lane / PW, pl = lane % PW;
    const int64_t wave = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int64_t i = wave * QPW + sub;
    const bool qv = i < n;
    const float invK = 1.0f / (float)K;
    for (int k = 0; k < K; k++) {
        const int64_t m = qv ? idx[i * K + k] : -1;
        const float w = qv ? expf(-10.f * dsq[i * K + k]) : 0.f;
        float gw = 0.f;  // d loss / d w of this (point, slot)
        if (m != -1) {
            for (int p = pl; p < P; p += PW) {
                const float c = gmean[i * P + p] * invK + (argmax[i * P + p] == k ? gmax[i * P + p] : 0.f);
                gw += feat[m * P + p] * c;
                atomicAdd(&gfeat[m * P + p], w * c);
            }
        }
#pragma unroll
        for (int o = PW / 2; o > 0; o >>= 1) gw += __shfl_xor(gw, o, 64);
        if (qv && pl == 0) gdsq[i * K + k] = -10.f * w * gw;
    }
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
    if (n_vert < 0 || K < 1 || P < 1) return FGC_EINVAL;
    if (n_vert == 0) return FGC_OK;
    hipStream_t s = (hipStream_t)stream;
    const int pw = pick_pw(P);
    const unsigned blocks = (unsigned)fgc_cdiv(fgc_cdiv(n_vert, 64 / pw), 4);
#define FGC_L(PWW)                                                                                    \
    hipLaunchKernelGGL((k_gravnet_fwd<PWW>), dim3(blocks), dim3(256), 0, s, d_idx, d_distsq, d_feat, \
                       d_fmean, d_fmax, d_argmax, n_vert, (int)K, (int)P)
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
    if (n_vert < 0 || K < 1 || P < 1) return FGC_EINVAL;
    if (n_vert == 0) return FGC_OK;
    hipStream_t s = (hipStream_t)stream;
    const int pw = pick_pw(P);
    const unsigned blocks = (unsigned)fgc_cdiv(fgc_cdiv(n_vert, 64 / pw), 4);
#define FGC_L(PWW)                                                                                     \
    hipLaunchKernelGGL((k_gravnet_bwd<PWW>), dim3(blocks), dim3(256), 0, s, d_idx, d_distsq, d_feat,  \
                       d_argmax, d_grad_fmean, d_grad_fmax, d_grad_feat, d_grad_distsq, n_vert, (int)K, \
                       (int)P)
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
