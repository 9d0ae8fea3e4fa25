// Weight gradient of a dense layer over a long point list (gfx950, MFMA fp32).
//
//   dW[o, i] = sum_n dY[n, o] * X[n, i]      db[o] = sum_n dY[n, o]
//
// In a GravNet layer O and I are at most a few hundred while n is 10^5..10^6: the output is tiny and the
// reduction runs over the points, the shape on which a tiled library GEMM leaves most of the chip idle (one
// workgroup per output tile).  Here the points are split over many wavefronts; each accumulates a (32 TM) x 64
// block of dW with v_mfma_f32_32x32x2f32 - two points per instruction, the operands read straight from the
// row-major dY and X (lanes 0..31 / 32..63 read 32 consecutive floats of two consecutive rows) - and writes
// its partial block; a second kernel adds the partials in a fixed order, so the result is reproducible.
#include "fgc_common.h"

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int WG_TN = 2;          // 32-wide tiles along I per wavefront
constexpr int WG_UNROLL = 4;      // point pairs in flight

template <int TM>
__global__ __launch_bounds__(256) void k_linear_wgrad(const float *__restrict__ dy, const float *__restrict__ x,
                                                      int64_t n, int O, int I, int groups_i, int n_splits,
                                                      int64_t pts_per_split, float *__restrict__ part_w,
                                                      float *__restrict__ part_b)
{
    const int lane = fgc_lane();
    const int wave = (int)(((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6);
    const int group = wave / n_splits, split = wave - group * n_splits;
    const int go = group / groups_i, gi = group - go * groups_i;
    const int o0 = go * 32 * TM, i0 = gi * 32 * WG_TN;
    if (o0 >= O) return;
    const int col = lane & 31, kk = lane >> 5;
    floatx16 acc[TM][WG_TN];
#pragma unroll
    for (int a = 0; a < TM; a++)
#pragma unroll
        for (int b = 0; b < WG_TN; b++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[a][b][r] = 0.f;
    float bsum[TM];
#pragma unroll
    for (int a = 0; a < TM; a++) bsum[a] = 0.f;
    const int64_t p0 = (int64_t)split * pts_per_split;
    const int64_t p1 = min(n, p0 + pts_per_split);
    bool ov[TM], iv[WG_TN];
#pragma unroll
    for (int a = 0; a < TM; a++) ov[a] = o0 + a * 32 + col < O;
#pragma unroll
    for (int b = 0; b < WG_TN; b++) iv[b] = i0 + b * 32 + col < I;
    for (int64_t p = p0; p < p1; p += 2 * WG_UNROLL) {
        float av[WG_UNROLL][TM], bv[WG_UNROLL][WG_TN];
#pragma unroll
        for (int u = 0; u < WG_UNROLL; u++) {
            const int64_t row = p + 2 * u + kk;
            const bool rv = row < p1;
#pragma unroll
            for (int a = 0; a < TM; a++) av[u][a] = (rv && ov[a]) ? dy[row * O + o0 + a * 32 + col] : 0.f;
#pragma unroll
            for (int b = 0; b < WG_TN; b++) bv[u][b] = (rv && iv[b]) ? x[row * I + i0 + b * 32 + col] : 0.f;
        }
#pragma unroll
        for (int u = 0; u < WG_UNROLL; u++) {
#pragma unroll
            for (int a = 0; a < TM; a++) {
                bsum[a] += av[u][a];
#pragma unroll
                for (int b = 0; b < WG_TN; b++)
                    acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[u][a], bv[u][b], acc[a][b], 0, 0, 0);
            }
        }
    }
    // accumulator layout of the 32x32 result: column = lane % 32, row = 8 * (r / 4) + 4 * (lane / 32) + r % 4
    float *pw = part_w + (int64_t)split * O * I;
#pragma unroll
    for (int a = 0; a < TM; a++)
#pragma unroll
        for (int b = 0; b < WG_TN; b++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int o = o0 + a * 32 + 8 * (r >> 2) + 4 * kk + (r & 3);
                const int i = i0 + b * 32 + col;
                if (o < O && i < I) pw[(int64_t)o * I + i] = acc[a][b][r];
            }
    if (part_b && gi == 0) {
#pragma unroll
        for (int a = 0; a < TM; a++) {
            const float s = bsum[a] + __shfl_xor(bsum[a], 32, 64);
            if (kk == 0 && ov[a]) part_b[(int64_t)split * O + o0 + a * 32 + col] = s;
        }
    }
}

// out[e] = sum over the splits of part[s * count + e], for two arrays in one launch (weights: blocks 0 .. blocks_a - 1,
// bias: the blocks after them).  A block owns 64 consecutive outputs; its four wavefronts sum every fourth split
// (eight loads in flight) and the four sums are added in wavefront order: a fixed order, so the result is
// reproducible.
__global__ __launch_bounds__(256) void k_sum_partials(const float *__restrict__ part_a, int64_t count_a,
                                                      float *__restrict__ out_a, int blocks_a,
                                                      const float *__restrict__ part_b, int64_t count_b,
                                                      float *__restrict__ out_b, int n_splits)
{
    __shared__ float s_sum[4][64];
    const int lane = fgc_lane(), w = threadIdx.x >> 6;
    const bool second = (int)blockIdx.x >= blocks_a;
    const float *__restrict__ part = second ? part_b : part_a;
    float *__restrict__ out = second ? out_b : out_a;
    const int64_t count = second ? count_b : count_a;
    const int64_t e = (int64_t)(second ? (int)blockIdx.x - blocks_a : (int)blockIdx.x) * 64 + lane;
    float acc[8];
#pragma unroll
    for (int u = 0; u < 8; u++) acc[u] = 0.f;
    if (e < count) {
        for (int k0 = w; k0 < n_splits; k0 += 32) {
#pragma unroll
            for (int u = 0; u < 8; u++) {
                const int k = k0 + 4 * u;
                acc[u] += (k < n_splits) ? part[(int64_t)k * count + e] : 0.f;
            }
        }
    }
    s_sum[w][lane] = ((acc[0] + acc[1]) + (acc[2] + acc[3])) + ((acc[4] + acc[5]) + (acc[6] + acc[7]));
    __syncthreads();
    if (w == 0 && e < count) out[e] = (s_sum[0][lane] + s_sum[1][lane]) + (s_sum[2][lane] + s_sum[3][lane]);
}

struct WgradPlan {
    int tm, groups_o, groups_i, n_splits;
    int64_t pts_per_split;
    size_t part_w, part_b, total;
};

WgradPlan wgrad_plan(int64_t n, int O, int I)
{
    WgradPlan p;
    p.tm = O > 32 ? 2 : 1;
    p.groups_o = (int)fgc_cdiv(O, 32 * p.tm);
    p.groups_i = (int)fgc_cdiv(I, 32 * WG_TN);
    const int groups = p.groups_o * p.groups_i;
    int64_t splits = 1024 / groups;                          // about one wavefront per SIMD over the chip
    const int64_t max_splits = fgc_cdiv(n > 0 ? n : 1, 64);  // at least 64 points per wavefront
    if (splits > max_splits) splits = max_splits;
    if (splits < 1) splits = 1;
    int64_t pps = fgc_cdiv(n > 0 ? n : 1, splits);
    pps = (pps + 2 * WG_UNROLL - 1) / (2 * WG_UNROLL) * (2 * WG_UNROLL);
    p.pts_per_split = pps;
    p.n_splits = (int)fgc_cdiv(n > 0 ? n : 1, pps);
    p.part_w = 0;
    p.part_b = fgc_align((size_t)p.n_splits * O * I * 4);
    p.total = p.part_b + fgc_align((size_t)p.n_splits * O * 4);
    return p;
}

}  // namespace

extern "C" size_t fgc_linear_wgrad_workspace_bytes(int64_t n, int32_t n_out, int32_t n_in)
{
    if (n < 0 || n_out < 1 || n_in < 1) return 0;
    return wgrad_plan(n, n_out, n_in).total;
}

extern "C" int fgc_linear_wgrad_f32(const float *d_grad_out, const float *d_input, int64_t n, int32_t n_out,
                                    int32_t n_in, float *d_grad_weight, float *d_grad_bias, void *d_ws,
                                    size_t ws_bytes, void *stream)
{
    if (n < 0 || n_out < 1 || n_in < 1 || n_out > 4096 || n_in > 4096 || !d_grad_weight) return FGC_EINVAL;
    hipStream_t s = (hipStream_t)stream;
    if (n == 0) {
        int rc = fgc_fill_u32(d_grad_weight, 0u, (int64_t)n_out * n_in, s);
        if (rc) return rc;
        return d_grad_bias ? fgc_fill_u32(d_grad_bias, 0u, n_out, s) : FGC_OK;
    }
    if (!d_grad_out || !d_input) return FGC_EINVAL;
    const WgradPlan p = wgrad_plan(n, n_out, n_in);
    if (!d_ws || ws_bytes < p.total) return FGC_ENOSPACE;
    float *part_w = (float *)((char *)d_ws + p.part_w);
    float *part_b = d_grad_bias ? (float *)((char *)d_ws + p.part_b) : nullptr;
    const int64_t waves = (int64_t)p.groups_o * p.groups_i * p.n_splits;
    const dim3 grid((unsigned)fgc_cdiv(waves, 4)), block(256);
    if (p.tm == 2)
        hipLaunchKernelGGL((k_linear_wgrad<2>), grid, block, 0, s, d_grad_out, d_input, n, (int)n_out, (int)n_in,
                           p.groups_i, p.n_splits, p.pts_per_split, part_w, part_b);
    else
        hipLaunchKernelGGL((k_linear_wgrad<1>), grid, block, 0, s, d_grad_out, d_input, n, (int)n_out, (int)n_in,
                           p.groups_i, p.n_splits, p.pts_per_split, part_w, part_b);
    FGC_LAUNCH_CHECK();
    const int64_t cw = (int64_t)n_out * n_in;
    const int blocks_w = (int)fgc_cdiv(cw, 64), blocks_b = d_grad_bias ? (int)fgc_cdiv(n_out, 64) : 0;
    hipLaunchKernelGGL(k_sum_partials, dim3((unsigned)(blocks_w + blocks_b)), block, 0, s, (const float *)part_w, cw,
                       d_grad_weight, blocks_w, (const float *)part_b, (int64_t)n_out, d_grad_bias, p.n_splits);
    FGC_LAUNCH_CHECK();
    return FGC_OK;
}
