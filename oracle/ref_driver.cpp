// C-ABI driver around the reference's own CPU kernels (test infrastructure).
//
// The four functions declared below are defined by the reference's sources
// (bin_by_coordinates_cpu.cpp:102, binned_select_knn_cpu.cpp:211,
// binned_select_knn_grad_cpu.cpp:96, index_replacer_cpu.cpp:28), which
// oracle/build_oracle.py compiles unmodified from the reference checkout.
// This file only wraps caller memory in tensors and copies results out, so
// that the checker can call them through ctypes without registering torch
// ops.  The reference's dispatcher glue and its CUDA twins are not part of
// this build.
#include <torch/torch.h>
#include <cstring>
#include <tuple>

std::tuple<torch::Tensor, torch::Tensor, torch::Tensor> bin_by_coordinates_cpu_fn(
    torch::Tensor coordinates, torch::Tensor row_splits, torch::Tensor bin_width,
    torch::Tensor nbins, bool calc_n_per_bin);

std::tuple<torch::Tensor, torch::Tensor> binned_select_knn_cpu(
    torch::Tensor coordinates, torch::Tensor bin_idx, torch::Tensor dim_bin_idx,
    torch::Tensor bin_boundaries, torch::Tensor n_bins, torch::Tensor bin_width,
    torch::Tensor direction, bool tf_compat, bool use_direction, int64_t K);

torch::Tensor binned_select_knn_grad_cpu_fn(torch::Tensor grad_distances,
                                            torch::Tensor indices,
                                            torch::Tensor distances,
                                            torch::Tensor coordinates);

torch::Tensor index_replacer_cpu_fn(torch::Tensor to_be_replaced,
                                    torch::Tensor replacements);

namespace {
torch::Tensor f32(const float *p, std::initializer_list<int64_t> s) {
    return torch::from_blob(const_cast<float *>(p), s, torch::kFloat32);
}
torch::Tensor i64(const int64_t *p, std::initializer_list<int64_t> s) {
    return torch::from_blob(const_cast<int64_t *>(p), s, torch::kInt64);
}
template <typename T> void copy_out(const torch::Tensor &t, T *dst) {
    auto c = t.contiguous();
    std::memcpy(dst, c.data_ptr<T>(), sizeof(T) * c.numel());
}
}  // namespace

extern "C" {

int fgc_ref_bin_points(const float *coords, const int64_t *row_splits, float bin_width,
                       const int64_t *n_bins, int64_t *assigned, int64_t *flat,
                       int64_t *n_per_bin, int64_t n_vert, int64_t n_dims, int64_t n_rs) {
    try {
        auto bw = torch::full({1}, bin_width, torch::kFloat32);
        auto r = bin_by_coordinates_cpu_fn(f32(coords, {n_vert, n_dims}), i64(row_splits, {n_rs}),
                                           bw, i64(n_bins, {n_dims}), true);
        copy_out<int64_t>(std::get<0>(r), assigned);
        copy_out<int64_t>(std::get<1>(r), flat);
        copy_out<int64_t>(std::get<2>(r), n_per_bin);
        return 0;
    } catch (...) { return 1; }
}

int fgc_ref_knn_sorted(const float *coord, const int64_t *bin_idx, const int64_t *direction,
                       const int64_t *dim_bin_idx, const int64_t *bin_boundaries,
                       const int64_t *n_bins, float bin_width, int64_t *out_idx, float *out_dist,
                       int64_t n_vert, int64_t K, int64_t n_coords, int64_t n_bin_dims,
                       int64_t n_bboundaries, int tf_compat, int use_direction) {
    try {
        auto bw = torch::full({1}, bin_width, torch::kFloat32);
        auto dir = use_direction ? i64(direction, {n_vert}) : torch::empty({0}, torch::kInt64);
        auto r = binned_select_knn_cpu(f32(coord, {n_vert, n_coords}), i64(bin_idx, {n_vert}),
                                       i64(dim_bin_idx, {n_vert, n_bin_dims + 1}),
                                       i64(bin_boundaries, {n_bboundaries}),
                                       i64(n_bins, {n_bin_dims}), bw, dir, tf_compat != 0,
                                       use_direction != 0, K);
        copy_out<int64_t>(std::get<0>(r), out_idx);
        copy_out<float>(std::get<1>(r), out_dist);
        return 0;
    } catch (...) { return 1; }
}

int fgc_ref_knn_grad(const float *grad_dist, const int64_t *idx, const float *dist,
                     const float *coord, float *grad_coord, int64_t n_vert, int64_t K,
                     int64_t n_coords) {
    try {
        auto r = binned_select_knn_grad_cpu_fn(f32(grad_dist, {n_vert, K}), i64(idx, {n_vert, K}),
                                               f32(dist, {n_vert, K}),
                                               f32(coord, {n_vert, n_coords}));
        copy_out<float>(r, grad_coord);
        return 0;
    } catch (...) { return 1; }
}

int fgc_ref_index_replacer(const int64_t *in, const int64_t *repl, int64_t *out, int64_t n,
                           int64_t n_repl) {
    try {
        auto r = index_replacer_cpu_fn(i64(in, {n}), i64(repl, {n_repl}));
        copy_out<int64_t>(r, out);
        return 0;
    } catch (...) { return 1; }
}

}  // extern "C"
