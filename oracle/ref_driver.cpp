// C-ABI driver around the reference's own CPU kernels (test infrastructure).
//
// The functions declared below are defined by the reference's sources
// (bin_by_coordinates_cpu.cpp:102, binned_select_knn_cpu.cpp:211,
// binned_select_knn_grad_cpu.cpp:96, index_replacer_cpu.cpp:28,
// oc_helper_cpu.cpp:118, oc_helper_helper.cpp:30, select_knn_cpu.cpp:158), which
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

// oc_helper_cpu.cpp:118 and oc_helper_helper.cpp:30
std::tuple<torch::Tensor, torch::Tensor> oc_helper_cpu(
    torch::Tensor asso_idx, torch::Tensor unique_idx, torch::Tensor unique_rs_asso, torch::Tensor rs,
    torch::Tensor max_n_unique_over_splits, torch::Tensor max_n_in_splits, bool calc_m_not);

// select_knn_cpu.cpp:158
std::tuple<torch::Tensor, torch::Tensor> select_knn_cpu(torch::Tensor coords, torch::Tensor row_splits,
                                                        torch::Tensor mask, int64_t n_neighbours,
                                                        double max_radius, int64_t mask_mode);

std::tuple<torch::Tensor, torch::Tensor, torch::Tensor> max_same_valued_entries_per_row_split(
    const torch::Tensor &asso_idx, torch::Tensor row_splits, bool filter_negative);

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

// M [n_unique, n_maxuq] and M_not [n_unique, n_maxrs] of oc_helper_cpu (M_not is left untouched when
// calc_m_not is 0: the reference returns uninitialised memory for it then)
int fgc_ref_oc_helper(const int64_t *asso, const int64_t *unique_idx, const int64_t *unique_rs,
                      const int64_t *rs, int64_t *M, int64_t *M_not, int64_t n_vert, int64_t n_unique,
                      int64_t n_rs, int64_t n_maxuq, int64_t n_maxrs, int calc_m_not) {
    try {
        auto uq = torch::full({1}, n_maxuq, torch::kInt64);
        auto mrs = torch::full({1}, n_maxrs, torch::kInt64);
        auto r = oc_helper_cpu(i64(asso, {n_vert}), i64(unique_idx, {n_unique}), i64(unique_rs, {n_unique}),
                               i64(rs, {n_rs}), uq, mrs, calc_m_not != 0);
        copy_out<int64_t>(std::get<0>(r), M);
        if (calc_m_not) copy_out<int64_t>(std::get<1>(r), M_not);
        return 0;
    } catch (...) { return 1; }
}

// max_per_split [n_rs-1], global_max [1], objects_per_split [n_rs-1]
int fgc_ref_max_same_valued(const int64_t *asso, const int64_t *rs, int64_t *max_per_split,
                            int64_t *global_max, int64_t *objects_per_split, int64_t n_vert, int64_t n_rs,
                            int filter_negative) {
    try {
        auto r = max_same_valued_entries_per_row_split(i64(asso, {n_vert}), i64(rs, {n_rs}),
                                                       filter_negative != 0);
        copy_out<int64_t>(std::get<0>(r), max_per_split);
        global_max[0] = std::get<1>(r).item<int64_t>();
        copy_out<int64_t>(std::get<2>(r), objects_per_split);
        return 0;
    } catch (...) { return 1; }
}

int fgc_ref_select_knn(const float *coord, const int64_t *row_splits, int64_t *idx, float *dist, int64_t n_vert,
                       int64_t K, int64_t n_coords, int64_t n_rs, double max_radius) {
    try {
        auto mask = torch::zeros({n_vert}, torch::kInt64);
        auto r = select_knn_cpu(f32(coord, {n_vert, n_coords}), i64(row_splits, {n_rs}), mask, K, max_radius, 0);
        copy_out<int64_t>(std::get<0>(r), idx);
        copy_out<float>(std::get<1>(r), dist);
        return 0;
    } catch (...) { return 1; }
}

}  // extern "C"
