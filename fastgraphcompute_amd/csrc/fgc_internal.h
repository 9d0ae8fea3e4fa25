// Launchers shared between the translation units of libfgc_hip.so.
#pragma once
#include "fgc_common.h"

size_t fgc_sort_workspace_bytes(int64_t n);
int fgc_sort_keys(uint32_t *keys, uint32_t *vals, int64_t n, int key_bits, void *d_ws, hipStream_t s,
                  uint32_t **keys_sorted, uint32_t **vals_sorted, bool vals_given = false);
int fgc_launch_bin_keys(const float *d_coords, int n, int ld, int nbd, int sub_bits, const float *d_geom,
                        const int64_t *d_rs, int n_rs, uint32_t *d_keys, int *d_status, hipStream_t s);
// the tail of the preparation in one launch (sorted coordinates, boxes, bin boundaries), and for small inputs
// everything before it (range, geometry, keys, sort) in two launches plus one per sort pass
int fgc_launch_prepare_tail(const float *coords, int ld_in, const uint32_t *order, const uint32_t *skeys, int n, int D,
                            int ldc, float *sc, const int64_t *direction, unsigned char *sdir, float *sp, int sp_half,
                            float *box_lo, float *box_hi, float *sbox_lo, float *sbox_hi, int key_shift,
                            int n_bins_total, int *bb, unsigned *zero2, hipStream_t s);
bool fgc_sort_fused_fits(int64_t n);
int fgc_keys_and_sort_fused(const float *coords, int n, int ld, int nbd, const int64_t *n_bins, int sub_bits,
                            int key_bits, const int64_t *rs, int n_rs, float *partial, float *geom, uint32_t *keys,
                            uint32_t *vals, void *d_sort_ws, int *status, hipStream_t s, uint32_t **keys_sorted,
                            uint32_t **vals_sorted);

// kNN search over bin-sorted points (fgc_knn.hip)
struct KnnArgs {
    const float *sc;            // sorted coordinates, structure of arrays [D][ldc]
    int ldc;
    const float *sp;            // sorted coordinates as rows of 8 floats (matrix-core search only), or NULL
    const void *spa;            // the same points as float16 matrix operands relative to their group's centre, and
    const float *grp;           // the group records (fgc_launch_mf_operands); matrix-core search only
    const unsigned *mfstat;     // [2] chunks counted / chunks of groups far wider than the chunk (fgc_launch_mf_operands)
    const uint32_t *skeys;      // sorted key per point: (flat bin << key_shift) | Hilbert index inside the bin
    int key_shift;
    const float *box_lo;        // per 64-point chunk bounding boxes [D][n_chunks]
    const float *box_hi;
    int n_chunks;
    const float *sbox_lo;       // bounding boxes of aligned groups of 64 chunks [D][n_super]
    const float *sbox_hi;
    int n_super;
    const uint32_t *order;      // sorted position -> original row
    const int *bb;              // bin boundaries [n_bins_total + 1]
    const float *geom;          // geometry record
    const unsigned char *sdir;  // sorted direction flags or NULL
    int n;                      // points
    int D;                      // coordinates per point
    int nbd;                    // binned dimensions
    int K;
    int tf_compat;              // padding slots name the query itself instead of -1
    int any_order;              // rows may be written in pool order (slot 0 still the query itself) instead of by distance
    float tau0;                 // initial bound on the squared neighbour distance (INFINITY: none); exclusive
    int pool_cap;               // candidate pool slots per query (set by fgc_launch_knn)
    int64_t *out_idx;           // [n, K] original order
    float *out_dist;            // [n, K]
    int *out_sorted;            // optional [n, K]: the same rows in sorted space (row = sorted position of the
                                // query, entries = sorted positions), for the gradient kernel
    unsigned long long *stats;  // optional counters
    unsigned char *redo;        // NULL, or one flag per sorted position: the matrix-core search sets the flags of the
                                // queries it leaves out, and the vector search then handles the flagged queries only
};
int fgc_launch_knn(const KnnArgs &a, hipStream_t s);        // a.stats is ignored
int fgc_launch_knn_stats(const KnnArgs &a, hipStream_t s);  // the same search, counting into a.stats (slower)

// kNN search with the candidates screened on the matrix cores (fgc_knn_mfma.hip): 5 to 8 coordinates, K <= 256,
// needs a.sp.  Same rows as fgc_launch_knn up to the order inside a row and the choice between exactly tied candidates.
bool fgc_knn_uses_mfma(int D, int K);
inline int fgc_knn_sp_half(int D) { return D <= 6 ? 3 : 4; }   // coordinates per half row of sp
// Float16 operands of the matrix-core search.  A group is 16 consecutive chunks (1024 sorted points); grp[g] holds 16
// floats: the centre of the group's bounding box in the layout of sp (8), the scale sigma_g (a power of two with
// |c - centre| sigma_g <= 150 for every point of the group), the squared radius R_g^2 of the box, padding.  spa holds
// per point two halves of 8 float16: (c - centre) sigma_g for the half's coordinates (4, zero padded), then in the
// first half |c - centre|^2 sigma_g^2 (1 - 1.03 * 2^-10) as a (high, low) pair and 1, 1 - zeros in the second half.  A
// point with a non-finite coordinate, and the padding rows, carry an infinite norm.  mfstat[0] counts the chunks,
// mfstat[1] those whose group's squared radius is more than 24 times the chunk's own.
#define FGC_MF_GROUP_CHUNKS 16
#define FGC_MF_GRP_FLOATS 16
int fgc_launch_mf_operands(const float *sp, const float *box_lo, const float *box_hi, int n, int D, int ldc,
                           float *grp, void *spa, unsigned *mfstat, hipStream_t s);
int fgc_launch_knn_mfma(const KnnArgs &a, hipStream_t s);
int fgc_launch_knn_mfma_stats(const KnnArgs &a, hipStream_t s);
