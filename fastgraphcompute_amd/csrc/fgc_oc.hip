// Object / vertex index matrices of the object-condensation helper (gfx950).
//
// The reference builds them from torch.unique calls on the host side plus one thread per object that scans its
// whole row split (oc_helper.py:152-229, oc_helper_cuda_kernel.cu:19-116).  Here one stable radix sort of the
// vertices by (row split, association index) makes every object a contiguous run of the sorted order:
//   objects pass   keys -> sort -> run boundaries -> object table (start, end, row split, value), the object id
//                  of every vertex, the widest object and the per-split counts;
//   fill pass      M is a gather of the sorted order; a row of M_not is a stream compaction of the row split's
//                  vertex range that drops the object's own members (one 64-ary search per wavefront gives the
//                  number of members before the wavefront's slice, ballots do the rest).
// The fill pass is a pure HBM write stream of 8 * n_unique * (n_maxuq + n_maxrs) bytes.
#include "fgc_internal.h"

namespace {

constexpr int OC_BLOCK = 256;
#ifndef FGC_OC_NOT_CHUNK
#define FGC_OC_NOT_CHUNK 4096
#endif
constexpr int OC_NOT_CHUNK = FGC_OC_NOT_CHUNK;     // vertex offsets of one row handled by one block
constexpr int OC_NOT_WAVE = OC_NOT_CHUNK / 4;      // ... by one wavefront
#ifndef FGC_OC_FEW
#define FGC_OC_FEW 16
#endif
constexpr int OC_FEW = FGC_OC_FEW;                 // members per slice up to which gaps are computed, not compacted
enum { OC_KEY_NARROW = 0, OC_KEY_LO = 1, OC_KEY_HI = 2, OC_KEY_RS = 3 };

// summary record (int64 words)
enum { OC_SUM_NUNIQUE = 0, OC_SUM_MAXUQ = 1, OC_SUM_FLAGS = 2 };

// row split of vertex i: the r with rs[r] <= i < rs[r + 1] (empty splits are skipped over)
__device__ __forceinline__ int oc_split_of(const int64_t *__restrict__ rs, int n_rs, int64_t i)
{
    int lo = 0, hi = n_rs - 1;      // invariant: rs[lo] <= i, answer in [lo, hi)
    while (hi - lo > 1) {
        int mid = (lo + hi) >> 1;
        if (rs[mid] <= i) lo = mid; else hi = mid;
    }
    return lo;
}

// order-preserving unsigned code of an association index; with `filter` all negative values share code 0
__device__ __forceinline__ unsigned long long oc_code(int64_t v, bool filter)
{
    if (filter) return v < 0 ? 0ull : (unsigned long long)v + 1ull;
    return (unsigned long long)v ^ 0x8000000000000000ull;
}

__global__ __launch_bounds__(OC_BLOCK) void k_oc_keys(const int64_t *__restrict__ asso, int n,
                                                      const int64_t *__restrict__ rs, int n_rs, int mode,
                                                      int value_bits, bool filter,
                                                      const uint32_t *__restrict__ perm_in,
                                                      uint32_t *__restrict__ keys,
                                                      unsigned long long *__restrict__ summary)
{
    int p = blockIdx.x * OC_BLOCK + threadIdx.x;
    if (p >= n) return;
    const int64_t i = (mode == OC_KEY_NARROW || mode == OC_KEY_LO) ? p : (int64_t)perm_in[p];
    if (mode == OC_KEY_RS) { keys[p] = (uint32_t)oc_split_of(rs, n_rs, i); return; }
    const unsigned long long u = oc_code(asso[i], filter);
    if (mode == OC_KEY_LO) { keys[p] = (uint32_t)u; return; }
    if (mode == OC_KEY_HI) { keys[p] = (uint32_t)(u >> 32); return; }
    const unsigned long long lim = 1ull << value_bits;
    uint32_t code = (uint32_t)u;
    if (u >= lim) {                       // does not fit beside the row split: the caller repeats with wide keys
        atomicOr(summary + OC_SUM_FLAGS, 1ull);
        code = (uint32_t)(lim - 1);
    }
    keys[p] = value_bits >= 32 ? code : (((uint32_t)oc_split_of(rs, n_rs, i) << value_bits) | code);
}

// Per sorted position: bit 0 = first vertex of an object, bit 1 = belongs to an object, bit 2 = last vertex of
// an object.  block_heads[b] = objects starting inside block b.
__global__ __launch_bounds__(OC_BLOCK) void k_oc_segments(const int64_t *__restrict__ asso,
                                                          const uint32_t *__restrict__ perm, int n,
                                                          const int64_t *__restrict__ rs, int n_rs, bool filter,
                                                          unsigned char *__restrict__ flags,
                                                          uint32_t *__restrict__ block_heads)
{
    __shared__ unsigned long long s_u[OC_BLOCK + 2];
    __shared__ int s_r[OC_BLOCK + 2];
    __shared__ int s_cnt[4];
    const int t = threadIdx.x, p = blockIdx.x * OC_BLOCK + t;
    auto load = [&](int q, int slot) {
        if (q >= 0 && q < n) {
            int64_t i = perm[q];
            s_u[slot] = oc_code(asso[i], filter);
            s_r[slot] = oc_split_of(rs, n_rs, i);
        } else {
            s_u[slot] = 0ull;
            s_r[slot] = -1;           // no vertex: differs from every real one
        }
    };
    load(p, t + 1);
    if (t == 0) load(p - 1, 0);
    if (t == OC_BLOCK - 1) load(p + 1, OC_BLOCK + 1);
    __syncthreads();
    bool head = false;
    if (p < n) {
        const unsigned long long u = s_u[t + 1];
        const int r = s_r[t + 1];
        const bool is_obj = !(filter && u == 0ull);
        const bool first = (s_r[t] != r) || (s_u[t] != u);
        const bool last = (s_r[t + 2] != r) || (s_u[t + 2] != u);
        head = first && is_obj;
        flags[p] = (unsigned char)((head ? 1 : 0) | (is_obj ? 2 : 0) | ((last && is_obj) ? 4 : 0));
    }
    const unsigned long long m = fgc_ballot(head);
    if (fgc_lane() == 0) s_cnt[t >> 6] = __popcll(m);
    __syncthreads();
    if (t == 0) block_heads[blockIdx.x] = (uint32_t)(s_cnt[0] + s_cnt[1] + s_cnt[2] + s_cnt[3]);
}

// in-place exclusive scan of the per-block counts by one block; the total goes to the summary record
__global__ __launch_bounds__(OC_BLOCK) void k_oc_scan_blocks(uint32_t *__restrict__ block_heads, int nblk,
                                                             unsigned long long *__restrict__ summary)
{
    __shared__ uint32_t s_w[4];
    __shared__ uint32_t s_carry;
    const int t = threadIdx.x, lane = t & 63, w = t >> 6;
    if (t == 0) s_carry = 0;
    __syncthreads();
    for (int b0 = 0; b0 < nblk; b0 += OC_BLOCK) {
        const int b = b0 + t;
        const uint32_t v = b < nblk ? block_heads[b] : 0u;
        uint32_t incl = v;
        for (int o = 1; o < 64; o <<= 1) {
            uint32_t x = __shfl_up(incl, o, 64);
            if (lane >= o) incl += x;
        }
        if (lane == 63) s_w[w] = incl;
        __syncthreads();
        uint32_t off = s_carry;
        for (int k = 0; k < w; k++) off += s_w[k];
        if (b < nblk) block_heads[b] = off + incl - v;
        __syncthreads();
        if (t == OC_BLOCK - 1) s_carry = off + incl;
        __syncthreads();
    }
    if (t == 0) summary[OC_SUM_NUNIQUE] = s_carry;
}

// object table and the object id of every vertex
__global__ __launch_bounds__(OC_BLOCK) void k_oc_objects(const int64_t *__restrict__ asso,
                                                         const uint32_t *__restrict__ perm,
                                                         const unsigned char *__restrict__ flags,
                                                         const uint32_t *__restrict__ block_off, int n,
                                                         const int64_t *__restrict__ rs, int n_rs,
                                                         int *__restrict__ oid, int *__restrict__ obj_start,
                                                         int *__restrict__ obj_end, int *__restrict__ obj_rs,
                                                         int64_t *__restrict__ obj_val)
{
    __shared__ int s_cnt[4];
    const int t = threadIdx.x, p = blockIdx.x * OC_BLOCK + t, w = t >> 6;
    const int f = p < n ? (int)flags[p] : 0;
    const unsigned long long m = fgc_ballot((f & 1) != 0);
    if (fgc_lane() == 0) s_cnt[w] = __popcll(m);
    __syncthreads();
    int incl = (int)block_off[blockIdx.x] + fgc_mbcnt(m) + (f & 1);
    for (int k = 0; k < w; k++) incl += s_cnt[k];
    if (p >= n) return;
    const int k = incl - 1;       // object of this position when bit 1 is set
    const int64_t i = perm[p];
    oid[i] = (f & 2) ? k : -1;
    if (f & 1) {
        obj_start[k] = p;
        obj_rs[k] = oc_split_of(rs, n_rs, i);
        obj_val[k] = asso[i];
    }
    if (f & 4) obj_end[k] = p + 1;
}

__device__ __forceinline__ int oc_wave_max(int v)
{
    for (int o = 32; o > 0; o >>= 1) v = max(v, __shfl_xor(v, o, 64));
    return v;
}

// widest object overall and per row split, objects per row split
__global__ __launch_bounds__(OC_BLOCK) void k_oc_finish(const int *__restrict__ obj_start,
                                                        const int *__restrict__ obj_end,
                                                        const int *__restrict__ obj_rs,
                                                        unsigned long long *__restrict__ summary,
                                                        unsigned long long *__restrict__ max_per_split,
                                                        unsigned long long *__restrict__ objects_per_split)
{
    const int n_obj = (int)summary[OC_SUM_NUNIQUE];
    const int stride = gridDim.x * OC_BLOCK;
    for (int k0 = blockIdx.x * OC_BLOCK; k0 < n_obj; k0 += stride) {     // uniform trip count per wavefront
        const int k = k0 + threadIdx.x;
        const bool valid = k < n_obj;
        const int cnt = valid ? obj_end[k] - obj_start[k] : 0;
        const int r = valid ? obj_rs[k] : -1;
        const int wmax = oc_wave_max(cnt);
        const int r0 = fgc_readlane_i(r, 0);
        const bool same = fgc_ballot(valid && r != r0) == 0ull;        // lane 0 is valid whenever any lane is
        if (same) {
            const int nv = __popcll(fgc_ballot(valid));
            if (fgc_lane() == 0 && nv > 0) {
                atomicMax(max_per_split + r0, (unsigned long long)wmax);
                atomicAdd(objects_per_split + r0, (unsigned long long)nv);
            }
        } else if (valid) {
            atomicMax(max_per_split + r, (unsigned long long)cnt);
            atomicAdd(objects_per_split + r, 1ull);
        }
        if (fgc_lane() == 0 && wmax > 0) atomicMax(summary + OC_SUM_MAXUQ, (unsigned long long)wmax);
    }
}

// row of the object table for each (value, row split) pair of the caller, -1 when there is no such object
__global__ __launch_bounds__(OC_BLOCK) void k_oc_lookup(const int64_t *__restrict__ q_val,
                                                        const int64_t *__restrict__ q_rs, int n_q,
                                                        const int *__restrict__ obj_rs,
                                                        const int64_t *__restrict__ obj_val,
                                                        const unsigned long long *__restrict__ summary,
                                                        int *__restrict__ map)
{
    const int q = blockIdx.x * OC_BLOCK + threadIdx.x;
    if (q >= n_q) return;
    const int n_obj = (int)summary[OC_SUM_NUNIQUE];
    const int64_t v = q_val[q], r = q_rs[q];
    int lo = 0, hi = n_obj;           // first object not below (r, v)
    while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        const int64_t mr = obj_rs[mid];
        if (mr < r || (mr == r && obj_val[mid] < v)) lo = mid + 1; else hi = mid;
    }
    map[q] = (lo < n_obj && obj_rs[lo] == r && obj_val[lo] == v) ? lo : -1;
}

__global__ __launch_bounds__(OC_BLOCK) void k_oc_fill_m(const uint32_t *__restrict__ perm,
                                                        const int *__restrict__ obj_start,
                                                        const int *__restrict__ obj_end,
                                                        const int *__restrict__ map, int64_t n_rows, int n_maxuq,
                                                        int64_t *__restrict__ M, int *__restrict__ status)
{
    const int64_t total = n_rows * n_maxuq;
    const int64_t stride = (int64_t)gridDim.x * OC_BLOCK;
    for (int64_t e = (int64_t)blockIdx.x * OC_BLOCK + threadIdx.x; e < total; e += stride) {
        const int64_t row = e / n_maxuq;
        const int j = (int)(e - row * n_maxuq);
        const int k = map ? map[row] : (int)row;
        int64_t out = -1;
        if (k >= 0) {
            const int s = obj_start[k], cnt = obj_end[k] - s;
            if (j < cnt) out = perm[s + j];
            if (j == 0 && cnt > n_maxuq && status) atomicOr(status, FGC_ST_OC_TRUNCATED);
        }
        M[e] = out;
    }
}

// members of the sorted run [mem, mem + cnt) that are smaller than x (64 probes per step, whole wavefront)
__device__ __forceinline__ int oc_rank_below(const uint32_t *__restrict__ mem, int cnt, uint32_t x)
{
    int lo = 0, len = cnt;
    const int lane = fgc_lane();
    while (len > 0) {
        const int step = (len + 63) >> 6;
        const int probe = lo + (lane + 1) * step - 1;           // last element of this lane's piece
        const bool below = (lane * step < len) && mem[min(probe, lo + len - 1)] < x;
        const int t = __popcll(fgc_ballot(below));              // pieces entirely below x
        if (step == 1) return lo + t;
        if (t * step >= len) return lo + len;
        const int piece = min(step, len - t * step);            // its last element is not below x
        lo += t * step;
        len = piece - 1;
    }
    return lo;
}

// dst[j] = value(j) for j in [0, count) by one wavefront: a single 8-byte store brings dst to a 16-byte
// boundary, then every lane stores two elements at a time
template <class F>
__device__ __forceinline__ void oc_stream_out(int64_t *__restrict__ dst, int count, int lane, F value)
{
    if (count <= 0) return;
    const int head = (int)(((uintptr_t)dst >> 3) & 1);
    if (head && lane == 0) dst[0] = value(0);
    const int pairs = (count - head) >> 1;
    longlong2 *d2 = (longlong2 *)(dst + head);
    for (int j = lane; j < pairs; j += 64) {
        longlong2 v;
        v.x = value(head + 2 * j);
        v.y = value(head + 2 * j + 1);
        d2[j] = v;
    }
    if (((count - head) & 1) && lane == 63) dst[count - 1] = value(count - 1);
}

// M_not: for block (row, chunk) the vertex offsets [chunk * OC_NOT_CHUNK, +OC_NOT_CHUNK) of the row's split,
// compacted to the vertices outside the object, plus the -1 padding that falls into the same output range.
__global__ __launch_bounds__(OC_BLOCK) void k_oc_fill_m_not(const uint32_t *__restrict__ perm,
                                                            const int *__restrict__ oid,
                                                            const int *__restrict__ obj_start,
                                                            const int *__restrict__ obj_end,
                                                            const int *__restrict__ obj_rs,
                                                            const int *__restrict__ map,
                                                            const int64_t *__restrict__ q_rs,
                                                            const int64_t *__restrict__ rs, int n_rs, int n_vert,
                                                            int n_chunks, int n_maxrs, int64_t *__restrict__ M_not)
{
    __shared__ int s_buf[4][OC_NOT_WAVE];
    const int row = blockIdx.x / n_chunks, chunk = blockIdx.x - row * n_chunks;
    const int lane = fgc_lane(), wv = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    int *buf = s_buf[wv];
    const int k = map ? map[row] : row;
    int r;
    if (q_rs) {
        const int64_t qr = q_rs[row];
        r = (qr >= 0 && qr < n_rs - 1) ? (int)qr : -1;
    } else {
        r = obj_rs[k];
    }
    int64_t *out = M_not + (int64_t)row * n_maxrs;
    int lo = 0, len = 0;
    bool clipped = false;
    if (r >= 0) {
        int64_t a = rs[r], b = rs[r + 1];
        if (b > n_vert) b = n_vert;
        if (a < 0) a = 0;
        if (b - a > n_maxrs) { b = a + n_maxrs; clipped = true; }       // as the reference's kernel clips
        if (b > a) { lo = (int)a; len = (int)(b - a); }
    }
    const uint32_t *mem = perm + (k >= 0 ? obj_start[k] : 0);
    const int cnt = k >= 0 ? obj_end[k] - obj_start[k] : 0;
    const int o0 = chunk * OC_NOT_CHUNK + wv * OC_NOT_WAVE;
    const int o1 = min(o0 + OC_NOT_WAVE, len);
    if (o0 < len) {
        // members of the object below the slice (r0) and below its end (r1)
        int r0 = 0, r1 = 0;
        uint32_t mine = 0xffffffffu;                 // member r0 + lane when the slice holds at most 64 of them
        if (cnt > 0 && cnt <= 64) {
            const uint32_t v = lane < cnt ? mem[lane] : 0xffffffffu;
            r0 = __popcll(fgc_ballot(v < (uint32_t)(lo + o0)));
            r1 = __popcll(fgc_ballot(v < (uint32_t)(lo + o1)));
            mine = (uint32_t)__shfl((int)v, (r0 + lane) & 63, 64);
            if (lane >= r1 - r0) mine = 0xffffffffu;
        } else if (cnt > 64) {
            r0 = oc_rank_below(mem, cnt, (uint32_t)(lo + o0));
            r1 = r0 + oc_rank_below(mem + r0, min(cnt - r0, OC_NOT_WAVE), (uint32_t)(lo + o1));
            if (r1 - r0 <= OC_FEW && lane < r1 - r0) mine = mem[r0 + lane];
        }
        const int base = o0 - r0, in_slice = r1 - r0, kept = (o1 - o0) - in_slice;
        if (in_slice <= OC_FEW) {
            // few gaps: element j of the output is offset o0 + j + (members that come before it); member i
            // comes before element j when the kept vertices in front of it, d_i, number at most j
            const int d = mine == 0xffffffffu ? 0x7fffffff : (int)mine - lo - o0 - lane;
            oc_stream_out(out + base, kept, lane, [&](int j) {
                int t = 0;
                for (int i = 0; i < in_slice; i++) t += (fgc_readlane_i(d, i) <= j) ? 1 : 0;
                return (int64_t)(lo + o0 + j + t);
            });
        } else {
            // many gaps: compact the kept vertices in LDS by ballots over the object id of every vertex
            int pos = 0;
            for (int g = o0; g < o1; g += 256) {
                int id[4];
#pragma unroll
                for (int u = 0; u < 4; u++) {
                    const int off = g + u * 64 + lane;
                    id[u] = off < o1 ? oid[lo + off] : k;
                }
#pragma unroll
                for (int u = 0; u < 4; u++) {
                    const int off = g + u * 64 + lane;
                    const bool keep = off < o1 && id[u] != k;
                    const unsigned long long m = fgc_ballot(keep);
                    if (keep) buf[pos + fgc_mbcnt(m)] = lo + off;
                    pos += __popcll(m);
                }
            }
            oc_stream_out(out + base, pos, lane, [&](int j) { return (int64_t)buf[j]; });
        }
    }
    // padding positions inside this wavefront's output range
    const int e1 = min(o0 + OC_NOT_WAVE, n_maxrs);
    if (e1 > len - cnt) {
        int members = cnt;
        if (clipped && cnt > 0) members = oc_rank_below(mem, cnt, (uint32_t)(lo + len));
        const int pad0 = max(o0, len - members);
        oc_stream_out(out + pad0, e1 - pad0, lane, [](int) { return (int64_t)-1; });
    }
}

__global__ void k_oc_export(const int *__restrict__ obj_rs, const int64_t *__restrict__ obj_val, int n_obj,
                            int64_t *__restrict__ out_val, int64_t *__restrict__ out_rs)
{
    int k = blockIdx.x * blockDim.x + threadIdx.x;
    if (k >= n_obj) return;
    if (out_val) out_val[k] = obj_val[k];
    if (out_rs) out_rs[k] = obj_rs[k];
}

struct OcPlan {
    size_t sort, keys, perm, oid, obj_start, obj_end, obj_rs, obj_val, flags, blocks, map, total;
};

OcPlan oc_plan(int64_t n)
{
    OcPlan w;
    const size_t n1 = (size_t)(n > 0 ? n : 1);
    size_t o = 0;
    auto take = [&](size_t bytes) { size_t at = o; o += fgc_align(bytes); return at; };
    w.sort = take(fgc_sort_workspace_bytes(n));
    w.keys = take(n1 * 4);
    w.perm = take(n1 * 4);
    w.oid = take(n1 * 4);
    w.obj_start = take(n1 * 4);
    w.obj_end = take(n1 * 4);
    w.obj_rs = take(n1 * 4);
    w.obj_val = take(n1 * 8);
    w.flags = take(n1);
    w.blocks = take(((size_t)fgc_cdiv(n1, OC_BLOCK) + 1) * 4);
    w.map = take(n1 * 4);
    w.total = o;
    return w;
}

int oc_bits(int64_t v)       // bits needed to hold values 0..v
{
    int b = 0;
    while (v > 0) { b++; v >>= 1; }
    return b;
}

}  // namespace

extern "C" {

size_t fgc_oc_helper_workspace_bytes(int64_t n_vert)
{
    if (n_vert < 0) return 0;
    return oc_plan(n_vert).total;
}

int fgc_oc_helper_objects_i64(const int64_t *d_asso, int64_t n_vert, const int64_t *d_row_splits, int32_t n_rs,
                              int32_t filter_negative, int32_t wide_keys, int64_t *d_max_per_split,
                              int64_t *d_objects_per_split, int64_t *d_summary, void *d_ws, size_t ws_bytes,
                              void *stream)
{
    if (n_vert < 0 || n_vert >= (1ll << 31) - 4096 || n_rs < 2 || !d_row_splits || !d_summary ||
        !d_max_per_split || !d_objects_per_split || (n_vert > 0 && !d_asso))
        return FGC_EINVAL;
    const OcPlan w = oc_plan(n_vert);
    if (!d_ws || ws_bytes < w.total) return FGC_ENOSPACE;
    hipStream_t s = (hipStream_t)stream;
    int rc;
    if ((rc = fgc_fill_u32(d_summary, 0u, 2 * FGC_OC_SUMMARY_WORDS, s))) return rc;
    if ((rc = fgc_fill_u32(d_max_per_split, 0u, 2 * (int64_t)(n_rs - 1), s))) return rc;
    if ((rc = fgc_fill_u32(d_objects_per_split, 0u, 2 * (int64_t)(n_rs - 1), s))) return rc;
    if (n_vert == 0) return FGC_OK;

    char *ws = (char *)d_ws;
    uint32_t *keys = (uint32_t *)(ws + w.keys), *perm = (uint32_t *)(ws + w.perm);
    unsigned long long *summary = (unsigned long long *)d_summary;
    const int n = (int)n_vert;
    const bool filter = filter_negative != 0;
    const dim3 grid((unsigned)fgc_cdiv(n, OC_BLOCK)), block(OC_BLOCK);
    const int rs_bits = oc_bits(n_rs - 2);
    const int value_bits = 32 - rs_bits;
    const bool wide = wide_keys != 0 || !filter || value_bits < 8;
    uint32_t *ks, *vs;
    auto settle = [&]() -> int {          // bring the sorted payload back into `perm`
        if (vs != perm) return fgc_copy_u32(perm, vs, n, s);
        return FGC_OK;
    };
    if (!wide) {
        hipLaunchKernelGGL(k_oc_keys, grid, block, 0, s, d_asso, n, d_row_splits, (int)n_rs, (int)OC_KEY_NARROW,
                           value_bits, filter, (const uint32_t *)nullptr, keys, summary);
        FGC_LAUNCH_CHECK();
        if ((rc = fgc_sort_keys(keys, perm, n, 32, ws + w.sort, s, &ks, &vs, false))) return rc;
        if ((rc = settle())) return rc;
    } else {
        hipLaunchKernelGGL(k_oc_keys, grid, block, 0, s, d_asso, n, d_row_splits, (int)n_rs, (int)OC_KEY_LO, 0,
                           filter, (const uint32_t *)nullptr, keys, summary);
        FGC_LAUNCH_CHECK();
        if ((rc = fgc_sort_keys(keys, perm, n, 32, ws + w.sort, s, &ks, &vs, false))) return rc;
        if ((rc = settle())) return rc;
        hipLaunchKernelGGL(k_oc_keys, grid, block, 0, s, d_asso, n, d_row_splits, (int)n_rs, (int)OC_KEY_HI, 0,
                           filter, (const uint32_t *)perm, keys, summary);
        FGC_LAUNCH_CHECK();
        if ((rc = fgc_sort_keys(keys, perm, n, 32, ws + w.sort, s, &ks, &vs, true))) return rc;
        if ((rc = settle())) return rc;
        if (n_rs > 2) {
            hipLaunchKernelGGL(k_oc_keys, grid, block, 0, s, d_asso, n, d_row_splits, (int)n_rs, (int)OC_KEY_RS,
                               0, filter, (const uint32_t *)perm, keys, summary);
            FGC_LAUNCH_CHECK();
            if ((rc = fgc_sort_keys(keys, perm, n, rs_bits, ws + w.sort, s, &ks, &vs, true))) return rc;
            if ((rc = settle())) return rc;
        }
    }
    unsigned char *flags = (unsigned char *)(ws + w.flags);
    uint32_t *blocks = (uint32_t *)(ws + w.blocks);
    hipLaunchKernelGGL(k_oc_segments, grid, block, 0, s, d_asso, (const uint32_t *)perm, n, d_row_splits,
                       (int)n_rs, filter, flags, blocks);
    FGC_LAUNCH_CHECK();
    hipLaunchKernelGGL(k_oc_scan_blocks, dim3(1), block, 0, s, blocks, (int)grid.x, summary);
    FGC_LAUNCH_CHECK();
    hipLaunchKernelGGL(k_oc_objects, grid, block, 0, s, d_asso, (const uint32_t *)perm,
                       (const unsigned char *)flags, (const uint32_t *)blocks, n, d_row_splits, (int)n_rs,
                       (int *)(ws + w.oid), (int *)(ws + w.obj_start), (int *)(ws + w.obj_end),
                       (int *)(ws + w.obj_rs), (int64_t *)(ws + w.obj_val));
    FGC_LAUNCH_CHECK();
    unsigned fin = (unsigned)fgc_cdiv(n, OC_BLOCK);
    if (fin > 1024) fin = 1024;
    hipLaunchKernelGGL(k_oc_finish, dim3(fin), block, 0, s, (const int *)(ws + w.obj_start),
                       (const int *)(ws + w.obj_end), (const int *)(ws + w.obj_rs), summary,
                       (unsigned long long *)d_max_per_split, (unsigned long long *)d_objects_per_split);
    FGC_LAUNCH_CHECK();
    return FGC_OK;
}

int fgc_oc_helper_fill_i64(int64_t n_vert, const int64_t *d_row_splits, int32_t n_rs, int64_t n_rows,
                           int64_t n_maxuq, int64_t n_maxrs, const int64_t *d_unique_idx,
                           const int64_t *d_unique_rs, const int64_t *d_summary, int64_t *d_M, int64_t *d_M_not,
                           int64_t *d_obj_idx_out, int64_t *d_obj_rs_out, int32_t *d_status, const void *d_ws,
                           size_t ws_bytes, void *stream)
{
    if (n_vert < 0 || n_vert >= (1ll << 31) - 4096 || n_rs < 2 || !d_row_splits || n_rows < 0 ||
        n_rows > n_vert || n_maxuq < 0 || n_maxuq >= (1ll << 31) || n_maxrs < 0 || n_maxrs >= (1ll << 31) - 4096 ||
        ((d_unique_idx == nullptr) != (d_unique_rs == nullptr)) || (d_unique_idx && !d_summary))
        return FGC_EINVAL;
    const OcPlan w = oc_plan(n_vert);
    if (!d_ws || ws_bytes < w.total) return FGC_ENOSPACE;
    if (n_rows == 0) return FGC_OK;
    hipStream_t s = (hipStream_t)stream;
    const char *ws = (const char *)d_ws;
    const uint32_t *perm = (const uint32_t *)(ws + w.perm);
    const int *obj_start = (const int *)(ws + w.obj_start), *obj_end = (const int *)(ws + w.obj_end);
    const int *obj_rs = (const int *)(ws + w.obj_rs);
    const int64_t *obj_val = (const int64_t *)(ws + w.obj_val);
    int *map = nullptr;
    const dim3 block(OC_BLOCK);
    if (d_unique_idx) {
        map = (int *)(ws + w.map);     // scratch inside the caller's workspace
        hipLaunchKernelGGL(k_oc_lookup, dim3((unsigned)fgc_cdiv(n_rows, OC_BLOCK)), block, 0, s, d_unique_idx,
                           d_unique_rs, (int)n_rows, obj_rs, obj_val, (const unsigned long long *)d_summary, map);
        FGC_LAUNCH_CHECK();
    }
    if (d_M && n_maxuq > 0) {
        int64_t blocks = fgc_cdiv(n_rows * n_maxuq, OC_BLOCK);
        if (blocks > 65536) blocks = 65536;
        hipLaunchKernelGGL(k_oc_fill_m, dim3((unsigned)blocks), block, 0, s, perm, obj_start, obj_end,
                           (const int *)map, n_rows, (int)n_maxuq, d_M, d_status);
        FGC_LAUNCH_CHECK();
    }
    if (d_M_not && n_maxrs > 0) {
        const int64_t n_chunks = fgc_cdiv(n_maxrs, OC_NOT_CHUNK);
        if (n_rows * n_chunks >= (1ll << 31)) return FGC_EINVAL;
        hipLaunchKernelGGL(k_oc_fill_m_not, dim3((unsigned)(n_rows * n_chunks)), block, 0, s, perm,
                           (const int *)(ws + w.oid), obj_start, obj_end, obj_rs, (const int *)map, d_unique_rs,
                           d_row_splits, (int)n_rs, (int)n_vert, (int)n_chunks, (int)n_maxrs, d_M_not);
        FGC_LAUNCH_CHECK();
    }
    if (!d_unique_idx && (d_obj_idx_out || d_obj_rs_out)) {
        hipLaunchKernelGGL(k_oc_export, dim3((unsigned)fgc_cdiv(n_rows, OC_BLOCK)), block, 0, s, obj_rs, obj_val,
                           (int)n_rows, d_obj_idx_out, d_obj_rs_out);
        FGC_LAUNCH_CHECK();
    }
    return FGC_OK;
}

}  // extern "C"
