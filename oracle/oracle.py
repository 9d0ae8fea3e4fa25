"""CPU checker for the graph-building path (TEST INFRASTRUCTURE, not product).

Python side of the oracle: the host-level glue of the reference restated with
numpy float32 arithmetic, on top of the plain-C kernels in fgc_oracle.c.  Only
tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
this module; the product package never does and has no CPU fallback.

All file:line citations are relative to the reference checkout.

Pinning status (what fixes each function independently of this restatement):

  normalise / bin_by_coordinates   known answers of the reference's tests
                                   (tests/test_bin_by_coordinates.py:32-43,
                                   114-139), invariants (:195-216), and the
                                   reference's compiled `calc` (oracle/_ref).
  optimal_n_bins                   the five hand-computed benchmark values; the
                                   pow is evaluated with the same ATen CPU op
                                   as the reference (binned_knn_autograd_
                                   kernel.cpp:78-81).
  knn_sorted / binned_select_knn   brute force (knn_brute, and torch.cdist +
                                   topk as tests/test_binned_select_knn.py:
                                   28-78), the reference's compiled kernel
                                   (oracle/_ref) slot for slot.
  index_replacer                   golden array tests/test_index_replacer.py:
                                   52-71, oracle/_ref.
  knn_grad                         float64 closed form / torch autograd through
                                   the gathered distances (tests/
                                   test_binned_select_knn.py:209-226),
                                   oracle/_ref bit for bit.
  select_with_default,
  gravnet_aggregate, gravnet_aggregate_torch, gravnet_forward_torch
                                   the reference's tests hold no numeric values
                                   for GravNetOp (tests/test_gnn_ops.py checks
                                   shapes and script-vs-eager only), so these are
                                   pinned by what gnn_ops.py:90-102 fixes
                                   mathematically (tests/test_oracle_gravnet.py):
                                   hand-computed known answers with weights 1,
                                   1/2, 1/4 (padding counts as 0, the mean
                                   divides by K, the padding's 0 can be the
                                   maximum, the first of two equal maxima takes
                                   the gradient; forward, both gradients, and the
                                   whole layer with hand-set weights), closed
                                   forms (zero distances = numpy.take + mean /
                                   max, K = 1 = own features, a common distance
                                   scales the result), a float64 loop over the
                                   definition, and central differences of that
                                   loop for the aggregation's and the layer's
                                   gradients.
  oc_helper_inputs,
  max_same_valued_entries_per_row_split
                                   numpy.unique per row split, the routine the
                                   reference's own test restates them with
                                   (tests/test_oc_helper_helper.py:63-111); the
                                   known answers of tests/test_oc_helper.py:
                                   55-57 and the reference's compiled
                                   oc_helper_helper.cpp (oracle/_ref).
  select_knn                       the definition (numpy float64 brute force inside the radius), the
                                   reference's compiled select_knn_cpu (oracle/_ref) slot for slot; the
                                   reference holds no test or fixture for this op.
  oc_calc_m / oc_helper_matrices   the hand-written expectation of tests/
                                   test_oc_helper.py:80-112, the stored
                                   matrices tests/test_oc_helper_large_M*.npy
                                   (:205-230), the reference's compiled calc_m
                                   (oracle/_ref) element for element.
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None
_REF = None

_f32p = ctypes.POINTER(ctypes.c_float)
_i64p = ctypes.POINTER(ctypes.c_int64)


def _fp(a):
    return a.ctypes.data_as(_f32p) if a is not None else None


def _ip(a):
    return a.ctypes.data_as(_i64p) if a is not None else None


def lib():
    """The compiled C restatement (oracle/libfgc_oracle.so)."""
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "libfgc_oracle.so")
        if not os.path.exists(path):
            raise RuntimeError("oracle library not built: run python oracle/build_oracle.py")
        _LIB = ctypes.CDLL(path)
        _LIB.fgc_oracle_bin_points.restype = ctypes.c_int64
        _LIB.fgc_oracle_knn_sorted.restype = ctypes.c_int64
    return _LIB


def ref_lib():
    """The reference's own CPU kernels (oracle/_ref/libfgc_ref.so) or None."""
    global _REF
    if _REF is None:
        path = os.path.join(_HERE, "_ref", "libfgc_ref.so")
        if not os.path.exists(path):
            return None
        import torch  # noqa: F401  (loads libtorch, which the .so links to)
        _REF = ctypes.CDLL(path)
    return _REF


def _c(a, dt):
    return np.ascontiguousarray(a, dtype=dt)


# --------------------------------------------------------------------------
# bin_by_coordinates
# --------------------------------------------------------------------------
def normalise(coords, bin_width=None, n_bins=None, pre_normalized=False):
    """Host preprocessing of bin_by_coordinates (bin_by_coordinates.py:40-92,
    repeated by bin_by_coordinates.cpp:57-111): subtract the global per-dim
    minimum, take the per-dim range (+1 where it is zero, +1e-3), and derive the
    single cubic bin width max_d(range_d / n_bins_d), or n_bins from a given
    width.  Every step is one float32 operation."""
    c = _c(coords, np.float32)
    if not np.all(np.isfinite(c)):
        raise ValueError("BinByCoordinates: input coordinates contain non-finite values")
    if not pre_normalized and c.shape[0] > 0:
        c = c - c.min(axis=0, keepdims=True)
    dmax = c.max(axis=0)
    dmin = c.min(axis=0)
    dmax = np.where(dmin == dmax, dmax + np.float32(1.0), dmax).astype(np.float32)
    dmax = (dmax + np.float32(1e-3)).astype(np.float32)
    dmax = np.where(np.isfinite(dmax), dmax, np.float32(1.0)).astype(np.float32)
    if not np.all(dmax > 0):
        raise ValueError("BinByCoordinates: dmax_coords must be greater than zero.")
    if bin_width is None:
        if n_bins is None:
            raise ValueError("Either bin_width or n_bins must be provided.")
        nb = np.asarray(n_bins, dtype=np.int64)
        if nb.ndim == 0:
            nb = np.repeat(nb, c.shape[1])
        bw = (dmax / nb.astype(np.float32)).astype(np.float32)
        bw = np.array([bw.max()], dtype=np.float32)
    else:
        bw = _c(bin_width, np.float32).reshape(-1)
        if n_bins is None:
            nb = (dmax / bw).astype(np.float32).astype(np.int64) + 1
        else:
            nb = np.asarray(n_bins, dtype=np.int64)
            if nb.ndim == 0:
                nb = np.repeat(nb, c.shape[1])
    if not np.all(nb > 0):
        raise ValueError("BinByCoordinates: n_bins must be greater than zero.")
    if not np.all(bw > 0):
        raise ValueError("BinByCoordinates: bin_width must be greater than zero.")
    return np.ascontiguousarray(c), bw, np.ascontiguousarray(nb)


def bin_points(norm_coords, row_splits, bin_width, n_bins, calc_n_per_bin=True, use_ref=False):
    """The per-point kernel (`calc`, bin_by_coordinates_cpu.cpp:7-99)."""
    c = _c(norm_coords, np.float32)
    rs = _c(row_splits, np.int64)
    nb = _c(n_bins, np.int64)
    n, d = c.shape
    B = int(np.prod(nb)) * (len(rs) - 1)
    assigned = np.zeros((n, d + 1), dtype=np.int64)
    flat = np.zeros(n, dtype=np.int64)
    nper = np.zeros(B, dtype=np.int64)
    bw = float(np.float32(np.asarray(bin_width).reshape(-1)[0]))
    if use_ref:
        r = ref_lib()
        rc = r.fgc_ref_bin_points(_fp(c), _ip(rs), ctypes.c_float(bw), _ip(nb), _ip(assigned),
                                  _ip(flat), _ip(nper), ctypes.c_int64(n), ctypes.c_int64(d),
                                  ctypes.c_int64(len(rs)))
        if rc:
            raise RuntimeError("reference bin_by_coordinates_cpu_fn raised")
        return assigned, flat, nper, 0
    clamped = lib().fgc_oracle_bin_points(
        _fp(c), _ip(rs), ctypes.c_float(bw), _ip(nb), _ip(assigned), _ip(flat), _ip(nper),
        ctypes.c_int64(n), ctypes.c_int64(d), ctypes.c_int64(len(rs)), ctypes.c_int64(B),
        ctypes.c_int(1 if calc_n_per_bin else 0))
    return assigned, flat, nper, int(clamped)


def bin_by_coordinates(coordinates, row_splits, bin_width=None, n_bins=None,
                       calc_n_per_bin=True, pre_normalized=False, use_ref=False):
    """bin_by_coordinates.py:11-111 -> (assigned [N,Db+1], flat [N], n_bins [Db],
    bin_width [1], n_per_bin [B])."""
    c, bw, nb = normalise(coordinates, bin_width, n_bins, pre_normalized)
    assigned, flat, nper, _ = bin_points(c, row_splits, bw, nb, calc_n_per_bin, use_ref)
    return assigned, flat, nb, bw, nper


# --------------------------------------------------------------------------
# binned_select_knn
# --------------------------------------------------------------------------
def optimal_n_bins(row_splits, K, max_bin_dims):
    """calculate_optimal_bins, binned_knn_autograd_kernel.cpp:67-82.  Divides by
    len(row_splits) (events + 1), truncates twice, clamps to [5, 30]."""
    import torch
    rs = torch.as_tensor(np.asarray(row_splits, dtype=np.int64))
    if rs.numel() > 0:
        elems = (rs.max().to(torch.float32) / float(rs.numel()) + 1).to(torch.int64)
    else:
        elems = torch.tensor(1, dtype=torch.int64)
    k32 = np.float32(K) / np.float32(32.0)
    n = torch.pow(elems.to(torch.float32) / float(k32), float(np.float32(1.0) / np.float32(max_bin_dims)))
    n = n.to(torch.int64)
    return int(torch.clamp(n, 5, 30))


def knn_sorted(scoords, sbin, sdbin, bin_boundaries, n_bins, bin_width, K, sdirection=None,
               tf_compat=False, n_threads=1, use_ref=False, query_stride=1, query_offset=0):
    """The kNN kernel in bin-sorted space (select_knn_kernel_cpu,
    binned_select_knn_cpu.cpp:56-208).  Returns (idx, dist, C_eval, d_stop)."""
    c = _c(scoords, np.float32)
    n, D = c.shape
    sbin = _c(sbin, np.int64)
    sdbin = _c(sdbin, np.int64)
    bb = _c(bin_boundaries, np.int64)
    nb = _c(n_bins, np.int64)
    bw = np.array([np.float32(np.asarray(bin_width).reshape(-1)[0])], dtype=np.float32)
    use_dir = sdirection is not None and len(sdirection) > 0
    sdir = _c(sdirection, np.int64) if use_dir else np.zeros(1, dtype=np.int64)
    idx = np.empty((n, K), dtype=np.int64)
    dist = np.empty((n, K), dtype=np.float32)
    if use_ref:
        r = ref_lib()
        rc = r.fgc_ref_knn_sorted(_fp(c), _ip(sbin), _ip(sdir), _ip(sdbin), _ip(bb), _ip(nb),
                                  ctypes.c_float(float(bw[0])), _ip(idx), _fp(dist),
                                  ctypes.c_int64(n), ctypes.c_int64(K), ctypes.c_int64(D),
                                  ctypes.c_int64(len(nb)), ctypes.c_int64(len(bb)),
                                  ctypes.c_int(int(tf_compat)), ctypes.c_int(int(use_dir)))
        if rc:
            raise RuntimeError("reference binned_select_knn_cpu raised")
        return idx, dist, None, None
    d_stop = np.zeros(n, dtype=np.int64)
    evals = lib().fgc_oracle_knn_sorted(
        _fp(c), _ip(sbin), _ip(sdir), _ip(sdbin), _ip(bb), _ip(nb), _fp(bw), _ip(idx), _fp(dist),
        ctypes.c_int64(n), ctypes.c_int64(K), ctypes.c_int64(D), ctypes.c_int64(len(nb)),
        ctypes.c_int64(len(bb)), ctypes.c_int(int(tf_compat)), ctypes.c_int(int(use_dir)),
        _ip(d_stop), ctypes.c_int(int(n_threads)), ctypes.c_int64(int(query_stride)),
        ctypes.c_int64(int(query_offset)))
    if evals < 0:
        raise ValueError("Unsupported number of binning dimensions.")
    return idx, dist, int(evals), d_stop


def sorted_space(coords, row_splits, K, n_bins=None, max_bin_dims=3, direction=None):
    """Everything of BinnedKNNAutograd::forward before the kernel call
    (binned_knn_autograd_kernel.cpp:100-139): n_bins policy, binning of the first
    Db coordinates, stable sort by flat bin, gathers, bin boundaries."""
    c = _c(coords, np.float32)
    rs = _c(row_splits, np.int64)
    n, D = c.shape
    Db = min(int(max_bin_dims), D)
    if n_bins is None:
        n_bins = optimal_n_bins(rs, K, Db)
    dbin, fbin, nb, bw, nper = bin_by_coordinates(np.ascontiguousarray(c[:, :Db]), rs, None, n_bins)
    order = np.argsort(fbin, kind="stable").astype(np.int64)
    bb = np.concatenate([np.zeros(1, np.int64), np.cumsum(nper, dtype=np.int64)])
    if n and int(bb.max()) != int(rs.max()):
        raise RuntimeError("Bin boundaries do not match row splits.")
    sdir = None
    if direction is not None and len(direction) > 0:
        sdir = _c(direction, np.int64)[order]
    return dict(order=order, scoords=np.ascontiguousarray(c[order]), sbin=fbin[order],
                sdbin=np.ascontiguousarray(dbin[order]), bin_boundaries=bb, n_bins=nb,
                bin_width=bw, sdirection=sdir, dbin=dbin, fbin=fbin, n_per_bin=nper)


def binned_select_knn(K, coords, row_splits, direction=None, n_bins=None, max_bin_dims=3,
                      torch_compatible_indices=False, n_threads=1, use_ref=False,
                      return_stats=False):
    """binned_select_knn.py:12-94 + BinnedKNNAutograd::forward
    (binned_knn_autograd_kernel.cpp:85-209): returns (idx int64 [N,K], distsq
    float32 [N,K]) in the original point order; slot 0 is the query itself."""
    c = _c(coords, np.float32)
    if c.ndim != 2 or c.shape[1] == 0:
        raise ValueError("Input coordinates must have at least one dimension. Got 0 dimensions.")
    if max_bin_dims == 0:
        raise ValueError("max_bin_dims must be greater than 0. Got 0.")
    mbd = max(min(int(max_bin_dims), c.shape[1], 5), 2)
    s = sorted_space(c, row_splits, K, n_bins, mbd, direction)
    if len(s["n_bins"]) < 2 or len(s["n_bins"]) > 5:
        raise ValueError("Unsupported number of binning dimensions.")
    idx_s, dist_s, evals, d_stop = knn_sorted(
        s["scoords"], s["sbin"], s["sdbin"], s["bin_boundaries"], s["n_bins"], s["bin_width"], K,
        s["sdirection"], torch_compatible_indices, n_threads, use_ref)
    order = s["order"]
    idx_u = index_replacer(idx_s, order)
    idx = np.empty_like(idx_u)
    dist = np.empty_like(dist_s)
    idx[order] = idx_u
    dist[order] = dist_s
    if return_stats:
        ds = None
        if d_stop is not None:
            ds = np.empty_like(d_stop)
            ds[order] = d_stop
        return idx, dist, dict(C_eval=evals, d_stop=ds, n_bins=s["n_bins"], bin_width=s["bin_width"])
    return idx, dist


def knn_brute(K, coords, row_splits):
    """Exact kNN per event by exhaustive search, rows sorted by distance with
    the query itself first (the definition the shell search must reproduce)."""
    c = _c(coords, np.float32)
    rs = _c(row_splits, np.int64)
    n, D = c.shape
    idx = np.empty((n, K), dtype=np.int64)
    dist = np.empty((n, K), dtype=np.float32)
    lib().fgc_oracle_knn_brute(_fp(c), _ip(rs), ctypes.c_int64(len(rs)), ctypes.c_int64(K),
                               ctypes.c_int64(D), _ip(idx), _fp(dist))
    return idx, dist


def index_replacer(to_be_replaced, replacements, use_ref=False):
    """index_replacer_cpu_kernel, index_replacer_cpu.cpp:7-26."""
    a = _c(to_be_replaced, np.int64)
    r = _c(replacements, np.int64)
    out = np.empty_like(a)
    if use_ref:
        rc = ref_lib().fgc_ref_index_replacer(_ip(a), _ip(r), _ip(out), ctypes.c_int64(a.size),
                                              ctypes.c_int64(r.size))
        if rc:
            raise RuntimeError("reference index_replacer_cpu_fn raised")
        return out
    lib().fgc_oracle_index_replacer(_ip(a), _ip(r), _ip(out), ctypes.c_int64(a.size),
                                    ctypes.c_int64(r.size))
    return out


def knn_grad(grad_dist, idx, coords, dist=None, use_ref=False):
    """binned_select_knn_grad_cpu_fn, binned_select_knn_grad_cpu.cpp:96-165."""
    g = _c(grad_dist, np.float32)
    i = _c(idx, np.int64)
    c = _c(coords, np.float32)
    n, D = c.shape
    K = i.shape[1]
    out = np.zeros((n, D), dtype=np.float32)
    if use_ref:
        d = _c(dist if dist is not None else np.zeros_like(g), np.float32)
        rc = ref_lib().fgc_ref_knn_grad(_fp(g), _ip(i), _fp(d), _fp(c), _fp(out), ctypes.c_int64(n),
                                        ctypes.c_int64(K), ctypes.c_int64(D))
        if rc:
            raise RuntimeError("reference binned_select_knn_grad_cpu_fn raised")
        return out
    lib().fgc_oracle_knn_grad(_fp(g), _ip(i), _fp(c), _fp(out), ctypes.c_int64(n),
                              ctypes.c_int64(K), ctypes.c_int64(D))
    return out


# --------------------------------------------------------------------------
# GravNet aggregation
# --------------------------------------------------------------------------
def select_with_default(idx, feat, default_value):
    """oc_helper.py:232-271: out[v,k,:] = feat[idx[v,k]] or default where idx == -1."""
    idx = np.asarray(idx).astype(np.int64)
    feat = np.asarray(feat)
    out = np.full(idx.shape + (feat.shape[1],), default_value, dtype=feat.dtype)
    m = idx != -1
    out[m] = feat[idx[m]]
    return out


def gravnet_aggregate(idx, distsq, feat):
    """C aggregation kernel: (fmean [N,P], fmax [N,P], argmax [N,P])."""
    i = _c(idx, np.int64)
    d = _c(distsq, np.float32)
    f = _c(feat, np.float32)
    n, K = i.shape
    P = f.shape[1]
    fmean = np.empty((n, P), dtype=np.float32)
    fmax = np.empty((n, P), dtype=np.float32)
    am = np.empty((n, P), dtype=np.int64)
    lib().fgc_oracle_gravnet_agg_fwd(_ip(i), _fp(d), _fp(f), _fp(fmean), _fp(fmax), _ip(am),
                                     ctypes.c_int64(n), ctypes.c_int64(K), ctypes.c_int64(P))
    return fmean, fmax, am


def gravnet_aggregate_torch(idx, distsq, feat):
    """The same aggregation composed from stock torch ops exactly as
    gnn_ops.py:90-102 does (differentiable: autograd gives the reference
    backward).  idx: LongTensor [N,K]; distsq [N,K]; feat [N,P]."""
    import torch
    w = torch.exp(-10. * distsq)
    V, K = idx.shape
    out = torch.full((V, K, feat.shape[1]), 0.0, dtype=feat.dtype)
    valid = idx != -1
    pos = valid.nonzero()
    out[pos[:, 0], pos[:, 1]] = feat[idx[valid]]
    out = out * w.unsqueeze(-1)
    return torch.mean(out, dim=1), torch.max(out, dim=1).values


def gravnet_forward_torch(x, row_splits, weights, k, n_threads=8):
    """GravNetOp.forward (gnn_ops.py:66-109) on CPU: torch Linear layers, the
    oracle kNN with its gradient, the torch aggregation.  `weights` is a dict
    with the reference module's state_dict names.  Returns (out, idx, distsq,
    space); differentiable wrt x and the weights."""
    import torch

    class _KNN(torch.autograd.Function):
        @staticmethod
        def forward(ctx, space):
            idx, dist = binned_select_knn(k, space.detach().numpy(), row_splits, n_threads=n_threads)
            idx_t, dist_t = torch.from_numpy(idx), torch.from_numpy(dist)
            ctx.save_for_backward(idx_t, space.detach())
            ctx.mark_non_differentiable(idx_t)
            return idx_t, dist_t

        @staticmethod
        def backward(ctx, _gi, gd):
            idx_t, space = ctx.saved_tensors
            return torch.from_numpy(knn_grad(gd.contiguous().numpy(), idx_t.numpy(), space.numpy()))

    lin = torch.nn.functional.linear
    space = lin(x, weights["space_transformations.weight"], weights["space_transformations.bias"])
    prop = lin(x, weights["propagate_transformations.weight"], weights["propagate_transformations.bias"])
    idx, distsq = _KNN.apply(space.contiguous())
    fmean, fmax = gravnet_aggregate_torch(idx, distsq, prop)
    cat = torch.cat([x, fmean, fmax], dim=1)
    out = torch.relu(lin(cat, weights["output_transformations.0.weight"],
                         weights["output_transformations.0.bias"]))
    return out, idx, distsq, space


# --------------------------------------------------------------------------
# object-condensation helper matrices
# --------------------------------------------------------------------------
def max_same_valued_entries_per_row_split(asso_idx, row_splits, filter_negative=True, use_ref=False):
    """oc_helper_helper.cpp:30-94: per row split the largest multiplicity of one value and the number of
    distinct values (negative values dropped first when filter_negative), and the maximum over the splits."""
    a = _c(asso_idx, np.int64)
    rs = _c(row_splits, np.int64)
    n_rs = len(rs) - 1
    mx = np.zeros(n_rs, dtype=np.int64)
    nobj = np.zeros(n_rs, dtype=np.int64)
    if use_ref:
        g = np.zeros(1, dtype=np.int64)
        rc = ref_lib().fgc_ref_max_same_valued(_ip(a), _ip(rs), _ip(mx), _ip(g), _ip(nobj),
                                               ctypes.c_int64(a.size), ctypes.c_int64(len(rs)),
                                               ctypes.c_int(int(filter_negative)))
        if rc:
            raise RuntimeError("reference max_same_valued_entries_per_row_split raised")
        return mx, int(g[0]), nobj
    for r in range(n_rs):
        sl = a[rs[r]:rs[r + 1]]
        if filter_negative:
            sl = sl[sl >= 0]
        if sl.size == 0:
            continue
        vals, counts = np.unique(sl, return_counts=True)
        mx[r] = counts.max()
        nobj[r] = vals.size
    return mx, int(mx.max()) if n_rs > 0 else 0, nobj


def oc_helper_inputs(truth_indices, row_splits, filter_negative=True):
    """_helper_inputs, oc_helper.py:18-149: the distinct (value, row split) pairs with value != -1 (and >= 0
    when filter_negative), here ordered by (row split, value); the reference orders them by an unstable argsort
    over the row split (oc_helper.py:196-198), so only the set of pairs is defined.  Returns (unique_vals,
    unique_row_splits, max_same_unique_per_split, lengths, max_length, objects_per_split)."""
    a = _c(truth_indices, np.int64)
    rs = _c(row_splits, np.int64)
    lengths = rs[1:] - rs[:-1]
    uv, ur = [], []
    for r in range(len(rs) - 1):
        sl = a[rs[r]:rs[r + 1]]
        sl = sl[sl != -1]
        if filter_negative:
            sl = sl[sl >= 0]
        v = np.unique(sl)
        uv.append(v)
        ur.append(np.full(v.size, r, dtype=np.int64))
    uv = np.concatenate(uv) if uv else np.zeros(0, np.int64)
    ur = np.concatenate(ur) if ur else np.zeros(0, np.int64)
    _, gmax, nobj = max_same_valued_entries_per_row_split(a, rs, filter_negative)
    return uv, ur, gmax, lengths, int(lengths.max()), nobj


def oc_calc_m(asso_idx, unique_idx, unique_rs_asso, row_splits, n_maxuq, n_maxrs, calc_m_not=True,
              use_ref=False):
    """oc_helper_cpu, oc_helper_cpu.cpp:118-156 (calc_m :17-82).  Returns (M [U, n_maxuq], M_not [U, n_maxrs]
    or None when calc_m_not is False: the reference leaves that buffer uninitialised on the CPU and returns a
    [0, 0] tensor from its CUDA twin, oc_helper_cuda_kernel.cu:171-176)."""
    a = _c(asso_idx, np.int64)
    uq = _c(unique_idx, np.int64)
    ur = _c(unique_rs_asso, np.int64)
    rs = _c(row_splits, np.int64)
    U = uq.size
    M = np.empty((U, n_maxuq), dtype=np.int64)
    M_not = np.empty((U, n_maxrs), dtype=np.int64) if calc_m_not else None
    if use_ref:
        rc = ref_lib().fgc_ref_oc_helper(_ip(a), _ip(uq), _ip(ur), _ip(rs), _ip(M), _ip(M_not),
                                         ctypes.c_int64(a.size), ctypes.c_int64(U), ctypes.c_int64(len(rs)),
                                         ctypes.c_int64(n_maxuq), ctypes.c_int64(n_maxrs),
                                         ctypes.c_int(int(calc_m_not)))
        if rc:
            raise RuntimeError("reference oc_helper_cpu raised")
        return M, M_not
    f = lib().fgc_oracle_oc_calc_m
    f.restype = ctypes.c_int64
    f(_ip(a), _ip(uq), _ip(ur), _ip(rs), _ip(M), _ip(M_not), ctypes.c_int64(a.size), ctypes.c_int64(U),
      ctypes.c_int64(n_maxuq), ctypes.c_int64(n_maxrs), ctypes.c_int(int(calc_m_not)))
    return M, M_not


def oc_helper_matrices(truth_idxs, row_splits, calc_m_not=True, use_ref=False):
    """oc_helper_matrices, oc_helper.py:152-229: (M, M_not, objects_per_split); rows ordered by (row split,
    value)."""
    uv, ur, gmax, _lengths, max_len, nobj = oc_helper_inputs(truth_idxs, row_splits, True)
    M, M_not = oc_calc_m(truth_idxs, uv, ur, row_splits, gmax, max_len, calc_m_not, use_ref=use_ref)
    return M, M_not, nobj


def oc_sort_rows(M, M_not):
    """The canonical form the reference's tests compare in (tests/test_oc_helper.py:11-26): entries of every
    row ascending with -1 last, rows ordered by their first M entry."""
    def rows_sorted(A):
        if A.size == 0:
            return A
        big = A.max() + 100
        key = np.where(A == -1, big, A)
        return np.take_along_axis(A, np.argsort(key, axis=1, kind="stable"), axis=1)
    M = rows_sorted(np.asarray(M))
    M_not = rows_sorted(np.asarray(M_not)) if M_not is not None else None
    order = np.argsort(M[:, 0], kind="stable") if M.size else np.arange(M.shape[0])
    return M[order], (M_not[order] if M_not is not None else None)


# --------------------------------------------------------------------------
# brute-force kNN with a radius limit
# --------------------------------------------------------------------------
def select_knn(K, coords, row_splits, max_radius=-1.0, use_ref=False):
    """select_knn_cpu, select_knn_cpu.cpp:158-205 (the mask arguments are unused there)."""
    c = _c(coords, np.float32)
    rs = _c(row_splits, np.int64)
    n, D = c.shape
    idx = np.empty((n, K), dtype=np.int64)
    dist = np.empty((n, K), dtype=np.float32)
    args = (_fp(c), _ip(rs), _ip(idx), _fp(dist), ctypes.c_int64(n), ctypes.c_int64(K), ctypes.c_int64(D),
            ctypes.c_int64(len(rs)), ctypes.c_double(float(max_radius)))
    if use_ref:
        if ref_lib().fgc_ref_select_knn(*args):
            raise RuntimeError("reference select_knn_cpu raised")
    else:
        lib().fgc_oracle_select_knn(*args)
    return idx, dist
