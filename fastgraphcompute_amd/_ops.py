"""Dispatcher registration of the ops behind the Python wrappers.

The reference registers its C++ kernels as torch ops and its wrappers call
them through `torch.ops.*`, which is what makes the wrappers and GravNetOp
TorchScript-scriptable (fastgraphcompute/extensions/bin_by_coordinates.cpp:
143-153, index_replacer.cpp:43-53, binned_select_knn_grad.cpp:58-70,
binned_knn_autograd_kernel.cpp:271-277).  The same schemas are registered here
with `torch.library`; the implementations call libfgc_hip.so through ctypes.
Two ops have no counterpart in the reference: the fused GravNet aggregation and
the float32 select_with_default kernel.
"""
import ctypes
import struct
import threading
import weakref
from typing import List, Optional, Tuple

import torch

from . import _lib, config

_LIBS = []          # keep the Library objects alive
last_stats = {}     # counters of the most recent kNN call when config.collect_stats is set


def _define(ns: str, schema: str):
    try:
        lib = torch.library.Library(ns, "FRAGMENT")
        lib.define(schema)
    except RuntimeError as e:      # already defined (module imported twice under two names)
        if "already" not in str(e) and "multiple" not in str(e).lower():
            raise
        lib = torch.library.Library(ns, "FRAGMENT")
    _LIBS.append(lib)
    return lib


# ------------------------------------------------------------------ bin_by_coordinates
def _bin_by_coordinates_impl(coordinates: torch.Tensor, row_splits: torch.Tensor, bin_width: Optional[torch.Tensor],
                             n_bins: Optional[torch.Tensor], calc_n_per_bin: bool, pre_normalized: bool):
    _lib.require_device(coordinates)
    L = _lib.lib()
    dev = coordinates.device
    coords = coordinates.to(torch.float32).contiguous()
    if coords.dim() != 2:
        raise ValueError("coordinates must be [n_vert, n_coords]")
    n, d = coords.shape
    if d < 1 or d > 5:
        raise ValueError("Unsupported number of binning dimensions.")
    rs = row_splits.to(device=dev, dtype=torch.int64).contiguous()
    n_rs = rs.numel()
    if (bin_width is None or bin_width.numel() == 0) and (n_bins is None or n_bins.numel() == 0):
        raise ValueError("Either bin_width or n_bins must be provided.")
    nb_host = None
    if n_bins is not None and n_bins.numel() > 0:
        nb_t = n_bins.to(torch.int64).cpu()
        if nb_t.dim() == 0:
            nb_t = nb_t.repeat(d)
        nb_host = [int(v) for v in nb_t.tolist()]
        if len(nb_host) != d:
            raise ValueError("bin_by_coordinates: coordinates.size(1) must be equal to nbins.size(0)")
        if not all(v > 0 for v in nb_host):
            raise ValueError("BinByCoordinates: n_bins must be greater than zero.")
    bw_host = 0.0
    have_bw = bin_width is not None and bin_width.numel() > 0
    if have_bw:
        if bin_width.numel() != 1:
            raise ValueError("bin_by_coordinates: bin_width must be a singleton tensor")
        bw_host = float(bin_width.to(torch.float32).reshape(-1)[0].item())
        if not bw_host > 0:
            raise ValueError("BinByCoordinates: bin_width must be greater than zero.")
    if n == 0:
        nb_out = torch.tensor(nb_host if nb_host is not None else [1] * d, dtype=torch.int64, device=dev)
        B = int(torch.prod(nb_out).item()) * max(n_rs - 1, 0)
        return (torch.empty((0, d + 1), dtype=torch.int64, device=dev),
                torch.empty((0,), dtype=torch.int64, device=dev), nb_out,
                torch.tensor([bw_host], dtype=torch.float32, device=dev),
                torch.zeros((B,), dtype=torch.int64, device=dev))
    geom = torch.empty(16, dtype=torch.float32, device=dev)
    status = torch.zeros(4, dtype=torch.int32, device=dev)
    ws_bytes = L.fgc_bin_geometry_workspace_bytes(n)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    nb_arr = _lib.host_i64(nb_host if nb_host is not None else [1] * d)
    with _lib.on_device(dev):
        st = _lib.stream_ptr()
        _lib.check(L.fgc_bin_geometry_f32(_lib.ptr(coords), n, d, d, 1 if have_bw else 0, nb_arr,
                                          1 if nb_host is not None else 0, bw_host, 1 if pre_normalized else 0,
                                          _lib.ptr(geom), _lib.ptr(status), _lib.ptr(ws), ws_bytes, st))
        g = geom.cpu()  # one synchronisation: n_bins sizes the outputs, the flags carry the input checks
        flags = int(g[11:12].view(torch.int32).item())
        if flags & _lib.ST_NONFINITE:
            raise ValueError("BinByCoordinates: input coordinates contain non-finite values")
        nb_final = [int(v) for v in g[6:6 + d].view(torch.int32).tolist()]
        if flags & _lib.ST_BAD_RANGE:
            if not all(v > 0 for v in nb_final):
                raise ValueError("BinByCoordinates: n_bins must be greater than zero.")
            raise ValueError("BinByCoordinates: dmax_coords must be greater than zero.")
        B = max(n_rs - 1, 0)
        for v in nb_final:
            B *= v
        assigned = torch.empty((n, d + 1), dtype=torch.int64, device=dev)
        flat = torch.empty((n,), dtype=torch.int64, device=dev)
        nper = torch.zeros((B,), dtype=torch.int64, device=dev)
        _lib.check(L.fgc_bin_points_f32(_lib.ptr(coords), n, d, d, _lib.ptr(geom), _lib.ptr(rs), n_rs,
                                        _lib.host_i64(nb_final), _lib.ptr(assigned), _lib.ptr(flat),
                                        _lib.ptr(nper) if calc_n_per_bin else None, _lib.ptr(status), st))
    nb_out = torch.tensor(nb_final, dtype=torch.int64, device=dev)
    return assigned, flat, nb_out, geom[5:6].clone(), nper


# ------------------------------------------------------------------ kNN forward / backward
def calculate_optimal_bins(row_splits_host: torch.Tensor, K: int, max_bin_dims: int) -> int:
    """n_bins heuristic of the reference (binned_knn_autograd_kernel.cpp:67-82),
    evaluated with the same float32 tensor ops on the host: points per
    row-split entry (the length of row_splits, not the number of events),
    divided by K/32, to the power 1/dims, truncated, clamped to [5, 30]."""
    rs = row_splits_host
    if rs.numel() > 0:
        elems = (torch.max(rs).to(torch.float32) / float(rs.numel()) + 1).to(torch.int64)
    else:
        elems = torch.tensor(1, dtype=torch.int64)
    k32 = torch.tensor(float(K), dtype=torch.float32) / torch.tensor(32.0, dtype=torch.float32)
    expo = torch.tensor(1.0, dtype=torch.float32) / torch.tensor(float(max_bin_dims), dtype=torch.float32)
    n_bins = torch.pow(elems.to(torch.float32) / float(k32), float(expo)).to(torch.int64)
    return int(torch.clamp(n_bins, 5, 30))


def choose_search_grid(row_splits_host: torch.Tensor, n_coords: int, max_bin_dims: int):
    """(binned dimensions, bins per dimension) of the library's own search grid.

    The grid never changes the result (the search is exact), only the time.  This search prunes with the
    bounding boxes of 64-point chunks of a sort along a Hilbert curve inside each bin, so it wants far coarser bins
    than the reference's thread-per-query shell walk: up to five binned dimensions (the curve then runs through
    all of them) and about 150 chunks per bin row, 300 with four and 1000 with five binned dimensions (optima on 2- to
    10-dimensional point clouds from 5 000 to 1 000 000 points per event).  With config.auto_grid = False the
    reference's heuristic (calculate_optimal_bins) and max_bin_dims are used."""
    rs = row_splits_host
    n_events = max(1, int(rs.numel()) - 1)
    n = int(torch.max(rs)) if rs.numel() > 0 else 0
    nbd = max(2, min(int(n_coords), 5))
    rows = (n / n_events) / 64.0 / (150.0 if nbd <= 3 else (300.0 if nbd == 4 else 1000.0))
    nb = int(round(max(rows, 1.0) ** (1.0 / (nbd - 1))))
    return nbd, max(1, min(nb, 30))


def knn_grad(grad_distsq: torch.Tensor, idx: torch.Tensor, coords: torch.Tensor,
             order: Optional[torch.Tensor] = None) -> torch.Tensor:
    _lib.require_device(grad_distsq, idx, coords)
    L = _lib.lib()
    g = grad_distsq.to(torch.float32).contiguous()
    ii = idx.to(torch.int64).contiguous()
    x = coords.to(torch.float32).contiguous()
    n, D = x.shape
    K = ii.shape[1]
    out = torch.empty((n, D), dtype=torch.float32, device=x.device)
    status = torch.zeros(4, dtype=torch.int32, device=x.device)
    if order is not None:
        order = order.to(device=x.device, dtype=torch.int32).contiguous()
        if order.numel() != n:
            raise ValueError("order must hold one entry per point")
    with _lib.on_device(x.device):
        _lib.check(L.fgc_binned_select_knn_grad_f32(_lib.ptr(g), _lib.ptr(ii), _lib.ptr(x), _lib.ptr(out), n, K, D,
                                                    _lib.ptr(order), _lib.ptr(status), _lib.stream_ptr()))
    _raise_on_bad_index(status, "binned_select_knn_grad")
    return out


def _raise_on_bad_index(status: torch.Tensor, what: str):
    """For the ops that follow neighbour indices supplied by the caller: with config.sync_checks, wait for the op's
    status word and raise if an index named a row that does not exist (the kernels treat such an entry as an empty
    slot and set FGC_ST_BAD_INDEX; the reference would read out of bounds).  The autograd paths, whose indices come
    from the library's own search, do not wait."""
    if config.sync_checks and (int(status[0].item()) & _lib.ST_BAD_INDEX):
        raise IndexError("%s: a neighbour index is not below the number of rows" % what)


_PINNED = threading.local()


def _pinned_status(dev: torch.device) -> torch.Tensor:
    """One pinned int32[4] per device and host thread for the asynchronous read-back of the status word (each use
    ends with a wait on its own event, so the buffer is free again when the thread's next call starts; calls from
    other threads have buffers of their own)."""
    key = dev.index if dev.index is not None else torch.cuda.current_device()
    bufs = getattr(_PINNED, "bufs", None)
    if bufs is None:
        bufs = _PINNED.bufs = {}
    buf = bufs.get(key)
    if buf is None:
        buf = torch.empty(4, dtype=torch.int32, pin_memory=True)
        bufs[key] = buf
    return buf


def knn_grad_sorted(grad_distsq: torch.Tensor, nbr_sorted: torch.Tensor, coords: torch.Tensor,
                    order: torch.Tensor, n_coords: Optional[int] = None,
                    out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """d(loss)/d(coords) from d(loss)/d(distsq) with the neighbour rows and permutation of the forward's sorted
    order (what binned_select_knn keeps for its backward).  With `n_coords` the coordinates are the first n_coords
    columns of the (wider) matrix `coords`, and `out` (same row length as it likes) receives the gradient in its
    first n_coords columns."""
    _lib.require_device(grad_distsq, nbr_sorted, coords, order)
    L = _lib.lib()
    g = grad_distsq.to(torch.float32).contiguous()
    x = coords.to(torch.float32).contiguous()
    n, ld = x.shape
    D = ld if n_coords is None else int(n_coords)
    K = nbr_sorted.shape[1]
    if out is None:
        out = torch.empty((n, D), dtype=torch.float32, device=x.device)
    ws_bytes = L.fgc_binned_select_knn_grad_sorted_workspace_bytes(n, D)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device)
    with _lib.on_device(x.device):
        # no status word: the rows come from the library's own search, and nothing on this path reads it
        _lib.check(L.fgc_binned_select_knn_grad_sorted_ld_f32(
            _lib.ptr(g), _lib.ptr(nbr_sorted), _lib.ptr(x), ld, _lib.ptr(order), _lib.ptr(out), out.stride(0), n, K, D,
            None, _lib.ptr(ws), ws_bytes, _lib.stream_ptr()))
    return out


_RS_HOST = {}       # id(tensor) -> (weak reference, version, data pointer, host copy); guarded by _RS_LOCK
_RS_LOCK = threading.Lock()
_STATS_LOCK = threading.Lock()


def host_row_splits(row_splits: torch.Tensor) -> torch.Tensor:
    """row_splits as an int64 host tensor.  The search is planned on the host, so a device tensor has to be copied
    back, which makes the host wait for everything queued before it.  A model calls the kNN of every layer with the
    same row_splits tensor: the copy is kept for as long as that very tensor object is alive and unmodified
    (object identity, version counter and data pointer are all checked), so only the first call waits.  The table
    is shared between host threads under a lock; when it is full the oldest entry goes."""
    if not row_splits.is_cuda:
        return row_splits.detach().to(torch.int64).contiguous()
    try:
        version = row_splits._version
    except RuntimeError:          # inference tensors have no version counter: no caching
        return row_splits.detach().to("cpu", torch.int64).contiguous()
    key = id(row_splits)
    with _RS_LOCK:
        ent = _RS_HOST.get(key)
    if ent is not None and ent[0]() is row_splits and ent[1] == version and ent[2] == row_splits.data_ptr():
        return ent[3]
    host = row_splits.detach().to("cpu", torch.int64).contiguous()     # the wait happens outside the lock
    with _RS_LOCK:
        _RS_HOST.pop(key, None)
        while len(_RS_HOST) >= 64:
            _RS_HOST.pop(next(iter(_RS_HOST)))                         # dicts keep insertion order: the oldest
        _RS_HOST[key] = (weakref.ref(row_splits), version, row_splits.data_ptr(), host)
    return host


def _knn_forward(coords: torch.Tensor, D: int, row_splits, K: int, direction, n_bins, max_bin_dims: int,
                 tf_compat: bool, want_backward: bool):
    """The whole forward of binned_select_knn on the first D columns of the float32 row-major matrix `coords`.
    Returns (idx, distsq, nbr_sorted, order); the last two (neighbour rows and permutation of the search's sorted
    order) only when a backward will follow."""
    L = _lib.lib()
    dev = coords.device
    n, ld = coords.shape
    nbd = min(int(max_bin_dims), D)
    if nbd < 2 or nbd > 5:
        raise ValueError("Unsupported number of binning dimensions.")
    if K < 1 or K > 1024:
        raise ValueError("binned_select_knn on MI355X supports 1 <= K <= 1024, got %d" % K)
    rs_host = host_row_splits(row_splits)
    plan = None
    plan_key = (n, D, K, nbd, bool(config.auto_grid))
    if n_bins is None or n_bins.numel() == 0:
        # a model calls every layer's search with the same row_splits: what follows from them alone (checks, grid,
        # host arrays, workspace size) is kept with their host copy
        plans = getattr(rs_host, "_fgc_plans", None)     # (dict reads and writes of single keys are atomic)
        plan = plans.get(plan_key) if plans is not None else None
    if plan is None:
        n_rs = rs_host.numel()
        if n_rs < 2:
            raise ValueError("row_splits needs at least two entries")
        cacheable = n_bins is None or n_bins.numel() == 0
        if cacheable:
            if config.auto_grid:
                nbd, nb1 = choose_search_grid(rs_host, D, nbd)
                nb = [nb1] * nbd
            else:
                nb = [calculate_optimal_bins(rs_host, K, nbd)] * nbd
        else:
            nbt = n_bins.detach().to("cpu", torch.int64)
            nb = [int(nbt.item())] * nbd if nbt.numel() == 1 else [int(v) for v in nbt.tolist()]
            if len(nb) != nbd:
                raise ValueError("bin_by_coordinates: coordinates.size(1) must be equal to nbins.size(0)")
            if not all(v > 0 for v in nb):
                raise RuntimeError("BinByCoordinates: n_bins must be greater than zero.")
        rs_list = rs_host.tolist()
        if n > 0 and (rs_list[0] != 0 or max(rs_list) != n or rs_list[-1] != n
                      or any(b < a for a, b in zip(rs_list, rs_list[1:]))):
            raise RuntimeError("Bin boundaries do not match row splits.")
        nb_arr = _lib.host_i64(nb)
        rs_arr = _lib.host_i64(rs_list)
        ws_bytes = L.fgc_binned_select_knn_workspace_bytes(n, D, nbd, nb_arr, n_rs, K) if n > 0 else 0
        plan = (nbd, nb, nb_arr, rs_arr, n_rs, ws_bytes)
        if cacheable and row_splits.is_cuda:
            # (rs_host is then the library's own copy, which nothing modifies; it lives as long as the row_splits tensor)
            if getattr(rs_host, "_fgc_plans", None) is None:
                rs_host._fgc_plans = {}
            rs_host._fgc_plans[plan_key] = plan
    nbd, nb, nb_arr, rs_arr, n_rs, ws_bytes = plan
    rs_dev = row_splits if (row_splits.is_cuda and row_splits.dtype == torch.int64) else rs_host.to(dev)
    rs_dev = rs_dev.contiguous()
    idx = torch.empty((n, K), dtype=torch.int64, device=dev)
    dist = torch.empty((n, K), dtype=torch.float32, device=dev)
    order = None
    nbr_sorted = None
    if n > 0:
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
        status = torch.zeros(4, dtype=torch.int32, device=dev)
        stats = torch.zeros(8, dtype=torch.int64, device=dev) if config.collect_stats else None
        dirt = None
        if direction is not None and direction.numel() > 0:
            dirt = direction.to(device=dev, dtype=torch.int64).contiguous()
        with _lib.on_device(dev):
            st = _lib.stream_ptr()
            # prepare and search are enqueued separately so that the input checks (status word, written by
            # the prepare stage) can be read back while the search is already queued behind them: the host
            # then waits for the short prepare stage only and the device never runs dry
            _lib.check(L.fgc_binned_knn_prepare_ld_f32(
                _lib.ptr(coords), n, D, ld, _lib.ptr(rs_dev), rs_arr, n_rs, K, nbd, nb_arr, _lib.ptr(dirt),
                _lib.ptr(status), _lib.ptr(ws), ws_bytes, st))
            checked = None
            if config.sync_checks:
                status_host = _pinned_status(dev)
                status_host.copy_(status, non_blocking=True)
                checked = torch.cuda.Event()
                checked.record()
            if want_backward:
                # the backward works in the search's sorted order: it gets the neighbour rows in that order
                # (int32) and the permutation
                nbr_sorted = torch.empty((n, K), dtype=torch.int32, device=dev)
            _lib.check(L.fgc_binned_knn_search_f32(
                n, D, rs_arr, n_rs, K, nbd, nb_arr, 1 if dirt is not None else 0,
                (_lib.KNN_TF_COMPAT if tf_compat else 0) | (0 if config.sorted_neighbours else _lib.KNN_ANY_ORDER)
                | (_lib.KNN_FORCE_MATRIX if config.matrix_search == "always" else
                   (0 if config.matrix_search else _lib.KNN_NO_MATRIX)),
                _lib.ptr(idx), _lib.ptr(dist), _lib.ptr(nbr_sorted), _lib.ptr(stats), _lib.ptr(ws), ws_bytes, st))
            if want_backward:
                order = torch.empty(n, dtype=torch.int32, device=dev)
                _lib.check(L.fgc_binned_knn_export_order_i32(n, D, rs_arr, n_rs, K, nbd, nb_arr,
                                                             1 if dirt is not None else 0, _lib.ptr(ws),
                                                             ws_bytes, _lib.ptr(order), st))
        if checked is not None:
            checked.synchronize()
            flags = int(status_host[0])
            if flags & _lib.ST_NONFINITE:
                raise RuntimeError("BinByCoordinates: input coordinates contain non-finite values")
            if flags & _lib.ST_BAD_RANGE:
                raise RuntimeError("BinByCoordinates: dmax_coords must be greater than zero.")
        if stats is not None:
            s = stats.tolist()
            with _STATS_LOCK:
                last_stats.update(distance_evaluations=s[0], candidate_chunks=s[1], pool_prunes=s[2],
                                  matrix_search_handed_over=s[3], matrix_search_collected=s[5],
                                  n_bins=nb, n_vert=n, K=K, n_coords=D)
    if nbr_sorted is None:
        nbr_sorted = torch.empty((0, K), dtype=torch.int32, device=dev)
    if order is None:
        order = torch.empty(0, dtype=torch.int32, device=dev)
    return idx, dist, nbr_sorted, order


class _BinnedKNN(torch.autograd.Function):
    @staticmethod
    def forward(ctx, coords, row_splits, K, direction, n_bins, max_bin_dims, tf_compat):
        _lib.require_device(coords)
        if coords.dim() != 2 or coords.shape[1] == 0:
            raise ValueError("Input coordinates must have at least one dimension.")
        if max_bin_dims <= 0:
            raise ValueError("max_bin_dims must be greater than 0.")
        coords = coords.to(torch.float32).contiguous()
        idx, dist, nbr_sorted, order = _knn_forward(coords, coords.shape[1], row_splits, K, direction, n_bins,
                                                    max_bin_dims, tf_compat, ctx.needs_input_grad[0])
        ctx.save_for_backward(nbr_sorted, coords, order)
        ctx.mark_non_differentiable(idx)
        ctx.set_materialize_grads(False)   # no zero tensors for unused output gradients
        return idx, dist

    @staticmethod
    def backward(ctx, _grad_idx, grad_dist):
        nbr_sorted, coords, order = ctx.saved_tensors
        if not ctx.needs_input_grad[0]:
            return None, None, None, None, None, None, None
        if grad_dist is None or coords.shape[0] == 0:
            return torch.zeros_like(coords), None, None, None, None, None, None
        g = knn_grad_sorted(grad_dist, nbr_sorted, coords, order)
        return g, None, None, None, None, None, None


def _knn_autograd_impl(coords, row_splits, K, direction, n_bins, max_bin_dims, torch_compatible_indices):
    return _BinnedKNN.apply(coords, row_splits, K, direction, n_bins, max_bin_dims, torch_compatible_indices)


def _knn_sorted_space_impl(coordinates, bin_idx, dim_bin_idx, bin_boundaries, n_bins, bin_width, direction,
                           tf_compat: bool, use_direction: bool, K: int):
    """The reference's inner op on already bin-sorted points (binned_select_knn.cpp:82-92): neighbour indices
    refer to the given (sorted) order.  Events are the groups of prod(n_bins) consecutive bins of
    bin_boundaries; the search builds its own grid, so bin_idx, dim_bin_idx and bin_width are not needed."""
    _lib.require_device(coordinates)
    per_event = int(torch.prod(n_bins.detach().to("cpu", torch.int64)))
    bb = bin_boundaries.detach().to("cpu", torch.int64)
    if per_event < 1 or (bb.numel() - 1) % per_event != 0:
        raise RuntimeError("bin_boundaries must hold prod(n_bins) bins per event plus one entry")
    row_splits = bb[::per_event].contiguous()
    d = direction if (use_direction and direction is not None and direction.numel() > 0) else None
    with torch.no_grad():
        idx, dist = _BinnedKNN.apply(coordinates, row_splits, int(K), d, None, 3, bool(tf_compat))
    return idx, dist


def _knn_grad_impl(grad_distances, indices, distances, coordinates):
    return knn_grad(grad_distances, indices, coordinates)


# ------------------------------------------------------------------ index_replacer
def _index_replacer_impl(to_be_replaced: torch.Tensor, replacements: torch.Tensor) -> torch.Tensor:
    _lib.require_device(to_be_replaced, replacements)
    L = _lib.lib()
    src = to_be_replaced.contiguous()
    rep = replacements.contiguous()
    out = torch.empty_like(src)
    with _lib.on_device(src.device):
        _lib.check(L.fgc_index_replacer_i64(_lib.ptr(src), _lib.ptr(rep), _lib.ptr(out), src.numel(), rep.numel(),
                                            _lib.stream_ptr()))
    return out


# ------------------------------------------------------------------ select_with_default (float32 kernel)
class _SelectWithDefault(torch.autograd.Function):
    @staticmethod
    def forward(ctx, idx, feat, default_value):
        _lib.require_device(idx, feat)
        L = _lib.lib()
        ii = idx.to(torch.int64).contiguous()
        ff = feat.contiguous()
        V, K = ii.shape
        rows, F = ff.shape
        out = torch.empty((V, K, F), dtype=ff.dtype, device=ff.device)
        with _lib.on_device(ff.device):
            if ff.dtype == torch.float32:
                _lib.check(L.fgc_select_with_default_f32(_lib.ptr(ii), _lib.ptr(ff), _lib.ptr(out), V, K, F, rows,
                                                         float(default_value), _lib.stream_ptr()))
            elif ff.dtype in (torch.int64, torch.float64):
                # 8-byte elements travel as bit patterns; the default is converted as torch.full would do it
                packed = struct.pack("<q", int(default_value)) if ff.dtype == torch.int64 \
                    else struct.pack("<d", float(default_value))
                _lib.check(L.fgc_select_with_default_b64(_lib.ptr(ii), _lib.ptr(ff), _lib.ptr(out), V, K, F, rows,
                                                         struct.unpack("<Q", packed)[0], _lib.stream_ptr()))
            else:
                raise RuntimeError("select_with_default kernel: unsupported feature dtype %s" % ff.dtype)
        ctx.save_for_backward(ii)
        ctx.rows = rows
        return out

    @staticmethod
    def backward(ctx, g):
        (ii,) = ctx.saved_tensors
        if g is None or not ctx.needs_input_grad[1]:
            return None, None, None
        F = g.shape[-1]
        valid = (ii != -1).reshape(-1)
        tgt = torch.where(ii < 0, ii + ctx.rows, ii).reshape(-1)[valid]
        gf = torch.zeros((ctx.rows, F), dtype=g.dtype, device=g.device)
        gf.index_add_(0, tgt, g.reshape(-1, F)[valid])
        return None, gf, None


def _select_with_default_impl(idx, feat, default_value):
    return _SelectWithDefault.apply(idx, feat, default_value)


# ------------------------------------------------------------------ GravNet aggregation
class _GravNetAggregate(torch.autograd.Function):
    """(fmean, fmax) over the K neighbour slots of feat[idx] * exp(-10 distsq)."""

    @staticmethod
    def forward(ctx, idx, distsq, feat):
        _lib.require_device(idx, distsq, feat)
        L = _lib.lib()
        ii = idx.to(torch.int64).contiguous()
        d = distsq.to(torch.float32).contiguous()
        f = feat.to(torch.float32).contiguous()
        n, K = ii.shape
        P = f.shape[1]
        fmean = torch.empty((n, P), dtype=torch.float32, device=f.device)
        fmax = torch.empty((n, P), dtype=torch.float32, device=f.device)
        argmax = torch.empty((n, P), dtype=torch.int32, device=f.device)
        status = torch.zeros(4, dtype=torch.int32, device=f.device)
        with _lib.on_device(f.device):
            _lib.check(L.fgc_gravnet_aggregate_fwd_ld_f32(_lib.ptr(ii), _lib.ptr(d), _lib.ptr(f), P, f.shape[0],
                                                          _lib.ptr(fmean), _lib.ptr(fmax), P, _lib.ptr(argmax), n, K, P,
                                                          _lib.ptr(status), _lib.stream_ptr()))
        _raise_on_bad_index(status, "gravnet_aggregate")
        ctx.save_for_backward(ii, d, f, argmax)
        ctx.set_materialize_grads(False)
        return fmean, fmax

    @staticmethod
    def backward(ctx, g_mean, g_max):
        ii, d, f, argmax = ctx.saved_tensors
        if g_mean is None and g_max is None:
            return None, None, None
        L = _lib.lib()
        n, K = ii.shape
        P = f.shape[1]
        g_mean = torch.zeros((n, P), dtype=torch.float32, device=f.device) if g_mean is None \
            else g_mean.to(torch.float32).contiguous()
        g_max = torch.zeros((n, P), dtype=torch.float32, device=f.device) if g_max is None \
            else g_max.to(torch.float32).contiguous()
        g_feat = torch.zeros_like(f)
        g_dist = torch.empty_like(d)
        with _lib.on_device(f.device):
            _lib.check(L.fgc_gravnet_aggregate_bwd_f32(_lib.ptr(ii), _lib.ptr(d), _lib.ptr(f), _lib.ptr(argmax),
                                                       _lib.ptr(g_mean), _lib.ptr(g_max), _lib.ptr(g_feat),
                                                       _lib.ptr(g_dist), n, K, P, _lib.stream_ptr()))
        return None, g_dist, g_feat


def _gravnet_aggregate_impl(idx, distsq, feat):
    return _GravNetAggregate.apply(idx, distsq, feat)


class _GravNetLayerCore(torch.autograd.Function):
    """kNN in the learned coordinates plus the neighbour aggregation of one GravNet layer (gnn_ops.py:87-102 of the
    reference) as one autograd node: the aggregation writes (mean | max) side by side into one [N, 2P] matrix for
    the output layer (no concatenation), and the backward chains the aggregation's gradient with respect to the
    squared distances straight into the kNN gradient kernel, reading the output layer's input gradient in place
    (leading dimensions)."""

    @staticmethod
    def forward(ctx, space, features, row_splits, K):
        _lib.require_device(space, features)
        if space.dim() != 2 or features.dim() != 2 or space.shape[0] != features.shape[0] or space.shape[1] == 0:
            raise ValueError("space must be [N, S] and features [N, P]")
        L = _lib.lib()
        coords = space.to(torch.float32).contiguous()
        feat = features.to(torch.float32).contiguous()
        n, P = feat.shape
        dev = feat.device
        idx, dist, nbr_sorted, order = _knn_forward(coords, coords.shape[1], row_splits, K, None, None, 3, False,
                                                    ctx.needs_input_grad[0] or ctx.needs_input_grad[1])
        agg = torch.empty((n, 2 * P), dtype=torch.float32, device=dev)
        argmax = torch.empty((n, P), dtype=torch.int32, device=dev)
        if n > 0:
            with _lib.on_device(dev):
                _lib.check(L.fgc_gravnet_aggregate_fwd_ld_f32(
                    _lib.ptr(idx), _lib.ptr(dist), _lib.ptr(feat), P, n, _lib.ptr(agg),
                    ctypes.c_void_p(agg.data_ptr() + 4 * P), 2 * P, _lib.ptr(argmax), n, K, P, None,
                    _lib.stream_ptr()))
        ctx.save_for_backward(idx, dist, coords, feat, argmax, nbr_sorted, order)
        ctx.mark_non_differentiable(idx)
        ctx.set_materialize_grads(False)
        return idx, dist, agg

    @staticmethod
    def backward(ctx, _g_idx, g_dist, g_agg):
        idx, dist, coords, feat, argmax, nbr_sorted, order = ctx.saved_tensors
        L = _lib.lib()
        n, P = feat.shape
        K = idx.shape[1]
        g_feat = g_dsq = g_space = None
        if n > 0 and g_agg is not None:
            if g_agg.dtype != torch.float32 or g_agg.stride(1) != 1:
                g_agg = g_agg.to(torch.float32).contiguous()
            g_feat = torch.zeros_like(feat)
            g_dsq = torch.empty_like(dist)
            with _lib.on_device(feat.device):
                if config.tile_aggregation_backward and nbr_sorted.shape[0] == n and \
                        L.fgc_gravnet_aggregate_bwd_sorted_supported(n, K, P, P, P):
                    # rows that are neighbours in the search's sorted order share their targets: combined on chip
                    _lib.check(L.fgc_gravnet_aggregate_bwd_sorted_f32(
                        _lib.ptr(nbr_sorted), _lib.ptr(order), _lib.ptr(dist), _lib.ptr(feat), P, _lib.ptr(argmax),
                        _lib.ptr(g_agg), ctypes.c_void_p(g_agg.data_ptr() + 4 * P), g_agg.stride(0), _lib.ptr(g_feat),
                        P, _lib.ptr(g_dsq), n, K, P, None, _lib.stream_ptr()))
                else:
                    _lib.check(L.fgc_gravnet_aggregate_bwd_ld_f32(
                        _lib.ptr(idx), _lib.ptr(dist), _lib.ptr(feat), P, n, _lib.ptr(argmax), _lib.ptr(g_agg),
                        ctypes.c_void_p(g_agg.data_ptr() + 4 * P), g_agg.stride(0), _lib.ptr(g_feat), P,
                        _lib.ptr(g_dsq), n, K, P, None, _lib.stream_ptr()))
        if g_dist is not None:
            g_dsq = g_dist.to(torch.float32) if g_dsq is None else g_dsq + g_dist
        if ctx.needs_input_grad[0]:
            g_space = torch.zeros_like(coords) if (g_dsq is None or n == 0) \
                else knn_grad_sorted(g_dsq, nbr_sorted, coords, order)
        if not ctx.needs_input_grad[1]:
            g_feat = None
        elif g_feat is None:
            g_feat = torch.zeros_like(feat)
        return g_space, g_feat, None, None


def _gravnet_layer_core_impl(space, features, row_splits, K: int):
    return _GravNetLayerCore.apply(space, features, row_splits, K)


class _DenseSplit(torch.autograd.Function):
    """y = [x | a] W^T + b without building [x | a]: two products into one output, and in the backward one product
    for both input gradients (returned as column views of it) and the library's weight-gradient kernel per part."""

    @staticmethod
    def forward(ctx, x, a, weight, bias):
        _lib.require_device(x, a, weight)
        C = x.shape[1]
        ctx.save_for_backward(x, a, weight)
        ctx.has_bias = bias is not None
        w1, w2 = weight[:, :C], weight[:, C:]
        out = torch.addmm(bias, x, w1.t()) if bias is not None else x.matmul(w1.t())
        return out.addmm_(a, w2.t())

    @staticmethod
    def backward(ctx, g):
        x, a, weight = ctx.saved_tensors
        if g is None:
            return None, None, None, None
        g = g.contiguous()
        C = x.shape[1]
        gx = ga = gw = gb = None
        if ctx.needs_input_grad[0] or ctx.needs_input_grad[1]:
            both = g.matmul(weight)                   # [n, C + A]
            gx = both[:, :C] if ctx.needs_input_grad[0] else None
            ga = both[:, C:] if ctx.needs_input_grad[1] else None
        if ctx.needs_input_grad[2] or (ctx.has_bias and ctx.needs_input_grad[3]):
            if x.dtype == torch.float32 and a.dtype == torch.float32 and g.dtype == torch.float32:
                gw1, gb = linear_wgrad(g, x, ctx.has_bias)
                gw2, _ = linear_wgrad(g, a, False)
            else:
                gw1, gw2 = g.t().matmul(x), g.t().matmul(a)
                gb = g.sum(0) if ctx.has_bias else None
            gw = torch.cat([gw1, gw2], dim=1)
        return gx, ga, gw, gb


def _dense_split_impl(x, a, weight, bias):
    return _DenseSplit.apply(x, a, weight, bias)


# ------------------------------------------------------------------ object-condensation helper matrices
def _oc_check_inputs(asso: torch.Tensor, row_splits: torch.Tensor):
    _lib.require_device(asso, row_splits)
    # the reference's argument checks (oc_helper_cuda_kernel.cu:118-152, oc_helper_helper.cpp:43)
    if asso.dtype != torch.int64 or asso.dim() != 1:
        raise RuntimeError("asso_idx should be contiguous and of type int64")
    if row_splits.dtype != torch.int64 or row_splits.dim() != 1:
        raise RuntimeError("row_splits must be of type int64")
    if row_splits.numel() < 2:
        raise RuntimeError("row_splits needs at least two entries")


def _oc_objects(asso: torch.Tensor, row_splits: torch.Tensor, filter_negative: bool):
    """Objects pass of the library plus the single host read the output shapes need.  Returns (workspace,
    summary tensor, n_unique, n_maxuq, host row splits, max_per_split, objects_per_split)."""
    L = _lib.lib()
    dev = asso.device
    a = asso.contiguous()
    rs = row_splits.contiguous()
    n, n_rs = a.numel(), rs.numel()
    ws_bytes = L.fgc_oc_helper_workspace_bytes(n)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    summary = torch.empty(4, dtype=torch.int64, device=dev)
    max_per_split = torch.empty(n_rs - 1, dtype=torch.int64, device=dev)
    objects_per_split = torch.empty(n_rs - 1, dtype=torch.int64, device=dev)
    wide = 0
    while True:
        with _lib.on_device(dev):
            _lib.check(L.fgc_oc_helper_objects_i64(_lib.ptr(a), n, _lib.ptr(rs), n_rs, int(filter_negative), wide,
                                                   _lib.ptr(max_per_split), _lib.ptr(objects_per_split),
                                                   _lib.ptr(summary), _lib.ptr(ws), ws_bytes, _lib.stream_ptr()))
        host = torch.cat([summary, rs]).cpu()          # the one synchronisation of the call
        if wide == 0 and (int(host[2]) & 1):
            wide = 1                                    # a value needs more bits than the narrow key has
            continue
        break
    rs_host = host[4:]
    if int(rs_host[0]) != 0 or int(rs_host[-1]) != n or bool((rs_host[1:] < rs_host[:-1]).any()):
        raise ValueError("row_splits must start at 0, end at the number of vertices and not decrease")
    return a, rs, ws, ws_bytes, summary, int(host[0]), int(host[1]), rs_host, max_per_split, objects_per_split


def _oc_helper_matrices_impl(truth_idxs: torch.Tensor, row_splits: torch.Tensor, calc_m_not: bool):
    if truth_idxs.device != row_splits.device:
        raise AssertionError("Both truth_idxs and row_splits must be on the same device")
    _oc_check_inputs(truth_idxs, row_splits)
    L = _lib.lib()
    a, rs, ws, ws_bytes, summary, n_unique, n_maxuq, rs_host, _mx, objects_per_split = _oc_objects(
        truth_idxs, row_splits, True)
    dev = a.device
    n_maxrs = int((rs_host[1:] - rs_host[:-1]).max())
    M = torch.empty((n_unique, n_maxuq), dtype=torch.int64, device=dev)
    # without M_not the reference's device op hands back an empty [0, 0] tensor (oc_helper_cuda_kernel.cu:171-176)
    M_not = torch.empty((n_unique, n_maxrs) if calc_m_not else (0, 0), dtype=torch.int64, device=dev)
    with _lib.on_device(dev):
        _lib.check(L.fgc_oc_helper_fill_i64(a.numel(), _lib.ptr(rs), rs.numel(), n_unique, n_maxuq, n_maxrs, None, None,
                                            _lib.ptr(summary), _lib.ptr(M), _lib.ptr(M_not) if calc_m_not else None,
                                            None, None, None, _lib.ptr(ws), ws_bytes, _lib.stream_ptr()))
    return M, M_not, objects_per_split


def _oc_helper_cuda_impl(asso_idx: torch.Tensor, unique_idx: torch.Tensor, unique_rs_asso: torch.Tensor,
                         rs: torch.Tensor, max_n_unique_over_splits: torch.Tensor, max_n_in_splits: torch.Tensor,
                         calc_m_not: bool):
    """The reference's device op (oc_helper_cuda_kernel.cu:154-203): objects and widths come from the caller."""
    _oc_check_inputs(asso_idx, rs)
    for t, name in ((unique_idx, "unique_idx"), (unique_rs_asso, "unique_rs_asso"),
                    (max_n_unique_over_splits, "max_n_unique_over_splits"), (max_n_in_splits, "max_n_in_splits")):
        if t.dtype != torch.int64 or not t.is_contiguous():
            raise RuntimeError(name + " should be contiguous and of type int64")
        if t.device != asso_idx.device:
            raise RuntimeError("All inputs should be on the same device")
    if max_n_unique_over_splits.dim() != 1 or max_n_unique_over_splits.size(0) != 1:
        raise RuntimeError("max_n_unique_over_splits should have size 1")
    if max_n_in_splits.dim() != 1 or max_n_in_splits.size(0) != 1:
        raise RuntimeError("max_n_in_splits should have size 1")
    if unique_idx.numel() != unique_rs_asso.numel() or unique_idx.numel() > max(asso_idx.numel(), 0):
        raise RuntimeError("unique_idx and unique_rs_asso must list each object of asso_idx once")
    L = _lib.lib()
    dev = asso_idx.device
    widths = torch.cat([max_n_unique_over_splits, max_n_in_splits]).cpu()
    n_maxuq, n_maxrs = int(widths[0]), int(widths[1])
    # negative association indices are objects too when the caller lists them
    a, rsd, ws, ws_bytes, summary, _nu, _nm, _rs_host, _mx, _ops = _oc_objects(asso_idx, rs, False)
    n_rows = unique_idx.numel()
    M = torch.empty((n_rows, n_maxuq), dtype=torch.int64, device=dev)
    M_not = torch.empty((n_rows, n_maxrs) if calc_m_not else (0, 0), dtype=torch.int64, device=dev)
    status = torch.zeros(4, dtype=torch.int32, device=dev)
    with _lib.on_device(dev):
        _lib.check(L.fgc_oc_helper_fill_i64(a.numel(), _lib.ptr(rsd), rsd.numel(), n_rows, n_maxuq, n_maxrs,
                                            _lib.ptr(unique_idx), _lib.ptr(unique_rs_asso), _lib.ptr(summary),
                                            _lib.ptr(M), _lib.ptr(M_not) if calc_m_not else None, None, None,
                                            _lib.ptr(status), _lib.ptr(ws), ws_bytes, _lib.stream_ptr()))
    if config.sync_checks and (int(status[0]) & _lib.ST_OC_TRUNCATED):
        raise RuntimeError("an object has more vertices than max_n_unique_over_splits")
    return M, M_not


def _max_same_valued_impl(asso_idx: torch.Tensor, row_splits: torch.Tensor, filter_negative: bool):
    """max_same_valued_entries_per_row_split (oc_helper_helper.cpp:30-94); row_splits may live on the host as in
    the reference, the results are on asso_idx's device."""
    if row_splits.dtype != torch.int64:
        raise RuntimeError("row_splits must be of type int64")
    rs = row_splits.to(asso_idx.device)
    _oc_check_inputs(asso_idx, rs)
    out = _oc_objects(asso_idx, rs, filter_negative)
    max_per_split, objects_per_split = out[8], out[9]
    return max_per_split, max_per_split.max(), objects_per_split


# ------------------------------------------------------------------ brute-force style kNN with a radius limit
def _select_knn_impl(coords: torch.Tensor, row_splits: torch.Tensor, mask: torch.Tensor, n_neighbours: int,
                     max_radius: float, mask_mode: int):
    """select_knn of the reference (select_knn.cpp:60-70): neighbours of the same event within max_radius.
    mask and mask_mode are accepted and ignored, as in both of the reference's implementations."""
    _lib.require_device(coords, row_splits)
    if coords.dim() != 2 or coords.shape[1] == 0:
        raise ValueError("coords must be [n_vert, n_coords]")
    K = int(n_neighbours)
    if K < 1 or K > 1024:
        raise ValueError("select_knn on MI355X supports 1 <= n_neighbours <= 1024, got %d" % K)
    L = _lib.lib()
    dev = coords.device
    x = coords.to(torch.float32).contiguous()
    n, D = x.shape
    rs_host = row_splits.detach().to("cpu", torch.int64).contiguous()
    rs_list = rs_host.tolist()
    n_rs = len(rs_list)
    if n_rs < 2 or (n > 0 and (rs_list[0] != 0 or rs_list[-1] != n or any(b < a for a, b in zip(rs_list, rs_list[1:])))):
        raise RuntimeError("row_splits must start at 0, end at the number of points and not decrease")
    idx = torch.empty((n, K), dtype=torch.int64, device=dev)
    dist = torch.empty((n, K), dtype=torch.float32, device=dev)
    if n == 0:
        return idx, dist
    if D == 1:                       # the search bins at least two coordinates: add a constant one
        x = torch.cat([x, torch.zeros_like(x)], dim=1).contiguous()
        D = 2
    nbd, nb1 = choose_search_grid(rs_host, D, 3)
    nb_arr, rs_arr = _lib.host_i64([nb1] * nbd), _lib.host_i64(rs_list)
    rs_dev = rs_host.to(dev)
    ws_bytes = L.fgc_binned_select_knn_workspace_bytes(n, D, nbd, nb_arr, n_rs, K)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    status = torch.zeros(4, dtype=torch.int32, device=dev)
    with _lib.on_device(dev):
        _lib.check(L.fgc_select_knn_f32(_lib.ptr(x), n, D, _lib.ptr(rs_dev), rs_arr, n_rs, K, float(max_radius), nbd,
                                        nb_arr, _lib.ptr(idx), _lib.ptr(dist), _lib.ptr(status), _lib.ptr(ws),
                                        ws_bytes, _lib.stream_ptr()))
    if config.sync_checks and (int(status[0].item()) & _lib.ST_NONFINITE):
        raise RuntimeError("select_knn: input coordinates contain non-finite values")
    return idx, dist


# ------------------------------------------------------------------ dense layer with the library's weight gradient
def linear_wgrad(grad_out: torch.Tensor, x: torch.Tensor, with_bias: bool = True):
    """(grad_weight [O, I], grad_bias [O] or None) of y = x W^T + b from grad_out [n, O] and x [n, I]."""
    _lib.require_device(grad_out, x)
    L = _lib.lib()
    g = grad_out.to(torch.float32).contiguous()
    xx = x.to(torch.float32).contiguous()
    n, O = g.shape
    I = xx.shape[1]
    gw = torch.empty((O, I), dtype=torch.float32, device=g.device)
    gb = torch.empty(O, dtype=torch.float32, device=g.device) if with_bias else None
    ws_bytes = L.fgc_linear_wgrad_workspace_bytes(n, O, I)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=g.device)
    with _lib.on_device(g.device):
        _lib.check(L.fgc_linear_wgrad_f32(_lib.ptr(g), _lib.ptr(xx), n, O, I, _lib.ptr(gw), _lib.ptr(gb), _lib.ptr(ws),
                                          ws_bytes, _lib.stream_ptr()))
    return gw, gb


class _Dense(torch.autograd.Function):
    """y = x W^T + b.  Forward and input gradient are library GEMMs (tiled over the points, which is what they are
    good at); the weight gradient, a reduction over the points with a tiny output, is the library's own kernel."""

    @staticmethod
    def forward(ctx, x, weight, bias):
        _lib.require_device(x, weight)
        ctx.save_for_backward(x, weight)
        ctx.has_bias = bias is not None
        return torch.nn.functional.linear(x, weight, bias)

    @staticmethod
    def backward(ctx, g):
        x, weight = ctx.saved_tensors
        gx = gw = gb = None
        if g is None:
            return None, None, None
        g = g.contiguous()
        if ctx.needs_input_grad[0]:
            gx = g.matmul(weight)
        if ctx.needs_input_grad[1] or (ctx.has_bias and ctx.needs_input_grad[2]):
            x2 = x.reshape(-1, x.shape[-1])
            g2 = g.reshape(-1, g.shape[-1])
            if x2.dtype == torch.float32 and g2.dtype == torch.float32:
                gw, gb = linear_wgrad(g2, x2, ctx.has_bias)
            else:
                gw = g2.t().matmul(x2)
                gb = g2.sum(0) if ctx.has_bias else None
        return gx, gw, gb


def _dense_impl(x, weight, bias):
    return _Dense.apply(x, weight, bias)


# ------------------------------------------------------------------ registration
def _register():
    lib = _define("bin_by_coordinates",
                  "bin_by_coordinates(Tensor coordinates, Tensor row_splits, Tensor? bin_width, Tensor? n_bins, "
                  "bool calc_n_per_bin, bool pre_normalized) -> (Tensor, Tensor, Tensor, Tensor, Tensor)")
    lib.impl("bin_by_coordinates", _bin_by_coordinates_impl, "CUDA")
    lib.impl("bin_by_coordinates", _bin_by_coordinates_impl, "CPU")      # raises: no CPU fallback

    lib = _define("index_replacer", "index_replacer(Tensor to_be_replaced, Tensor replacements) -> Tensor")
    lib.impl("index_replacer", _index_replacer_impl, "CUDA")
    lib.impl("index_replacer", _index_replacer_impl, "CPU")

    lib = _define("binned_select_knn_grad",
                  "binned_select_knn_grad(Tensor grad_distances, Tensor indices, Tensor distances, "
                  "Tensor coordinates) -> Tensor")
    lib.impl("binned_select_knn_grad", _knn_grad_impl, "CUDA")
    lib.impl("binned_select_knn_grad", _knn_grad_impl, "CPU")

    lib = _define("binned_select_knn",
                  "binned_select_knn(Tensor coordinates, Tensor bin_idx, Tensor dim_bin_idx, Tensor bin_boundaries, "
                  "Tensor n_bins, Tensor bin_width, Tensor direction, bool tf_compat, bool use_direction, int K) "
                  "-> (Tensor, Tensor)")
    lib.impl("binned_select_knn", _knn_sorted_space_impl, "CUDA")
    lib.impl("binned_select_knn", _knn_sorted_space_impl, "CPU")

    lib = _define("fastgraphcompute_custom_ops",
                  "binned_select_knn_autograd(Tensor coords, Tensor row_splits, int K, Tensor? direction, "
                  "Tensor? n_bins, int max_bin_dims, bool torch_compatible_indices) -> (Tensor, Tensor)")
    lib.impl("binned_select_knn_autograd", _knn_autograd_impl, "Autograd")
    lib.define("gravnet_aggregate(Tensor neighbor_idx, Tensor distsq, Tensor features) -> (Tensor, Tensor)")
    lib.impl("gravnet_aggregate", _gravnet_aggregate_impl, "Autograd")
    lib.define("dense(Tensor x, Tensor weight, Tensor? bias) -> Tensor")
    lib.impl("dense", _dense_impl, "Autograd")
    lib.define("dense_split(Tensor x, Tensor a, Tensor weight, Tensor? bias) -> Tensor")
    lib.impl("dense_split", _dense_split_impl, "Autograd")
    lib.define("gravnet_layer_core(Tensor space, Tensor features, Tensor row_splits, int K) -> "
               "(Tensor, Tensor, Tensor)")
    lib.impl("gravnet_layer_core", _gravnet_layer_core_impl, "Autograd")
    lib.define("select_with_default_f32(Tensor idx, Tensor feat, float default_value) -> Tensor")
    lib.impl("select_with_default_f32", _select_with_default_impl, "Autograd")
    lib.define("select_with_default_b64(Tensor idx, Tensor feat, float default_value) -> Tensor")
    lib.impl("select_with_default_b64", _select_with_default_impl, "Autograd")

    lib = _define("select_knn",
                  "select_knn(Tensor coords, Tensor row_splits, Tensor mask, int n_neighbours, float max_radius, "
                  "int mask_mode) -> (Tensor, Tensor)")
    lib.impl("select_knn", _select_knn_impl, "CUDA")
    lib.impl("select_knn", _select_knn_impl, "CPU")

    lib = _define("oc_helper_cuda",
                  "oc_helper_cuda(Tensor asso_idx, Tensor unique_idx, Tensor unique_rs_asso, Tensor rs, "
                  "Tensor max_n_unique_over_splits, Tensor max_n_in_splits, bool calc_m_not) -> (Tensor, Tensor)")
    lib.impl("oc_helper_cuda", _oc_helper_cuda_impl, "CUDA")
    lib.impl("oc_helper_cuda", _oc_helper_cuda_impl, "CPU")
    lib.define("oc_helper_matrices(Tensor truth_idxs, Tensor row_splits, bool calc_m_not) -> "
               "(Tensor, Tensor, Tensor)")
    lib.impl("oc_helper_matrices", _oc_helper_matrices_impl, "CUDA")
    lib.impl("oc_helper_matrices", _oc_helper_matrices_impl, "CPU")
    lib.define("max_same_valued_entries_per_row_split(Tensor asso_idx, Tensor row_splits, bool filter_negative) "
               "-> (Tensor, Tensor, Tensor)")
    lib.impl("max_same_valued_entries_per_row_split", _max_same_valued_impl, "CUDA")
    lib.impl("max_same_valued_entries_per_row_split", _max_same_valued_impl, "CPU")


_register()
