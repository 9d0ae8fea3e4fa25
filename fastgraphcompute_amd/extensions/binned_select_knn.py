"""binned_select_knn on MI355X.

Mirrors fastgraphcompute/extensions/binned_select_knn.py:12-94 (argument
policy, dtypes, return tuple) and the autograd op behind it,
BinnedKNNAutograd (binned_knn_autograd_kernel.cpp:85-252): the forward is one
call into libfgc_hip.so (binning, sort, search, un-sort fused), the backward
is the gradient kernel.
"""
from typing import Optional, Tuple

import torch

from .. import _lib, config

last_stats = {}


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


class _BinnedKNN(torch.autograd.Function):
    @staticmethod
    def forward(ctx, coords, row_splits, K, direction, n_bins, max_bin_dims, tf_compat):
        L = _lib.lib()
        dev = coords.device
        n, D = coords.shape
        nbd = min(int(max_bin_dims), D)
        if nbd < 2 or nbd > 5:
            raise ValueError("Unsupported number of binning dimensions.")
        if K < 1 or K > 256:
            raise ValueError("binned_select_knn on MI355X supports 1 <= K <= 256, got %d" % K)
        rs_host = row_splits.detach().to("cpu", torch.int64).contiguous()
        n_rs = rs_host.numel()
        if n_rs < 2:
            raise ValueError("row_splits needs at least two entries")
        if n_bins is None:
            nb = [calculate_optimal_bins(rs_host, K, nbd)] * nbd
        else:
            nbt = n_bins.detach().to("cpu", torch.int64)
            nb = [int(nbt.item())] * nbd if nbt.dim() == 0 or nbt.numel() == 1 else [int(v) for v in nbt.tolist()]
            if len(nb) != nbd:
                raise ValueError("bin_by_coordinates: coordinates.size(1) must be equal to nbins.size(0)")
            if not all(v > 0 for v in nb):
                raise RuntimeError("BinByCoordinates: n_bins must be greater than zero.")
        rs_list = rs_host.tolist()
        if n > 0 and (rs_list[0] != 0 or max(rs_list) != n or rs_list[-1] != n
                      or any(b < a for a, b in zip(rs_list, rs_list[1:]))):
            raise RuntimeError("Bin boundaries do not match row splits.")
        rs_dev = row_splits if (row_splits.is_cuda and row_splits.dtype == torch.int64) else rs_host.to(dev)
        rs_dev = rs_dev.contiguous()
        idx = torch.empty((n, K), dtype=torch.int64, device=dev)
        dist = torch.empty((n, K), dtype=torch.float32, device=dev)
        order = None
        if n > 0:
            nb_arr = _lib.host_i64(nb)
            rs_arr = _lib.host_i64(rs_list)
            ws_bytes = L.fgc_binned_select_knn_workspace_bytes(n, D, nbd, nb_arr, n_rs, K)
            ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
            status = torch.zeros(4, dtype=torch.int32, device=dev)
            stats = torch.zeros(4, dtype=torch.int64, device=dev) if config.collect_stats else None
            dirt = None
            if direction is not None and direction.numel() > 0:
                dirt = direction.to(device=dev, dtype=torch.int64).contiguous()
            with torch.cuda.device(dev):
                _lib.check(L.fgc_binned_select_knn_f32(
                    _lib.ptr(coords), n, D, _lib.ptr(rs_dev), rs_arr, n_rs, K, nbd, nb_arr, _lib.ptr(dirt),
                    1 if tf_compat else 0, _lib.ptr(idx), _lib.ptr(dist), _lib.ptr(status), _lib.ptr(stats),
                    _lib.ptr(ws), ws_bytes, _lib.stream_ptr()))
            if coords.requires_grad:
                order = torch.empty(n, dtype=torch.int32, device=dev)
                with torch.cuda.device(dev):
                    _lib.check(L.fgc_binned_knn_export_order_i32(n, D, rs_arr, n_rs, K, nbd, nb_arr,
                                                                 1 if dirt is not None else 0, _lib.ptr(ws), ws_bytes,
                                                                 _lib.ptr(order), _lib.stream_ptr()))
            if config.sync_checks:
                flags = int(status[0].item())
                if flags & _lib.ST_NONFINITE:
                    raise RuntimeError("BinByCoordinates: input coordinates contain non-finite values")
                if flags & _lib.ST_BAD_RANGE:
                    raise RuntimeError("BinByCoordinates: dmax_coords must be greater than zero.")
            if stats is not None:
                s = stats.tolist()
                last_stats.update(distance_evaluations=s[0], candidate_chunks=s[1], insertions=s[2],
                                  n_bins=nb, n_vert=n, K=K, n_coords=D)
        if order is None:
            order = torch.empty(0, dtype=torch.int32, device=dev)
        ctx.save_for_backward(idx, coords, order)
        ctx.mark_non_differentiable(idx)
        ctx.set_materialize_grads(False)   # no zero tensors for unused output gradients
        return idx, dist

    @staticmethod
    def backward(ctx, _grad_idx, grad_dist):
        idx, coords, order = ctx.saved_tensors
        if not ctx.needs_input_grad[0]:
            return None, None, None, None, None, None, None
        if grad_dist is None:
            return torch.zeros_like(coords), None, None, None, None, None, None
        g = binned_select_knn_grad(grad_dist, idx, coords, order if order.numel() else None)
        return g, None, None, None, None, None, None


def binned_select_knn_grad(grad_distsq: torch.Tensor, idx: torch.Tensor, coords: torch.Tensor,
                           order: Optional[torch.Tensor] = None) -> torch.Tensor:
    """d loss / d coords from d loss / d distsq
    (binned_select_knn_grad_cuda_fn, binned_select_knn_grad_cuda_kernel.cu:90-164).
    `order` (int32 [N], optional) is a spatially coherent processing order of the
    points, e.g. the forward's bin-sorted order; it speeds the kernel up and does
    not change the result beyond float summation order."""
    _lib.require_device(grad_distsq, idx, coords)
    L = _lib.lib()
    g = grad_distsq.to(torch.float32).contiguous()
    ii = idx.to(torch.int64).contiguous()
    x = coords.to(torch.float32).contiguous()
    n, D = x.shape
    K = ii.shape[1]
    out = torch.empty((n, D), dtype=torch.float32, device=x.device)
    status = torch.zeros(4, dtype=torch.int32, device=x.device)
    with torch.cuda.device(x.device):
        if order is not None:
            order = order.to(device=x.device, dtype=torch.int32).contiguous()
            if order.numel() != n:
                raise ValueError("order must hold one entry per point")
        _lib.check(L.fgc_binned_select_knn_grad_f32(_lib.ptr(g), _lib.ptr(ii), _lib.ptr(x), _lib.ptr(out), n, K, D,
                                                    _lib.ptr(order), _lib.ptr(status), _lib.stream_ptr()))
    return out


def binned_select_knn(K: int, coords: torch.Tensor, row_splits: torch.Tensor,
                      direction: Optional[torch.Tensor] = None, n_bins: Optional[torch.Tensor] = None,
                      max_bin_dims: int = 3, torch_compatible_indices: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    """Exact K nearest neighbours of every point inside its own event.

    Returns (idx int64 [N, K], distsq float32 [N, K]); column 0 is the point
    itself with distance 0, the other columns its K-1 nearest neighbours (by
    increasing distance), -1 / 0 where the event has fewer than K points.
    """
    if coords.dim() != 2 or coords.shape[1] == 0:
        raise ValueError("Input coordinates must have at least one dimension. Got 0 dimensions.")
    if max_bin_dims == 0:
        raise ValueError("max_bin_dims must be greater than 0. Got 0.")
    K = int(K)
    max_bin_dims = int(max_bin_dims)
    max_bin_dims = max(min(max_bin_dims, coords.shape[1], 5), 2)
    _lib.require_device(coords)
    if not isinstance(row_splits, torch.Tensor):
        row_splits = torch.tensor(row_splits, dtype=torch.int64, device=coords.device)
    if coords.dtype != torch.float32:
        coords = coords.to(dtype=torch.float32)
    if n_bins is not None and not isinstance(n_bins, torch.Tensor):
        n_bins = torch.tensor(n_bins, dtype=torch.int64)
    coords = coords.contiguous()
    idx, dist = _BinnedKNN.apply(coords, row_splits, K, direction, n_bins, max_bin_dims,
                                 bool(torch_compatible_indices))
    return idx, dist
