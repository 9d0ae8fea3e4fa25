"""GravNetOp on MI355X.  Same constructor, sub-module names and forward return
tuple as fastgraphcompute/gnn_ops.py:9-109, so state_dicts interchange; the
neighbour aggregation (gnn_ops.py:90-102) is one fused HIP kernel per
direction instead of six tensor ops over a [N, K, P] intermediate."""
from typing import Tuple

import torch

from . import _lib
from .extensions import binned_select_knn


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
        with torch.cuda.device(f.device):
            _lib.check(L.fgc_gravnet_aggregate_fwd_f32(_lib.ptr(ii), _lib.ptr(d), _lib.ptr(f), _lib.ptr(fmean),
                                                       _lib.ptr(fmax), _lib.ptr(argmax), n, K, P, _lib.stream_ptr()))
        ctx.save_for_backward(ii, d, f, argmax)
        ctx.set_materialize_grads(False)
        return fmean, fmax

    @staticmethod
    def backward(ctx, g_mean, g_max):
        ii, d, f, argmax = ctx.saved_tensors
        L = _lib.lib()
        n, K = ii.shape
        P = f.shape[1]
        if g_mean is None and g_max is None:
            return None, None, None
        g_mean = torch.zeros((n, P), dtype=torch.float32, device=f.device) if g_mean is None \
            else g_mean.to(torch.float32).contiguous()
        g_max = torch.zeros((n, P), dtype=torch.float32, device=f.device) if g_max is None \
            else g_max.to(torch.float32).contiguous()
        g_feat = torch.zeros_like(f)
        g_dist = torch.empty_like(d)
        with torch.cuda.device(f.device):
            _lib.check(L.fgc_gravnet_aggregate_bwd_f32(_lib.ptr(ii), _lib.ptr(d), _lib.ptr(f), _lib.ptr(argmax),
                                                       _lib.ptr(g_mean), _lib.ptr(g_max), _lib.ptr(g_feat),
                                                       _lib.ptr(g_dist), n, K, P, _lib.stream_ptr()))
        return None, g_dist, g_feat


def gravnet_aggregate(neighbor_idx: torch.Tensor, distsq: torch.Tensor, features: torch.Tensor):
    """Distance-weighted mean and max of the neighbours' features: ([N, P], [N, P])."""
    return _GravNetAggregate.apply(neighbor_idx, distsq, features)


class GravNetOp(torch.nn.Module):
    """One GravNet layer [arxiv:1902.07987]: learned coordinates -> kNN graph ->
    exp(-10 d^2)-weighted mean/max aggregation of learned features -> dense output."""

    def __init__(self, in_channels, out_channels, space_dimensions, propagate_dimensions, k,
                 output_activation=torch.nn.ReLU(), optimization_arguments: dict = {}):
        super(GravNetOp, self).__init__()
        self.k = k
        self.space_transformations = torch.nn.Linear(in_channels, space_dimensions)
        self.propagate_transformations = torch.nn.Linear(in_channels, propagate_dimensions)
        self.output_transformations = torch.nn.Sequential(
            torch.nn.Linear(in_channels + 2 * propagate_dimensions, out_channels),
            output_activation
        )
        self.optimization_arguments = optimization_arguments

    def forward(self, x: torch.Tensor, row_splits: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
        space = self.space_transformations(x)
        propagate = self.propagate_transformations(x)
        neighbor_idx, distsq = binned_select_knn(self.k, space.contiguous(), row_splits)
        fmean, fmax = gravnet_aggregate(neighbor_idx, distsq, propagate)
        output = torch.cat([x, fmean, fmax], dim=1)
        out = self.output_transformations(output)
        return out, neighbor_idx, distsq, space
