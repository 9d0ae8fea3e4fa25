"""binned_select_knn on MI355X.

Mirrors fastgraphcompute/extensions/binned_select_knn.py:12-94 (a scripted
wrapper with the same argument policy, dtypes and return tuple) around
`torch.ops.fastgraphcompute_custom_ops.binned_select_knn_autograd`, whose
forward is one call into libfgc_hip.so (binning, sort, search, un-sort fused)
and whose backward is the gradient kernel
(BinnedKNNAutograd, binned_knn_autograd_kernel.cpp:85-252).
"""
from typing import Optional, Tuple

import torch

from .. import _ops
from .._ops import calculate_optimal_bins, last_stats  # noqa: F401  (re-exported)


@torch.jit.script
def binned_select_knn(K: int,
                      coords: torch.Tensor,
                      row_splits: torch.Tensor,
                      direction: Optional[torch.Tensor] = None,
                      n_bins: Optional[torch.Tensor] = None,
                      max_bin_dims: int = 3,
                      torch_compatible_indices: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    """Exact K nearest neighbours of every point inside its own event.

    Returns (idx int64 [N, K], distsq float32 [N, K]); column 0 is the point
    itself with distance 0, the other columns its K-1 nearest neighbours, then
    -1 / 0 where the event has fewer than K points.  Like the reference, the
    neighbours of a row come in no particular order; set
    config.sorted_neighbours for rows by increasing distance.
    `direction`: 0 = may only be a neighbour, 1 = may only have neighbours, 2 = neither.
    """
    if coords.dim() != 2 or coords.shape[1] == 0:
        raise ValueError("Input coordinates must have at least one dimension. Got 0 dimensions.")
    if max_bin_dims == 0:
        raise ValueError("max_bin_dims must be greater than 0. Got 0.")
    # only 2..5 binned dimensions exist, never more than the coordinates have
    coord_dims = coords.shape[1]
    max_bin_dims = min(max_bin_dims, coord_dims, 5)
    max_bin_dims = max(max_bin_dims, 2)
    if coords.dtype != torch.float32:
        coords = coords.to(dtype=torch.float32)
    coords = coords.contiguous()
    row_splits = row_splits.contiguous()
    if direction is not None:
        direction = direction.contiguous()
    if n_bins is not None:
        n_bins = n_bins.to(dtype=torch.int64).contiguous()
    idx, dist = torch.ops.fastgraphcompute_custom_ops.binned_select_knn_autograd(
        coords, row_splits, K, direction, n_bins, max_bin_dims, torch_compatible_indices)
    return idx, dist


def binned_select_knn_grad(grad_distsq: torch.Tensor, idx: torch.Tensor, coords: torch.Tensor,
                           order: Optional[torch.Tensor] = None) -> torch.Tensor:
    """d loss / d coords from d loss / d distsq
    (binned_select_knn_grad_cuda_fn, binned_select_knn_grad_cuda_kernel.cu:90-164).
    `order` (int32 [N], optional) is a spatially coherent processing order of the
    points, e.g. the forward's bin-sorted order; it speeds the kernel up and does
    not change the result beyond float summation order."""
    return _ops.knn_grad(grad_distsq, idx, coords, order)
