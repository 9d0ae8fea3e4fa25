"""select_knn on MI355X: the k nearest neighbours of every point inside its event and inside a radius.

The reference builds this op (extensions/select_knn.cpp:60-70, brute force per event, one CUDA launch per
event) but loads it from no Python file; callers reach it as torch.ops.select_knn.select_knn.  Here it is the
binned search of binned_select_knn started with the radius as its distance bound."""
from typing import Optional

import torch

from .. import _ops  # noqa: F401  (registers the ops)


@torch.jit.script
def select_knn(K: int, coords: torch.Tensor, row_splits: torch.Tensor, max_radius: float = -1.0,
               mask: Optional[torch.Tensor] = None, mask_mode: int = 0):
    """(idx int64 [N, K], distsq float32 [N, K]): slot 0 the point itself, then its up to K-1 nearest points
    of the same event with distance <= max_radius (no limit if max_radius <= 0) by increasing distance; -1 / 0
    where there are fewer.  mask and mask_mode are ignored, as in the reference."""
    m = mask if mask is not None else torch.zeros(0, dtype=torch.int64, device=coords.device)
    return torch.ops.select_knn.select_knn(coords, row_splits, m, K, max_radius, mask_mode)
