"""bin_by_coordinates on MI355X.  Mirrors the reference wrapper
fastgraphcompute/extensions/bin_by_coordinates.py:11-111 (same signature,
same five return values, same errors); the tensor preprocessing and the
per-point kernel run as HIP kernels behind `torch.ops.bin_by_coordinates`."""
from typing import Optional, Tuple

import torch

from .. import _ops  # noqa: F401  (registers the ops)


def bin_by_coordinates(coordinates: torch.Tensor, row_splits: torch.Tensor,
                       bin_width: Optional[torch.Tensor] = None, n_bins: Optional[torch.Tensor] = None,
                       calc_n_per_bin: bool = True, pre_normalized: bool = False,
                       name: str = "") -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """Assign every point to a bin of a regular grid, per event.

    Returns (bin_indices [N, D+1] int64 with column 0 the event, flat_bin_indices
    [N] int64, n_bins [D] int64, bin_width [1] float32, n_per_bin [B] int64).
    Scriptable; in eager mode `n_bins` / `bin_width` may also be plain numbers.
    """
    if not torch.jit.is_scripting():
        if bin_width is None and n_bins is None:
            raise ValueError("Either bin_width or n_bins must be provided.")
        if n_bins is not None and not torch.is_tensor(n_bins):
            n_bins = torch.tensor(n_bins, dtype=torch.int64, device=coordinates.device)
        if bin_width is not None and not torch.is_tensor(bin_width):
            bin_width = torch.tensor([bin_width], dtype=torch.float32, device=coordinates.device)
    return torch.ops.bin_by_coordinates.bin_by_coordinates(
        coordinates, row_splits.to(dtype=torch.int64), bin_width, n_bins, calc_n_per_bin, pre_normalized)
