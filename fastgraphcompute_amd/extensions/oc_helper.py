"""oc_helper_matrices and select_with_default on MI355X (fastgraphcompute/extensions/oc_helper.py).

The matrices come from two library calls around one host read (sort of the vertices by (row split, association
index), then a gather for M and a stream compaction per row for M_not) instead of the reference's torch.unique
passes and its thread-per-object scan of the row split."""
import torch

from .. import _ops  # noqa: F401  (registers the ops)


@torch.jit.script
def select_with_default(idx: torch.Tensor, feat: torch.Tensor, default_value: float) -> torch.Tensor:
    """out[v, k, :] = feat[idx[v, k], :], or default_value where idx[v, k] == -1.  Shape [V, K, F]."""
    if idx.dim() != 2 or feat.dim() != 2:
        raise ValueError("select_with_default expects idx [V, K] and feat [V', F]")
    if feat.dtype == torch.float32:
        return torch.ops.fastgraphcompute_custom_ops.select_with_default_f32(idx, feat, default_value)
    if feat.dtype == torch.int64 or feat.dtype == torch.float64:
        return torch.ops.fastgraphcompute_custom_ops.select_with_default_b64(idx, feat, default_value)
    # other feature types: the same rule through one gather on a table padded with the default
    rows = feat.shape[0]
    pad = torch.full((1, feat.shape[1]), default_value, dtype=feat.dtype, device=feat.device)
    table = torch.cat([feat, pad], dim=0)
    ii = idx.long()
    return table[torch.where(ii == -1, torch.full_like(ii, rows), ii)]


max_same_valued_entries_per_row_split = torch.ops.oc_helper_cuda.max_same_valued_entries_per_row_split


@torch.jit.script
def oc_helper_matrices(truth_idxs: torch.Tensor, row_splits: torch.Tensor, calc_m_not: bool = True):
    """(M, M_not, objects_per_split) as oc_helper.py:152-229 of the reference.

    M [n_objects, n_max_points_per_object]: row k lists the vertices whose truth index is object k's, inside the
    object's row split, ascending, padded with -1.  M_not [n_objects, n_max_points_per_row_split]: the other
    vertices of that row split (also those with negative truth index), ascending, padded with -1; an empty
    [0, 0] tensor when calc_m_not is False, like the reference's device op.  Negative truth indices form no
    object.  Rows are ordered by row split, then truth index.  objects_per_split [len(row_splits) - 1]."""
    torch._assert(truth_idxs.device == row_splits.device,
                  "Both truth_idxs and row_splits must be on the same device")
    M, M_not, obj_per_split = torch.ops.oc_helper_cuda.oc_helper_matrices(truth_idxs, row_splits, calc_m_not)
    return M, M_not, obj_per_split
