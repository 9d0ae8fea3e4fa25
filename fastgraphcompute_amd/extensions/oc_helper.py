"""select_with_default on MI355X (fastgraphcompute/extensions/oc_helper.py:232-271).

oc_helper_matrices belongs to the object-condensation loss, which is outside
the graph-building path this package implements."""
import torch

from .. import _ops  # noqa: F401  (registers the ops)


@torch.jit.script
def select_with_default(idx: torch.Tensor, feat: torch.Tensor, default_value: float) -> torch.Tensor:
    """out[v, k, :] = feat[idx[v, k], :], or default_value where idx[v, k] == -1.  Shape [V, K, F]."""
    if idx.dim() != 2 or feat.dim() != 2:
        raise ValueError("select_with_default expects idx [V, K] and feat [V', F]")
    if feat.dtype == torch.float32:
        return torch.ops.fastgraphcompute_custom_ops.select_with_default_f32(idx, feat, default_value)
    # other feature types: the same rule through one gather on a table padded with the default
    rows = feat.shape[0]
    pad = torch.full((1, feat.shape[1]), default_value, dtype=feat.dtype, device=feat.device)
    table = torch.cat([feat, pad], dim=0)
    ii = idx.long()
    return table[torch.where(ii == -1, torch.full_like(ii, rows), ii)]


def oc_helper_matrices(*args, **kwargs):
    raise NotImplementedError("oc_helper_matrices (object condensation) is outside the graph-building path of "
                              "fastgraphcompute_amd")
