"""select_with_default on MI355X (fastgraphcompute/extensions/oc_helper.py:232-271).

oc_helper_matrices belongs to the object-condensation loss, which is outside
the graph-building path this package implements."""
import torch

from .. import _lib


def select_with_default(idx: torch.Tensor, feat: torch.Tensor, default_value: float) -> torch.Tensor:
    """out[v, k, :] = feat[idx[v, k], :], or default_value where idx[v, k] == -1.  Shape [V, K, F]."""
    _lib.require_device(idx, feat)
    if idx.dim() != 2 or feat.dim() != 2:
        raise ValueError("select_with_default expects idx [V, K] and feat [V', F]")
    V, K = idx.shape
    rows, F = feat.shape
    if feat.dtype != torch.float32:
        # integer / other feature types: same rule through one gather on a padded table
        pad = torch.full((1, F), default_value, dtype=feat.dtype, device=feat.device)
        table = torch.cat([feat, pad], dim=0)
        ii = idx.long()
        return table[torch.where(ii == -1, torch.full_like(ii, rows), ii)]
    L = _lib.lib()
    ii = idx.to(torch.int64).contiguous()
    ff = feat.contiguous()
    out = torch.empty((V, K, F), dtype=torch.float32, device=feat.device)
    with torch.cuda.device(feat.device):
        _lib.check(L.fgc_select_with_default_f32(_lib.ptr(ii), _lib.ptr(ff), _lib.ptr(out), V, K, F, rows,
                                                 float(default_value), _lib.stream_ptr()))
    return out


def oc_helper_matrices(*args, **kwargs):
    raise NotImplementedError("oc_helper_matrices (object condensation) is outside the graph-building path of "
                              "fastgraphcompute_amd")
