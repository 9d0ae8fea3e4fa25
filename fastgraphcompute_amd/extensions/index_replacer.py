"""index_replacer on MI355X; mirrors fastgraphcompute/extensions/index_replacer.py:40-59."""
import torch

from .. import _lib


def index_replacer(to_be_replaced: torch.Tensor, replacements: torch.Tensor) -> torch.Tensor:
    """out[i] = replacements[to_be_replaced[i]] for 0 <= value < len(replacements); other values pass through."""
    if to_be_replaced.device != replacements.device:
        raise AssertionError("Tensors must be on the same device.")
    if to_be_replaced.dtype != torch.int64 or replacements.dtype != torch.int64:
        raise AssertionError("Tensors must be int64 type.")
    _lib.require_device(to_be_replaced)
    L = _lib.lib()
    src = to_be_replaced.contiguous()
    rep = replacements.contiguous()
    out = torch.empty_like(src)
    with torch.cuda.device(src.device):
        _lib.check(L.fgc_index_replacer_i64(_lib.ptr(src), _lib.ptr(rep), _lib.ptr(out), src.numel(), rep.numel(),
                                            _lib.stream_ptr()))
    return out
