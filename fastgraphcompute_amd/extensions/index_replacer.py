"""index_replacer on MI355X; mirrors fastgraphcompute/extensions/index_replacer.py:40-59."""
import torch

from .. import _ops  # noqa: F401  (registers the ops)


@torch.jit.script
def index_replacer(to_be_replaced: torch.Tensor, replacements: torch.Tensor) -> torch.Tensor:
    """out[i] = replacements[to_be_replaced[i]] for 0 <= value < len(replacements); other values pass through."""
    if to_be_replaced.device != replacements.device:
        raise AssertionError("Tensors must be on the same device.")
    if to_be_replaced.dtype != torch.int64 or replacements.dtype != torch.int64:
        raise AssertionError("Tensors must be int64 type.")
    return torch.ops.index_replacer.index_replacer(to_be_replaced, replacements)
