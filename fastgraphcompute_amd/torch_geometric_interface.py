"""row_splits <-> PyTorch Geometric `batch` vectors (fastgraphcompute/torch_geometric_interface.py:4-74).

Pure index arithmetic with torch ops, on whatever device the input lives."""
import torch


def row_splits_from_strict_batch(batch: torch.Tensor) -> torch.Tensor:
    """row_splits [num_graphs + 1] (int64) of a batch vector whose equal entries are contiguous:
    [0, 0, 0, 1, 1, 2, 2, 2] -> [0, 3, 5, 8].  An empty batch gives [0, 0]."""
    change = torch.nonzero(batch[1:] != batch[:-1], as_tuple=False).flatten()
    first = torch.zeros(1, dtype=torch.int64, device=batch.device)
    last = torch.full((1,), batch.numel(), dtype=torch.int64, device=batch.device)
    return torch.cat([first, change.to(torch.int64) + 1, last])


def strict_batch_from_row_splits(row_splits: torch.Tensor) -> torch.Tensor:
    """batch vector [V] (int64) of a row_splits tensor: [0, 3, 5, 8] -> [0, 0, 0, 1, 1, 2, 2, 2]."""
    row_splits = row_splits.to(torch.int64)
    lengths = row_splits[1:] - row_splits[:-1]
    return torch.repeat_interleave(torch.arange(lengths.numel(), dtype=torch.int64, device=row_splits.device),
                                   lengths)
