"""row_splits <-> batch conversion: the cases of the reference's tests/test_torch_geometric_interface.py."""
import pytest
import torch

from fastgraphcompute_amd.torch_geometric_interface import (row_splits_from_strict_batch,
                                                            strict_batch_from_row_splits)

CASES = [([0, 0, 0, 1, 1, 2, 2, 2], [0, 3, 5, 8]), ([0, 0, 0, 0], [0, 4]), ([], [0, 0]), ([0, 1, 2, 3], [0, 1, 2, 3, 4])]


@pytest.mark.parametrize("batch,rs", CASES)
def test_round_trip(batch, rs):
    b = torch.tensor(batch, dtype=torch.int64)
    r = torch.tensor(rs, dtype=torch.int64)
    got = row_splits_from_strict_batch(b)
    assert got.dtype == torch.int64 and torch.equal(got, r)
    back = strict_batch_from_row_splits(r)
    assert back.dtype == torch.int64 and torch.equal(back, b)


def test_int32_row_splits_and_unsorted_labels():
    assert torch.equal(strict_batch_from_row_splits(torch.tensor([0, 2, 2, 3], dtype=torch.int32)),
                       torch.tensor([0, 0, 2]))
    # labels only need to be contiguous, not 0..n-1
    assert torch.equal(row_splits_from_strict_batch(torch.tensor([7, 7, 3, 3, 3, 9])), torch.tensor([0, 2, 5, 6]))


@pytest.mark.gpu
def test_on_device_feeds_knn():
    from fastgraphcompute_amd import binned_select_knn
    b = torch.tensor([0] * 300 + [1] * 200, device="cuda")
    rs = row_splits_from_strict_batch(b)
    assert rs.is_cuda and rs.tolist() == [0, 300, 500]
    assert torch.equal(strict_batch_from_row_splits(rs), b)
    idx, _ = binned_select_knn(4, torch.rand(500, 3, device="cuda"), rs)
    assert bool((idx[:300] < 300).all()) and bool((idx[300:] >= 300).all())
