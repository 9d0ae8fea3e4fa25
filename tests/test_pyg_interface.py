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


@pytest.mark.gpu
def test_benchmark_csv_rows(tmp_path):
    """The timing sweep writes the columns the reference's published table is keyed on (size, k, dimension, fgc_time,
    count; graphing/master_data.csv, written by performance/generate_faiss_performance.py:95-135 and the scripts
    next to it) and times the K it writes - also beyond 256 neighbours."""
    import csv
    from fastgraphcompute_amd import benchmark_csv
    out = tmp_path / "t.csv"
    benchmark_csv.main(["--out", str(out), "--sizes", "3000", "--dims", "3", "6", "--k", "300", "--repeat", "2"])
    rows = list(csv.reader(open(out)))
    assert rows[0] == ["size", "k", "dimension", "fgc_time", "count"]
    assert len(rows) == 3
    for r, d in zip(rows[1:], (3.0, 6.0)):
        assert float(r[0]) == 3000.0 and float(r[1]) == 300.0 and float(r[2]) == d and float(r[4]) == 2.0
        assert 0.0 < float(r[3]) < 1e4
    with pytest.raises(SystemExit):
        benchmark_csv.main(["--out", str(out), "--sizes", "3000", "--dims", "3", "--k", "2000", "--repeat", "1"])
