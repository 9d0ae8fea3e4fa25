"""bin_by_coordinates on the GPU against the CPU checker: bit-exact bin indices."""
import os

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def _run(coords, rs, bin_width=None, n_bins=None, **kw):
    from fastgraphcompute_amd import bin_by_coordinates
    dev = "cuda"
    bw = None if bin_width is None else torch.as_tensor(bin_width, dtype=torch.float32, device=dev)
    nb = n_bins
    if n_bins is not None and not isinstance(n_bins, int):
        nb = torch.as_tensor(n_bins, dtype=torch.int64, device=dev)
    out = bin_by_coordinates(torch.as_tensor(coords, device=dev), torch.as_tensor(rs, device=dev), bw, nb, **kw)
    return [o.cpu().numpy() for o in out]


def _compare(oracle, coords, rs, bin_width=None, n_bins=None, **kw):
    got = _run(coords, rs, bin_width, n_bins, **kw)
    exp = oracle.bin_by_coordinates(coords, rs, bin_width, n_bins, **kw)
    names = ["assigned", "flat", "n_bins", "bin_width", "n_per_bin"]
    for g, e, nm in zip(got, exp, names):
        assert g.dtype == e.dtype, nm
        np.testing.assert_array_equal(g, e, err_msg=nm)
    return got


def test_known_answers_simple(oracle):
    # tests/test_bin_by_coordinates.py:26-82 of the reference
    coords = np.array([[0.1, 0.1], [2.5, 2.5], [4.9, 4.9]], dtype=np.float32)
    a, f, nb, bw, nper = _compare(oracle, coords, [0, 3], np.array([0.5], np.float32), np.array([10, 10]))
    np.testing.assert_array_equal(a, [[0, 0, 0], [0, 4, 4], [0, 9, 9]])
    np.testing.assert_array_equal(f, [0, 44, 99])
    assert nper.shape == (100,) and nper.sum() == 3 and nper[0] == nper[44] == nper[99] == 1


def test_known_answers_clamped(oracle):
    # tests/test_bin_by_coordinates.py:111-162 of the reference
    coords = np.array([[-1.0, -1.0], [5.1, 5.1], [0.7, 0.7]], dtype=np.float32)
    a, f, nb, bw, nper = _compare(oracle, coords, [0, 3], np.array([0.5], np.float32), np.array([10, 10]))
    np.testing.assert_array_equal(a, [[0, 0, 0], [0, 9, 9], [0, 3, 3]])
    np.testing.assert_array_equal(f, [0, 99, 33])


@pytest.mark.parametrize("ndims", [1, 2, 3, 4, 5])
def test_random_with_width(oracle, ndims):
    rng = np.random.default_rng(7 + ndims)
    coords = rng.random((1000, ndims)).astype(np.float32)
    rs = np.array([0, 300, 700, 1000])
    a, f, nb, bw, nper = _compare(oracle, coords, rs, np.array([0.5], np.float32), np.array([10] * ndims))
    ev = np.repeat(np.arange(3), np.diff(rs))
    np.testing.assert_array_equal(a[:, 0], ev)
    assert nper.sum() == 1000


@pytest.mark.parametrize("n,ndims,nb", [(5000, 3, 18), (20000, 2, 30), (4096, 4, 7), (777, 5, 5)])
def test_random_with_n_bins(oracle, n, ndims, nb):
    rng = np.random.default_rng(100 + n)
    coords = (rng.standard_normal((n, ndims)) * 3.0 + 10.0).astype(np.float32)
    rs = np.array([0, n // 3, n // 2, n])
    _compare(oracle, coords, rs, None, nb)
    _compare(oracle, coords, rs, None, np.array([nb] * ndims))


def test_width_without_n_bins(oracle):
    rng = np.random.default_rng(5)
    coords = rng.random((3000, 3)).astype(np.float32) * np.array([1.0, 2.0, 0.5], np.float32)
    _compare(oracle, coords, [0, 3000], np.array([0.07], np.float32), None)


def test_pre_normalized_and_zero_range(oracle):
    rng = np.random.default_rng(6)
    coords = rng.random((2000, 3)).astype(np.float32)
    coords[:, 1] = 0.25  # zero range in one dimension
    _compare(oracle, coords, [0, 500, 2000], None, 9)
    _compare(oracle, coords, [0, 500, 2000], None, 9, pre_normalized=True)


def test_reference_data_file(oracle):
    # the reference's own smoke input (tests/test_bin_by_coordinates.py:232-251), large dynamic range
    coords = np.load(os.path.join(GOLDEN, "bbc_coords.npy"), allow_pickle=False).astype(np.float32)
    _compare(oracle, coords, [0, coords.shape[0]], None, 21)


def test_non_finite_raises():
    from fastgraphcompute_amd import bin_by_coordinates
    c = torch.rand(100, 3, device="cuda")
    c[5, 1] = float("nan")
    with pytest.raises(ValueError):
        bin_by_coordinates(c, torch.tensor([0, 100], device="cuda"), n_bins=5)
    with pytest.raises(ValueError):
        bin_by_coordinates(torch.rand(10, 3, device="cuda"), torch.tensor([0, 10], device="cuda"))


def test_cpu_tensor_rejected():
    from fastgraphcompute_amd import bin_by_coordinates
    with pytest.raises(RuntimeError):
        bin_by_coordinates(torch.rand(10, 3), torch.tensor([0, 10]), n_bins=5)
