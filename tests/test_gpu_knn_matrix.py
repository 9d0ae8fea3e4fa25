"""The matrix-core search (5 to 8 coordinates, K <= 256, events of at most 65535 points) against the CPU checker and
against the vector-unit search: same neighbour sets, bit-identical distances."""
import numpy as np
import pytest
import torch

from tests.util import assert_knn_equal, check_knn_properties

pytestmark = pytest.mark.gpu


def _run(K, coords, rs, mode, sorted_rows=False, **kw):
    from fastgraphcompute_amd import binned_select_knn, config
    old = (config.matrix_search, config.sorted_neighbours)
    config.matrix_search, config.sorted_neighbours = mode, sorted_rows
    try:
        for k in ("direction",):
            if kw.get(k) is not None and not torch.is_tensor(kw[k]):
                kw[k] = torch.as_tensor(kw[k], device="cuda")
        idx, dist = binned_select_knn(K, torch.as_tensor(coords, device="cuda"), torch.as_tensor(rs, device="cuda"), **kw)
    finally:
        config.matrix_search, config.sorted_neighbours = old
    return idx.cpu().numpy(), dist.cpu().numpy()


def _both(oracle, K, coords, rs, check_oracle=True, **kw):
    """Forced matrix-core search against the vector-unit search (sorted rows: distances bit for bit) and the checker."""
    mi, md = _run(K, coords, rs, "always", True, **kw)
    vi, vd = _run(K, coords, rs, False, True, **kw)
    np.testing.assert_array_equal(md.view(np.uint32), vd.view(np.uint32), err_msg="distsq differs between the searches")
    assert_knn_equal(mi, md, vi, vd, what="matrix vs vector")
    ui, ud = _run(K, coords, rs, "always", False, **kw)      # rows in the order found
    assert_knn_equal(ui, ud, vi, vd, what="matrix (any order) vs vector")
    if check_oracle:
        okw = {k: (np.asarray(v.cpu()) if torch.is_tensor(v) else v) for k, v in kw.items()}
        oi, od = oracle.binned_select_knn(K, coords, rs, n_threads=8, **okw)
        assert_knn_equal(mi, md, oi, od, what="matrix vs checker")
    return mi, md


@pytest.mark.parametrize("D", [5, 6, 7, 8])
@pytest.mark.parametrize("K", [1, 10, 40])
def test_dimensions_and_small_k(oracle, D, K):
    rng = np.random.default_rng(100 * D + K)
    coords = rng.random((6000, D)).astype(np.float32)
    rs = [0, 2500, 2500, 3100, 6000]                       # an empty event too
    mi, md = _both(oracle, K, coords, rs)
    check_knn_properties(mi, md, coords, rs, K, ascending=True)


@pytest.mark.parametrize("K", [64, 65, 100, 128, 129, 200, 256])
def test_neighbour_counts(oracle, K):
    rng = np.random.default_rng(7 + K)
    coords = rng.standard_normal((5000, 8)).astype(np.float32)
    rs = [0, 1800, 5000]
    mi, md = _both(oracle, K, coords, rs)
    check_knn_properties(mi, md, coords, rs, K, ascending=True)


def test_events_smaller_than_k_and_than_a_column(oracle):
    # events of 1, 7, 40 and 90 points with K = 50: padding, and events collected whole without any screening
    rng = np.random.default_rng(3)
    sizes = [1, 7, 40, 90, 3000, 33, 64]
    rs = np.concatenate([[0], np.cumsum(sizes)])
    coords = rng.random((rs[-1], 6)).astype(np.float32)
    mi, md = _both(oracle, 50, coords, rs)
    check_knn_properties(mi, md, coords, rs, 50, ascending=True)
    mi, md = _both(oracle, 50, coords, rs, torch_compatible_indices=True)


def test_direction_flags(oracle):
    rng = np.random.default_rng(4)
    n = 4000
    coords = rng.random((n, 7)).astype(np.float32)
    direction = rng.integers(0, 3, n).astype(np.int64)
    _both(oracle, 12, coords, [0, 1500, n], direction=direction)


def test_clustered_points_far_from_the_origin(oracle):
    # tight clusters at coordinates around 1000: the screening must not lose neighbours to cancellation
    rng = np.random.default_rng(5)
    centres = 1000.0 + 50.0 * rng.random((40, 8))
    coords = (centres[rng.integers(0, 40, 8000)] + 0.01 * rng.standard_normal((8000, 8))).astype(np.float32)
    mi, md = _both(oracle, 24, coords, [0, 3000, 8000])
    check_knn_properties(mi, md, coords, [0, 3000, 8000], 24, ascending=True)


def test_duplicates_and_ties(oracle):
    # many identical points (more than K at distance 0) and points on a lattice (exact ties at the K-th distance):
    # queries the screening cannot resolve are handed to the vector-unit search
    rng = np.random.default_rng(6)
    lattice = rng.integers(0, 3, (3000, 5)).astype(np.float32)
    dup = np.repeat(rng.random((20, 5)).astype(np.float32), 100, axis=0)
    coords = np.concatenate([lattice, dup])
    rs = [0, 3000, 5000]
    mi, md = _run(8, coords, rs, "always", True)
    vi, vd = _run(8, coords, rs, False, True)
    np.testing.assert_array_equal(md.view(np.uint32), vd.view(np.uint32))
    check_knn_properties(mi, md, coords, rs, 8, ascending=True)
    bi, bd = oracle.knn_brute(8, coords, rs)
    np.testing.assert_allclose(np.sort(md, axis=1), np.sort(bd, axis=1), rtol=1e-6, atol=0)


def test_wide_range_of_scales(oracle):
    # one event with coordinates of order 1e-4, one of order 1e4, one mixing a dense core with far outliers
    rng = np.random.default_rng(8)
    a = (1e-4 * rng.random((2000, 6))).astype(np.float32)
    b = (1e4 * rng.standard_normal((2000, 6))).astype(np.float32)
    c = np.concatenate([0.001 * rng.standard_normal((1900, 6)), 100.0 * rng.standard_normal((100, 6))]).astype(np.float32)
    coords = np.concatenate([a, b, c])
    rs = [0, 2000, 4000, 6000]
    mi, md = _both(oracle, 16, coords, rs)
    check_knn_properties(mi, md, coords, rs, 16, ascending=True)


def test_large_event_takes_the_vector_search(oracle):
    # an event of more than 65535 points cannot use the 16-bit candidate positions: the library falls back by itself
    rng = np.random.default_rng(9)
    coords = rng.random((70000, 5)).astype(np.float32)
    mi, md = _run(8, coords, [0, 70000], "always", True)
    vi, vd = _run(8, coords, [0, 70000], False, True)
    np.testing.assert_array_equal(mi, vi)
    np.testing.assert_array_equal(md.view(np.uint32), vd.view(np.uint32))


def test_cfg5_scaled_forced(oracle):
    from fastgraphcompute_amd.workloads import CONFIGS
    w = CONFIGS["cfg5"](0.1)
    mi, md = _both(oracle, w["K"], w["coords"], w["row_splits"])
    check_knn_properties(mi, md, w["coords"], w["row_splits"], w["K"], ascending=True)


def test_gradient_through_the_matrix_search(oracle):
    from fastgraphcompute_amd import binned_select_knn, config
    rng = np.random.default_rng(10)
    n, K = 3000, 20
    coords = rng.random((n, 6)).astype(np.float32)
    rs = [0, 1200, n]
    old = config.matrix_search
    config.matrix_search = "always"
    try:
        x = torch.from_numpy(coords).cuda().requires_grad_(True)
        idx, dist = binned_select_knn(K, x, torch.tensor(rs, device="cuda"))
        up = rng.standard_normal((n, K)).astype(np.float32)
        dist.backward(torch.from_numpy(up).cuda())
    finally:
        config.matrix_search = old
    exp = oracle.knn_grad(up, idx.cpu().numpy(), coords)
    assert np.abs(x.grad.cpu().numpy() - exp).max() <= 1e-5 * np.abs(exp).max()


def test_the_matrix_search_is_the_one_that_runs():
    # counters of the statistics build: candidates collected by the matrix-core search, queries it handed over
    from fastgraphcompute_amd import binned_select_knn, config, _ops
    rng = np.random.default_rng(11)
    n, K = 8000, 32
    coords = torch.from_numpy(rng.random((n, 8)).astype(np.float32)).cuda()
    rs = torch.tensor([0, 5000, n], device="cuda")
    old = (config.matrix_search, config.collect_stats)
    try:
        config.collect_stats = True
        config.matrix_search = "always"
        binned_select_knn(K, coords, rs)
        forced = dict(_ops.last_stats)
        config.matrix_search = True          # 8 coordinates, events of 5000 and 3000 points: the library's own choice too
        binned_select_knn(K, coords, rs)
        auto = dict(_ops.last_stats)
        config.matrix_search = False
        binned_select_knn(K, coords, rs)
        vector = dict(_ops.last_stats)
    finally:
        config.matrix_search, config.collect_stats = old
    for st in (forced, auto):
        assert st["matrix_search_collected"] >= n * K and st["matrix_search_handed_over"] < n // 100, st
    assert vector["matrix_search_collected"] == 0 and vector["pool_prunes"] > 0, vector
