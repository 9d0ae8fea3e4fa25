"""binned_select_knn on the GPU against the CPU checker and brute force."""
import numpy as np
import pytest
import torch

from tests.util import assert_knn_equal, check_knn_properties

pytestmark = pytest.mark.gpu


def _gpu_knn(K, coords, rs, **kw):
    from fastgraphcompute_amd import binned_select_knn
    for k in ("direction", "n_bins"):
        if kw.get(k) is not None and not torch.is_tensor(kw[k]):
            kw[k] = torch.as_tensor(kw[k], device="cuda")
    if "n_bins" in kw and kw["n_bins"] is not None:
        kw["n_bins"] = kw["n_bins"].to(torch.int64)
    idx, dist = binned_select_knn(K, torch.as_tensor(coords, device="cuda"),
                                  torch.as_tensor(rs, device="cuda"), **kw)
    assert idx.dtype == torch.int64 and dist.dtype == torch.float32
    return idx.cpu().numpy(), dist.cpu().numpy()


def _padding_last(idx):
    """Empty slots (-1) only after the last neighbour of a row."""
    empty = idx < 0
    assert not np.any(empty[:, :-1] & ~empty[:, 1:]), "a neighbour after an empty slot"


def _check(oracle, K, coords, rs, threads=8, **kw):
    """GPU result against the checker - with the library's own search grid and, when the caller gives no n_bins,
    also with the reference's grid (its n_bins heuristic and max_bin_dims)."""
    from fastgraphcompute_amd import config
    gi, gd = _gpu_knn(K, coords, rs, **dict(kw))
    okw = {k: (v.cpu().numpy() if torch.is_tensor(v) else v) for k, v in kw.items()}
    oi, od = oracle.binned_select_knn(K, coords, rs, n_threads=threads, **okw)
    assert_knn_equal(gi, gd, oi, od, what="own grid")
    _padding_last(gi)
    # the same call with rows by increasing distance (config.sorted_neighbours; the default leaves slots 1.. in the
    # order the search found them, like the reference)
    config.sorted_neighbours = True
    try:
        si, sd = _gpu_knn(K, coords, rs, **dict(kw))
    finally:
        config.sorted_neighbours = False
    assert_knn_equal(si, sd, oi, od, what="rows by distance")
    _padding_last(si)
    if not kw.get("torch_compatible_indices"):
        filled = np.where(si[:, 1:] >= 0, sd[:, 1:], np.inf)
        with np.errstate(invalid="ignore"):
            step = np.diff(filled, axis=1)                      # inf - inf between two empty slots
        assert np.all((step >= 0) | np.isnan(step)), "rows not ascending with config.sorted_neighbours"
    if kw.get("n_bins") is None:
        config.auto_grid = False
        try:
            ri, rd = _gpu_knn(K, coords, rs, **dict(kw))
        finally:
            config.auto_grid = True
        assert_knn_equal(ri, rd, oi, od, what="reference grid")
    return gi, gd


def test_cfg1_full(oracle):
    from fastgraphcompute_amd.workloads import cfg1_uniform_small
    w = cfg1_uniform_small()
    gi, gd = _check(oracle, w["K"], w["coords"], w["row_splits"])
    check_knn_properties(gi, gd, w["coords"], w["row_splits"], w["K"])
    bi, bd = oracle.knn_brute(w["K"], w["coords"], w["row_splits"])
    assert_knn_equal(gi, gd, bi, bd, "vs brute force")


@pytest.mark.parametrize("name,scale", [("cfg2", 0.1), ("cfg4", 0.03), ("cfg5", 0.04)])
def test_benchmark_shapes_scaled(oracle, name, scale):
    from fastgraphcompute_amd.workloads import CONFIGS
    w = CONFIGS[name](scale)
    gi, gd = _check(oracle, w["K"], w["coords"], w["row_splits"])
    check_knn_properties(gi, gd, w["coords"], w["row_splits"], w["K"])


@pytest.mark.parametrize("D", [2, 3, 4, 5, 6, 7, 8, 9, 12, 13, 16, 17])
def test_dimensions(oracle, D):
    rng = np.random.default_rng(40 + D)
    coords = rng.random((3000, D)).astype(np.float32)
    _check(oracle, 10, coords, [0, 1000, 1500, 3000])


@pytest.mark.parametrize("K", [1, 2, 5, 50, 64, 65, 100, 128, 129, 200, 256])
def test_neighbour_counts(oracle, K):
    rng = np.random.default_rng(60 + K)
    coords = rng.random((2500, 3)).astype(np.float32)
    _check(oracle, K, coords, [0, 1200, 2500])


@pytest.mark.parametrize("K,D", [(257, 3), (400, 2), (512, 4), (513, 3), (700, 6), (1024, 3)])
def test_more_than_256_neighbours(oracle, K, D):
    # beyond 256 neighbours the search runs its slower any-K variant; one event smaller than K (padding) and the
    # gradient through the op's backward
    rng = np.random.default_rng(K + D)
    n = 2600
    coords = rng.random((n, D)).astype(np.float32)
    rs = [0, 1500, 1500 + 300, n]
    gi, gd = _check(oracle, K, coords, rs)
    check_knn_properties(gi, gd, coords, rs, K)
    from fastgraphcompute_amd import binned_select_knn
    x = torch.from_numpy(coords).cuda().requires_grad_(True)
    idx, dist = binned_select_knn(K, x, torch.tensor(rs, device="cuda"))
    up = rng.standard_normal((n, K)).astype(np.float32)
    dist.backward(torch.from_numpy(up).cuda())
    exp = oracle.knn_grad(up, idx.cpu().numpy(), coords)
    assert np.abs(x.grad.cpu().numpy() - exp).max() <= 1e-5 * np.abs(exp).max()


def test_neighbour_count_limit():
    from fastgraphcompute_amd import binned_select_knn
    with pytest.raises((ValueError, RuntimeError)):
        binned_select_knn(1025, torch.rand(3000, 3, device="cuda"), torch.tensor([0, 3000], device="cuda"))


@pytest.mark.parametrize("mbd", [2, 3, 4, 5])
def test_max_bin_dims(oracle, mbd):
    rng = np.random.default_rng(80 + mbd)
    coords = rng.random((4000, 6)).astype(np.float32)
    _check(oracle, 12, coords, [0, 4000], max_bin_dims=mbd)


def test_reference_style_large(oracle):
    # shape of the reference's own test (tests/test_binned_select_knn.py:95-163): N=10 000, K=50, three events
    g = torch.Generator().manual_seed(45)
    for D in (3, 8):
        coords = torch.rand((10000, D), generator=g).numpy()
        rs = [0, 3333, 5000, 10000]
        gi, gd = _check(oracle, 50, coords, rs)
        # and against cdist + topk exactly as the reference's baseline does
        c = torch.from_numpy(coords)
        for a, b in zip(rs[:-1], rs[1:]):
            dm = torch.cdist(c[a:b], c[a:b], compute_mode="donot_use_mm_for_euclid_dist")
            d, _ = torch.topk(dm, 50, largest=False)
            ref = np.sort((d ** 2).numpy(), axis=1)
            np.testing.assert_allclose(np.sort(gd[a:b], axis=1), ref, atol=1e-6, rtol=1e-4)


def test_user_n_bins(oracle):
    rng = np.random.default_rng(11)
    coords = (rng.random((1000, 2)) - 0.5).astype(np.float32)
    _check(oracle, 5, coords, [0, 1000], n_bins=torch.tensor(10, dtype=torch.int64, device="cuda"))
    coords = (rng.random((1000, 4)) - 0.5).astype(np.float32)
    _check(oracle, 10, coords, [0, 1000], n_bins=torch.tensor(10, dtype=torch.int64, device="cuda"))
    _check(oracle, 8, rng.standard_normal((100, 3)).astype(np.float32), [0, 50, 100],
           n_bins=torch.tensor(4, dtype=torch.int64, device="cuda"))


def test_small_and_empty_events(oracle):
    rng = np.random.default_rng(12)
    coords = rng.random((300, 3)).astype(np.float32)
    rs = [0, 3, 3, 40, 41, 300]   # events of 3, 0, 37, 1, 259 points with K = 20
    gi, gd = _check(oracle, 20, coords, rs)
    check_knn_properties(gi, gd, coords, rs, 20)
    assert (gi[:3, 3:] == -1).all() and (gd[:3, 3:] == 0).all()
    ti, td = _check(oracle, 20, coords, rs, torch_compatible_indices=True)
    assert (ti[:3, 3:] == np.arange(3)[:, None]).all()


def test_direction(oracle):
    rng = np.random.default_rng(13)
    coords = rng.random((4000, 3)).astype(np.float32)
    direction = rng.integers(0, 4, size=4000).astype(np.int64)   # 3 = unconstrained
    _check(oracle, 16, coords, [0, 1500, 4000], direction=direction)


def test_duplicates_and_ties(oracle):
    rng = np.random.default_rng(14)
    base = rng.random((200, 3)).astype(np.float32)
    coords = np.concatenate([base, base, base[:50], np.round(rng.random((500, 3)) * 8) / 8]).astype(np.float32)
    gi, gd = _gpu_knn(10, coords, [0, coords.shape[0]])
    oi, od = oracle.binned_select_knn(10, coords, [0, coords.shape[0]])
    np.testing.assert_array_equal(np.sort(gd, axis=1), np.sort(od, axis=1))
    check_knn_properties(gi, gd, coords, [0, coords.shape[0]], 10)


def test_int32_row_splits_and_double_coords(oracle):
    from fastgraphcompute_amd import binned_select_knn
    rng = np.random.default_rng(15)
    coords = rng.random((2000, 3))
    rs = torch.tensor([0, 900, 2000], dtype=torch.int32, device="cuda")
    idx, dist = binned_select_knn(7, torch.as_tensor(coords, device="cuda"), rs)
    oi, od = oracle.binned_select_knn(7, coords.astype(np.float32), [0, 900, 2000])
    assert_knn_equal(idx.cpu().numpy(), dist.cpu().numpy(), oi, od)


def test_argument_errors():
    from fastgraphcompute_amd import binned_select_knn
    rs = torch.tensor([0, 10], device="cuda")
    # scripted wrapper, as in the reference: argument errors surface as torch.jit.Error (a RuntimeError)
    with pytest.raises((ValueError, RuntimeError, torch.jit.Error)):
        binned_select_knn(3, torch.rand(10, 0, device="cuda"), rs)
    with pytest.raises((ValueError, RuntimeError, torch.jit.Error)):
        binned_select_knn(3, torch.rand(10, 3, device="cuda"), rs, max_bin_dims=0)
    with pytest.raises((ValueError, RuntimeError, torch.jit.Error)):   # one coordinate: unsupported number of binning dimensions
        binned_select_knn(3, torch.rand(10, 1, device="cuda"), rs)
    with pytest.raises(RuntimeError):  # row splits do not cover the points
        binned_select_knn(3, torch.rand(10, 3, device="cuda"), torch.tensor([0, 8], device="cuda"))
    c = torch.rand(10, 3, device="cuda")
    c[0, 0] = float("inf")
    with pytest.raises(RuntimeError):
        binned_select_knn(3, c, rs)
    with pytest.raises(RuntimeError):
        binned_select_knn(3, torch.rand(10, 3), torch.tensor([0, 10]))


@pytest.mark.parametrize("n,K", [(1, 1), (1, 5), (2, 3), (63, 64), (64, 64), (65, 64), (129, 7)])
def test_tiny_inputs(oracle, n, K):
    rng = np.random.default_rng(n * 100 + K)
    coords = rng.random((n, 3)).astype(np.float32)
    gi, gd = _check(oracle, K, coords, [0, n])
    check_knn_properties(gi, gd, coords, [0, n], K)


@pytest.mark.parametrize("n", [1023, 1024, 1025, 4096, 4097, 32767, 32768, 32769, 40000])
def test_sizes_around_the_preparation_paths(oracle, n):
    """Inputs of up to 32768 points sort with one launch per pass (digit tables summed by every block), larger ones with
    three; the bin boundaries come from the position after the last point, which lies in a chunk of its own when the
    point count is a multiple of 64.  Four events of unequal size, one of them clustered (most bins empty)."""
    rng = np.random.default_rng(n)
    cuts = np.sort(rng.choice(np.arange(1, n), size=3, replace=False))
    rs = np.concatenate([[0], cuts, [n]]).astype(np.int64)
    coords = rng.random((n, 3)).astype(np.float32)
    coords[rs[1]:rs[2]] = (0.5 + 0.01 * rng.standard_normal((rs[2] - rs[1], 3))).astype(np.float32)
    gi, gd = _check(oracle, 10, coords, rs)
    check_knn_properties(gi, gd, coords, rs, 10)


def test_all_points_coincident(oracle):
    coords = np.full((700, 3), 0.25, dtype=np.float32)
    gi, gd = _gpu_knn(10, coords, [0, 300, 700])
    check_knn_properties(gi, gd, coords, [0, 300, 700], 10)
    assert (gd == 0).all()
    oi, od = oracle.binned_select_knn(10, coords, [0, 300, 700])
    np.testing.assert_array_equal(od, gd)


def test_one_dense_cluster_plus_outliers(oracle):
    # extreme imbalance: almost every point in one bin, a few far away (large dynamic range)
    rng = np.random.default_rng(21)
    coords = (rng.standard_normal((20000, 3)) * 1e-3).astype(np.float32)
    coords[:5] = np.array([[50, 50, 50], [-40, 10, 0], [0, 0, 99], [7, -80, 3], [1, 1, 1]], np.float32)
    gi, gd = _check(oracle, 32, coords, [0, 20000])
    check_knn_properties(gi, gd, coords, [0, 20000], 32)


def test_single_bin_per_dimension(oracle):
    rng = np.random.default_rng(22)
    coords = rng.random((3000, 4)).astype(np.float32)
    _check(oracle, 9, coords, [0, 1000, 3000], n_bins=torch.tensor(1, device="cuda"))
    _check(oracle, 9, coords, [0, 1000, 3000], n_bins=torch.tensor(2, device="cuda"))


def test_many_events_with_one_point(oracle):
    rng = np.random.default_rng(23)
    coords = rng.random((200, 3)).astype(np.float32)
    rs = np.arange(0, 201, dtype=np.int64)          # 200 events of one point each
    gi, gd = _check(oracle, 4, coords, rs)
    assert (gi[:, 0] == np.arange(200)).all() and (gi[:, 1:] == -1).all()


def test_sorted_space_op(oracle):
    """torch.ops.binned_select_knn.binned_select_knn, the reference's inner op on bin-sorted input
    (binned_select_knn.cpp:82-92): indices refer to the sorted order."""
    import fastgraphcompute_amd  # noqa: F401  (registers the ops)
    rng = np.random.default_rng(77)
    coords = rng.random((4000, 3)).astype(np.float32)
    rs = np.array([0, 1500, 4000])
    direction = rng.integers(0, 3, 4000)
    s = oracle.sorted_space(coords, rs, 12, direction=direction)
    t = lambda a: torch.as_tensor(np.ascontiguousarray(a), device="cuda")
    for use_dir in (False, True):
        oi, od, _, _ = oracle.knn_sorted(s["scoords"], s["sbin"], s["sdbin"], s["bin_boundaries"], s["n_bins"],
                                         s["bin_width"], 12, sdirection=s["sdirection"] if use_dir else None)
        gi, gd = torch.ops.binned_select_knn.binned_select_knn(
            t(s["scoords"]), t(s["sbin"]), t(s["sdbin"]), t(s["bin_boundaries"]), t(s["n_bins"]), t(s["bin_width"]),
            t(s["sdirection"]), False, use_dir, 12)
        assert_knn_equal(gi.cpu().numpy(), gd.cpu().numpy(), oi, od, what="direction %s" % use_dir)


def _adversarial(name, n, rng):
    if name == "line":                       # a 1-D manifold in 3-D
        t = rng.random(n)
        return np.stack([t, 2 * t + 0.5, -t], axis=1)
    if name == "plane":
        c = rng.random((n, 3))
        c[:, 2] = 0.25 * c[:, 0] - c[:, 1]
        return c
    if name == "offset":                     # a small cloud far from the origin: few mantissa bits left
        return 1.0e6 + rng.random((n, 3))
    if name == "tiny":
        return rng.random((n, 3)) * 1e-18
    if name == "huge":
        return (rng.random((n, 3)) - 0.5) * 1e15
    if name == "lattice":                    # massive ties
        return rng.integers(0, 7, size=(n, 3)).astype(np.float64)
    if name == "cauchy":                     # heavy tails: a dense core and far outliers
        return rng.standard_cauchy((n, 3))
    if name == "constant_dim":
        c = rng.random((n, 4))
        c[:, 1] = 3.5
        return c
    if name == "two_scales":                 # one tight blob next to a wide one
        c = rng.standard_normal((n, 3))
        c[: n // 2] *= 1e-4
        return c
    if name == "shell":                      # points on a sphere: every query's ball is mostly empty space
        v = rng.standard_normal((n, 3))
        return v / np.linalg.norm(v, axis=1, keepdims=True)
    raise ValueError(name)


@pytest.mark.parametrize("name", ["line", "plane", "offset", "tiny", "huge", "lattice", "cauchy", "constant_dim",
                                  "two_scales", "shell"])
def test_adversarial_distributions(oracle, name):
    """Distributions that stress the bin / bounding-box filters: the result must still be the exact kNN."""
    rng = np.random.default_rng(sum(map(ord, name)))
    coords = _adversarial(name, 6000, rng).astype(np.float32)
    rs = [0, 2500, 6000]
    for K in (8, 70):
        bi, bd = oracle.knn_brute(K, coords, np.array(rs))
        for n_bins in (None, 11, 29):        # the library's own coarse grid, and fine grids with many rings
            gi, gd = _gpu_knn(K, coords, rs, n_bins=None if n_bins is None else torch.tensor(n_bins))
            assert_knn_equal(gi, gd, bi, bd, what="%s K=%d n_bins=%s" % (name, K, n_bins))


def test_row_splits_host_copy_follows_the_tensor(oracle):
    """The host copy of a device row_splits tensor is reused only while that very tensor is unchanged."""
    from fastgraphcompute_amd import binned_select_knn
    from fastgraphcompute_amd import _ops
    rng = np.random.default_rng(77)
    coords = rng.random((3000, 3)).astype(np.float32)
    c = torch.from_numpy(coords).cuda()
    rs = torch.tensor([0, 1000, 3000], dtype=torch.int64, device="cuda")
    i1, d1 = binned_select_knn(8, c, rs)
    n_cached = len(_ops._RS_HOST)
    i2, d2 = binned_select_knn(8, c, rs)                  # same object: the cached copy
    assert len(_ops._RS_HOST) == n_cached and torch.equal(i1, i2) and torch.equal(d1, d2)
    oi, od = oracle.binned_select_knn(8, coords, np.array([0, 1000, 3000]))
    assert_knn_equal(i1.cpu().numpy(), d1.cpu().numpy(), oi, od, what="first")
    rs[1] = 2000                                           # in place: the version counter moves
    i3, d3 = binned_select_knn(8, c, rs)
    oi, od = oracle.binned_select_knn(8, coords, np.array([0, 2000, 3000]))
    assert_knn_equal(i3.cpu().numpy(), d3.cpu().numpy(), oi, od, what="after in-place change")
    del rs                                                 # a new tensor, whatever its address
    rs = torch.tensor([0, 500, 3000], dtype=torch.int64, device="cuda")
    i4, d4 = binned_select_knn(8, c, rs)
    oi, od = oracle.binned_select_knn(8, coords, np.array([0, 500, 3000]))
    assert_knn_equal(i4.cpu().numpy(), d4.cpu().numpy(), oi, od, what="new tensor")


def test_two_host_threads_on_their_own_streams():
    """Calls from two host threads, each on a stream of its own, do not see each other's state: one thread searches
    valid points over and over and must get the same rows as a call on its own, the other feeds non-finite
    coordinates and must get the input error every time - and only that thread."""
    import threading
    from fastgraphcompute_amd import binned_select_knn
    rng = np.random.default_rng(77)
    good = torch.from_numpy(rng.random((60000, 3)).astype(np.float32)).cuda()
    rs_good = torch.tensor([0, 25000, 60000], dtype=torch.int64, device="cuda")
    bad_h = rng.random((40000, 3)).astype(np.float32)
    bad_h[12345, 1] = np.nan
    bad = torch.from_numpy(bad_h).cuda()
    rs_bad = torch.tensor([0, 40000], dtype=torch.int64, device="cuda")
    ref_i, ref_d = binned_select_knn(24, good, rs_good)
    torch.cuda.synchronize()
    out = {"good_ok": 0, "good_err": [], "bad_raised": 0, "bad_other": []}

    def run_good():
        s = torch.cuda.Stream()
        with torch.cuda.stream(s):
            for _ in range(25):
                try:
                    i, d = binned_select_knn(24, good, rs_good)
                    s.synchronize()
                    if torch.equal(i, ref_i) and torch.equal(d, ref_d):
                        out["good_ok"] += 1
                    else:
                        out["good_err"].append("different rows")
                except Exception as e:  # noqa: BLE001
                    out["good_err"].append(repr(e))

    def run_bad():
        s = torch.cuda.Stream()
        with torch.cuda.stream(s):
            for _ in range(25):
                try:
                    binned_select_knn(24, bad, rs_bad)
                    s.synchronize()
                    out["bad_other"].append("no error")
                except RuntimeError as e:
                    if "non-finite" in str(e):
                        out["bad_raised"] += 1
                    else:
                        out["bad_other"].append(repr(e))

    ta, tb = threading.Thread(target=run_good), threading.Thread(target=run_bad)
    ta.start(); tb.start(); ta.join(); tb.join()
    torch.cuda.synchronize()
    assert out["good_err"] == [] and out["good_ok"] == 25, out
    assert out["bad_other"] == [] and out["bad_raised"] == 25, out


def test_statistics_build_returns_the_same_rows():
    """A call that asks for the search counters runs a second build of the search kernels (with the counters in
    its inner loops): rows and distances must be identical to the plain build's, and the counters plausible."""
    from fastgraphcompute_amd import binned_select_knn, config
    rng = np.random.default_rng(31)
    for D, K in ((3, 16), (4, 40), (8, 100)):
        n = 6000
        coords = torch.from_numpy(rng.standard_normal((n, D)).astype(np.float32)).cuda()
        rs = torch.tensor([0, 2500, n], device="cuda")
        i0, d0 = binned_select_knn(K, coords, rs)
        config.collect_stats = True
        try:
            i1, d1 = binned_select_knn(K, coords, rs)
        finally:
            config.collect_stats = False
        assert torch.equal(i0, i1) and torch.equal(d0, d1)
        from fastgraphcompute_amd import _ops
        st = _ops.last_stats
        assert st["n_vert"] == n and st["K"] == K
        assert st["distance_evaluations"] >= n * min(K, 2500 - 1) and st["candidate_chunks"] > 0
