"""CPU tests: the checker (oracle/) against the reference's golden vectors, the
committed outputs of the reference's own CPU kernels, brute force and closed
forms - and, where it has been built, against those kernels directly."""
import os

import numpy as np
import pytest

from tests.util import assert_knn_equal, check_knn_properties

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


@pytest.fixture(scope="module")
def golden():
    z = np.load(os.path.join(GOLDEN, "ref_cpu_kernels.npz"), allow_pickle=False)
    names = sorted({k.split("/")[0] for k in z.files})
    return z, names


# ------------------------------------------------------------------ binning
def test_binning_known_answers(oracle):
    # tests/test_bin_by_coordinates.py:26-82 and :111-162 of the reference
    a, f, nb, bw, nper = oracle.bin_by_coordinates(
        np.array([[0.1, 0.1], [2.5, 2.5], [4.9, 4.9]], np.float32), [0, 3], np.array([0.5], np.float32),
        np.array([10, 10]))
    np.testing.assert_array_equal(a, [[0, 0, 0], [0, 4, 4], [0, 9, 9]])
    np.testing.assert_array_equal(f, [0, 44, 99])
    exp = np.zeros(100, np.int64)
    exp[[0, 44, 99]] = 1
    np.testing.assert_array_equal(nper, exp)
    a, f, _, _, nper = oracle.bin_by_coordinates(
        np.array([[-1.0, -1.0], [5.1, 5.1], [0.7, 0.7]], np.float32), [0, 3], np.array([0.5], np.float32),
        np.array([10, 10]))
    np.testing.assert_array_equal(a, [[0, 0, 0], [0, 9, 9], [0, 3, 3]])
    np.testing.assert_array_equal(f, [0, 99, 33])


@pytest.mark.parametrize("ndims", [2, 4])
def test_binning_invariants(oracle, ndims):
    # tests/test_bin_by_coordinates.py:175-230 of the reference
    rng = np.random.default_rng(ndims)
    c = rng.random((1000, ndims)).astype(np.float32)
    rs = np.array([0, 300, 700, 1000])
    a, f, nb, bw, nper = oracle.bin_by_coordinates(c, rs, np.array([0.5], np.float32), np.array([10] * ndims))
    np.testing.assert_array_equal(a[:, 0], np.repeat(np.arange(3), np.diff(rs)))
    assert nper.sum() == 1000
    flat = a[:, 0].copy()
    for d in range(ndims):
        flat = flat * 10 + a[:, d + 1]
    np.testing.assert_array_equal(flat, f)      # coordinate 0 most significant, event above it
    np.testing.assert_array_equal(np.bincount(f, minlength=nper.size), nper)


def test_binning_reference_data_runs(oracle):
    c = np.load(os.path.join(GOLDEN, "bbc_coords.npy"), allow_pickle=False)
    a, f, nb, bw, nper = oracle.bin_by_coordinates(c, [0, c.shape[0]], None, 21)
    assert nper.sum() == c.shape[0] and list(nb) == [21, 21, 21] and a.max() <= 20 and a.min() >= 0


def test_n_bins_heuristic_benchmark_values(oracle):
    from fastgraphcompute_amd.workloads import cfg5_many_events_d8
    assert oracle.optimal_n_bins([0, 6000, 10000], 16, 3) == 18
    assert oracle.optimal_n_bins(np.arange(5) * 50000, 40, 3) == 30
    assert oracle.optimal_n_bins([0, 150000, 300000], 40, 3) == 30
    assert oracle.optimal_n_bins([0, 1000000], 64, 3) == 30
    assert oracle.optimal_n_bins(cfg5_many_events_d8()["row_splits"], 100, 3) == 13
    assert oracle.optimal_n_bins([0, 3333, 5000, 10000], 50, 3) == 11   # the reference's own large test
    assert oracle.optimal_n_bins([0, 40], 64, 3) == 5                    # lower clamp


def test_binning_matches_reference_kernel_outputs(oracle, golden):
    z, names = golden
    for nm in names:
        c, rs = z[nm + "/coords"], z[nm + "/row_splits"]
        mbd = int(z[nm + "/max_bin_dims"])
        Db = min(mbd, c.shape[1])
        a, f, nb, bw, nper = oracle.bin_by_coordinates(np.ascontiguousarray(c[:, :Db]), rs, None, z[nm + "/n_bins"])
        np.testing.assert_array_equal(a, z[nm + "/assigned"], err_msg=nm)
        np.testing.assert_array_equal(f, z[nm + "/flat"], err_msg=nm)
        np.testing.assert_array_equal(nper, z[nm + "/n_per_bin"], err_msg=nm)
        np.testing.assert_array_equal(bw, z[nm + "/bin_width"], err_msg=nm)


# ------------------------------------------------------------------ kNN forward
def test_knn_matches_reference_kernel_outputs(oracle, golden):
    """Slot for slot identical to the reference's CPU kernel (same visit order, same replacement rule)."""
    z, names = golden
    for nm in names:
        c, rs, K = z[nm + "/coords"], z[nm + "/row_splits"], int(z[nm + "/K"])
        mbd = int(z[nm + "/max_bin_dims"])
        s = oracle.sorted_space(c, rs, K, None, mbd)
        idx_s, dist_s, evals, _ = oracle.knn_sorted(s["scoords"], s["sbin"], s["sdbin"], s["bin_boundaries"],
                                                    s["n_bins"], s["bin_width"], K)
        np.testing.assert_array_equal(idx_s, z[nm + "/idx_sorted_space"], err_msg=nm)
        np.testing.assert_array_equal(dist_s, z[nm + "/dist_sorted_space"], err_msg=nm)
        idx, dsq = oracle.binned_select_knn(K, c, rs, max_bin_dims=mbd)
        np.testing.assert_array_equal(idx, z[nm + "/idx"], err_msg=nm)
        np.testing.assert_array_equal(dsq, z[nm + "/distsq"], err_msg=nm)
        assert evals > 0


@pytest.mark.parametrize("n,D,K,rs", [(1500, 3, 16, [0, 900, 1500]), (800, 2, 5, [0, 800]), (900, 8, 50, [0, 300, 450, 900]),
                                       (300, 3, 20, [0, 3, 3, 40, 41, 300])])
def test_knn_vs_brute_force(oracle, n, D, K, rs):
    rng = np.random.default_rng(n + D)
    c = rng.random((n, D)).astype(np.float32)
    idx, dsq = oracle.binned_select_knn(K, c, rs)
    bi, bd = oracle.knn_brute(K, c, rs)
    assert_knn_equal(idx, dsq, bi, bd)
    si, sd = np.take_along_axis(idx, np.argsort(np.where(idx < 0, np.inf, dsq), axis=1, kind="stable"), 1), None
    # numpy brute force, independent of the C code
    for e in range(len(rs) - 1):
        a, b = rs[e], rs[e + 1]
        if b - a < 2:
            continue
        d2 = ((c[a:b, None, :].astype(np.float64) - c[None, a:b, :].astype(np.float64)) ** 2).sum(-1)
        kk = min(K, b - a)
        ref = np.sort(d2, axis=1)[:, :kk]
        got = np.sort(np.where(idx[a:b] < 0, np.inf, dsq[a:b]), axis=1)[:, :kk]
        np.testing.assert_allclose(got, ref, rtol=1e-5, atol=1e-7)


def test_knn_threads_and_sampling_agree(oracle):
    from fastgraphcompute_amd.workloads import cfg4_zipf_blobs
    w = cfg4_zipf_blobs(0.01)
    i1, d1, st1 = oracle.binned_select_knn(w["K"], w["coords"], w["row_splits"], n_threads=1, return_stats=True)
    i8, d8, st8 = oracle.binned_select_knn(w["K"], w["coords"], w["row_splits"], n_threads=4, return_stats=True)
    np.testing.assert_array_equal(i1, i8)
    np.testing.assert_array_equal(d1, d8)
    assert st1["C_eval"] == st8["C_eval"]
    check_knn_properties(*_sorted_rows(i1, d1), w["coords"], w["row_splits"], w["K"], ascending=True)


def _sorted_rows(idx, dist):
    key = np.argsort(np.where(idx[:, 1:] < 0, np.inf, dist[:, 1:]), axis=1, kind="stable")
    i = np.concatenate([idx[:, :1], np.take_along_axis(idx[:, 1:], key, 1)], 1)
    d = np.concatenate([dist[:, :1], np.take_along_axis(dist[:, 1:], key, 1)], 1)
    return i, d


def test_knn_direction_semantics(oracle):
    rng = np.random.default_rng(5)
    c = rng.random((400, 3)).astype(np.float32)
    direction = rng.integers(0, 4, 400)
    idx, dsq = oracle.binned_select_knn(6, c, [0, 400], direction=direction)
    for i in range(400):
        if direction[i] in (0, 2):          # may not have neighbours
            assert (idx[i, 1:] == -1).all()
        else:
            nb = idx[i, 1:]
            assert (nb >= 0).all() and not np.isin(direction[nb], (1, 2)).any()
            allowed = np.nonzero(~np.isin(direction, (1, 2)))[0]
            allowed = allowed[allowed != i]
            d2 = ((c[allowed] - c[i]) ** 2).sum(1)
            np.testing.assert_allclose(np.sort(dsq[i, 1:]), np.sort(d2)[:5], rtol=1e-5)


# ------------------------------------------------------------------ index_replacer / gradient / aggregation
def test_index_replacer_golden(oracle):
    np.random.seed(34)      # tests/test_index_replacer.py:11-74 of the reference
    tbr = np.arange(100)
    tbr[np.random.choice(100, 10, replace=False)] = -1
    np.random.shuffle(tbr)
    tbr = tbr.reshape(20, 5)
    rpl = np.arange(100)
    np.random.shuffle(rpl)
    out = oracle.index_replacer(tbr, rpl).reshape(20, 5)
    np.testing.assert_array_equal(out, np.load(os.path.join(GOLDEN, "index_replacer_expected.npy")))


def test_grad_matches_reference_kernel_outputs(oracle, golden):
    z, names = golden
    for nm in names:
        c, K = z[nm + "/coords"], int(z[nm + "/K"])
        gd = np.random.default_rng(99).standard_normal((c.shape[0], K)).astype(np.float32)
        g = oracle.knn_grad(gd, z[nm + "/idx"].astype(np.int64), c)
        np.testing.assert_array_equal(g, z[nm + "/grad_coords"], err_msg=nm)


def test_grad_closed_form_and_autograd(oracle):
    import torch
    rng = np.random.default_rng(8)
    n, D, K = 500, 4, 10
    c = rng.random((n, D)).astype(np.float32)
    idx, dsq = oracle.binned_select_knn(K, c, [0, n])
    gd = rng.standard_normal((n, K)).astype(np.float32)
    g = oracle.knn_grad(gd, idx, c)
    x = torch.from_numpy(c).double().requires_grad_(True)
    d = ((x[torch.from_numpy(idx)] - x[:, None, :]) ** 2).sum(-1)
    (d * torch.from_numpy(gd).double()).sum().backward()
    np.testing.assert_allclose(g, x.grad.numpy(), rtol=1e-4, atol=1e-5)


def test_select_with_default_properties(oracle):
    rng = np.random.default_rng(9)
    idx = rng.integers(-1, 50, (200, 10))
    feat = np.repeat(np.arange(50, dtype=np.float32)[:, None], 3, 1)
    out = oracle.select_with_default(idx, feat, -9.0)
    assert out.shape == (200, 10, 3)
    np.testing.assert_array_equal(out[..., 0], np.where(idx == -1, -9.0, idx))


def test_aggregation_c_kernel_vs_torch_composition(oracle):
    import torch
    rng = np.random.default_rng(10)
    n, K, P = 300, 12, 7
    c = rng.random((n, 3)).astype(np.float32)
    idx, dsq = oracle.binned_select_knn(K, c, [0, 5, n])
    feat = rng.standard_normal((n, P)).astype(np.float32)
    m, x, am = oracle.gravnet_aggregate(idx, dsq * 30, feat)
    tm, tx = oracle.gravnet_aggregate_torch(torch.from_numpy(idx), torch.from_numpy(dsq * 30), torch.from_numpy(feat))
    np.testing.assert_allclose(m, tm.numpy(), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(x, tx.numpy(), rtol=1e-5, atol=1e-6)
    assert (m[:5, :] * K == m[:5, :] * K).all() and am.min() >= 0 and am.max() < K


# ------------------------------------------------------------------ live comparison with the compiled reference kernels
def test_against_compiled_reference_kernels(oracle):
    if oracle.ref_lib() is None:
        pytest.skip("oracle/_ref not built (needs the reference checkout)")
    from fastgraphcompute_amd.workloads import cfg1_uniform_small, cfg2_blobs_4events
    for w in (cfg1_uniform_small(), cfg2_blobs_4events(0.05)):
        a = oracle.binned_select_knn(w["K"], w["coords"], w["row_splits"])
        b = oracle.binned_select_knn(w["K"], w["coords"], w["row_splits"], use_ref=True)
        np.testing.assert_array_equal(a[0], b[0])
        np.testing.assert_array_equal(a[1], b[1])
        gd = np.random.default_rng(1).standard_normal(a[1].shape).astype(np.float32)
        np.testing.assert_array_equal(oracle.knn_grad(gd, a[0], w["coords"]),
                                      oracle.knn_grad(gd, a[0], w["coords"], a[1], use_ref=True))
        Db = 3
        r1 = oracle.bin_by_coordinates(np.ascontiguousarray(w["coords"][:, :Db]), w["row_splits"], None, 17)
        r2 = oracle.bin_by_coordinates(np.ascontiguousarray(w["coords"][:, :Db]), w["row_splits"], None, 17, use_ref=True)
        for x, y in zip(r1, r2):
            np.testing.assert_array_equal(x, y)


def test_reference_kernel_on_a_query_sample(oracle):
    """How bench.py times the reference's own kernel on a bounded sample: direction flag 0 (may only be a neighbour)
    for all points but every s-th, a flag outside 0..2 for the sampled ones, use_direction on
    (binned_select_knn_cpu.cpp:80-83,157-160).  The sampled rows equal a search without any flags."""
    if oracle.ref_lib() is None:
        pytest.skip("oracle/_ref not built (needs the reference checkout)")
    from fastgraphcompute_amd.workloads import cfg2_blobs_4events
    w = cfg2_blobs_4events(0.03)
    K = 12
    s = oracle.sorted_space(w["coords"], w["row_splits"], K)
    args = (s["scoords"], s["sbin"], s["sdbin"], s["bin_boundaries"], s["n_bins"], s["bin_width"], K)
    n = w["coords"].shape[0]
    full_i, full_d, _, _ = oracle.knn_sorted(*args, use_ref=True)
    stride = 7
    direction = np.zeros(n, dtype=np.int64)
    direction[::stride] = 3
    samp_i, samp_d, _, _ = oracle.knn_sorted(*args, sdirection=direction, use_ref=True)
    np.testing.assert_array_equal(samp_i[::stride], full_i[::stride])
    np.testing.assert_array_equal(samp_d[::stride], full_d[::stride])
    port_i, port_d, _, _ = oracle.knn_sorted(*args, n_threads=1, query_stride=stride)
    np.testing.assert_array_equal(port_i[::stride], full_i[::stride])
    np.testing.assert_array_equal(port_d[::stride], full_d[::stride])
