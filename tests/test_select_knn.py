"""select_knn (k nearest neighbours inside a radius): the checker against the definition and the reference's
compiled CPU code; the GPU op against the checker.  The reference holds no test or fixture for this op, so the
committed vectors are outputs of its compiled select_knn_cpu."""
import os

import numpy as np
import pytest
import torch

from tests.util import assert_knn_equal

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def brute(K, c, rs, radius):
    """Definition in float64 distances of float32 differences (exactly the float32 sum for D <= 2 terms is not
    guaranteed, so the comparison below uses the tolerance of the parity contract)."""
    n = c.shape[0]
    idx = np.full((n, K), -1, dtype=np.int64)
    dist = np.zeros((n, K), dtype=np.float32)
    r2 = np.float32(radius * radius) if radius > 0 else None
    for e in range(len(rs) - 1):
        lo, hi = rs[e], rs[e + 1]
        for i in range(lo, hi):
            d = np.zeros(hi - lo, dtype=np.float32)
            for k in range(c.shape[1]):
                t = c[i, k] - c[lo:hi, k]
                d = d + t * t
            cand = [(d[j - lo], j) for j in range(lo, hi) if j != i and (r2 is None or d[j - lo] <= r2)]
            cand.sort()
            idx[i, 0] = i
            for s, (dd, j) in enumerate(cand[:K - 1]):
                idx[i, s + 1] = j
                dist[i, s + 1] = dd
    return idx, dist


@pytest.fixture(scope="module")
def golden():
    z = np.load(os.path.join(GOLDEN, "ref_select_knn.npz"), allow_pickle=False)
    return z, sorted({k.split("/")[0] for k in z.files})


def test_checker_against_committed_reference_outputs(oracle, golden):
    z, names = golden
    assert len(names) == 4
    for name in names:
        idx, dist = oracle.select_knn(int(z[name + "/K"]), z[name + "/coords"], z[name + "/row_splits"],
                                      float(z[name + "/max_radius"]))
        np.testing.assert_array_equal(idx, z[name + "/idx"], err_msg=name)        # slot for slot
        np.testing.assert_array_equal(dist, z[name + "/distsq"], err_msg=name)


def test_checker_against_the_definition(oracle):
    rng = np.random.default_rng(12)
    c = rng.random((400, 3)).astype(np.float32)
    rs = np.array([0, 150, 400])
    for radius in (-1.0, 0.15, 0.05, 1e-4):
        idx, dist = oracle.select_knn(7, c, rs, radius)
        bi, bd = brute(7, c, rs, radius)
        assert_knn_equal(idx, dist, bi, bd, what="radius %g" % radius)


def test_checker_against_compiled_reference(oracle):
    if oracle.ref_lib() is None:
        pytest.skip("reference CPU code not built here")
    rng = np.random.default_rng(13)
    for n, D, K, radius in ((500, 2, 5, 0.1), (900, 4, 16, 0.3), (50, 3, 64, -1.0), (300, 3, 1, 0.2)):
        c = rng.random((n, D)).astype(np.float32)
        rs = np.array([0, n // 3, n])
        a = oracle.select_knn(K, c, rs, radius)
        b = oracle.select_knn(K, c, rs, radius, use_ref=True)
        np.testing.assert_array_equal(a[0], b[0])
        np.testing.assert_array_equal(a[1], b[1])


# ------------------------------------------------------------------ GPU
def _gpu(K, c, rs, radius):
    from fastgraphcompute_amd.extensions.select_knn import select_knn
    idx, dist = select_knn(K, torch.as_tensor(c, device="cuda"), torch.as_tensor(rs, device="cuda"), radius)
    assert idx.dtype == torch.int64 and dist.dtype == torch.float32
    return idx.cpu().numpy(), dist.cpu().numpy()


@pytest.mark.gpu
def test_gpu_against_committed_reference_outputs(golden):
    z, names = golden
    for name in names:
        gi, gd = _gpu(int(z[name + "/K"]), z[name + "/coords"], z[name + "/row_splits"], float(z[name + "/max_radius"]))
        assert_knn_equal(gi, gd, z[name + "/idx"].astype(np.int64), z[name + "/distsq"], what=name)


@pytest.mark.gpu
@pytest.mark.parametrize("n,D,K,radius", [(20000, 3, 16, 0.03), (20000, 3, 16, -1.0), (5000, 4, 40, 0.2),
                                           (3000, 2, 100, 0.05), (8000, 8, 10, 0.6), (4000, 1, 6, 0.01),
                                           (2000, 3, 8, 1e-6)])
def test_gpu_against_checker(oracle, n, D, K, radius):
    rng = np.random.default_rng(n + D + K)
    c = rng.random((n, D)).astype(np.float32)
    rs = np.array([0, n // 4, n // 4, n])
    gi, gd = _gpu(K, c, rs, radius)
    oi, od = oracle.select_knn(K, c, rs, radius)
    assert_knn_equal(gi, gd, oi, od)
    if radius > 0:
        assert (gd <= np.float32(radius * radius)).all()


@pytest.mark.gpu
def test_gpu_radius_is_inclusive_and_op_name(oracle):
    # points on a line at spacing 0.25: radius 0.25 must include the direct neighbours (distsq == r^2 exactly)
    c = np.stack([np.arange(16, dtype=np.float32) * 0.25, np.zeros(16, np.float32)], axis=1)
    rs = np.array([0, 16])
    m = torch.zeros(16, dtype=torch.int64, device="cuda")
    idx, dist = torch.ops.select_knn.select_knn(torch.as_tensor(c, device="cuda"), torch.as_tensor(rs, device="cuda"),
                                                m, 4, 0.25, 0)
    oi, od = oracle.select_knn(4, c, rs, 0.25)
    assert_knn_equal(idx.cpu().numpy(), dist.cpu().numpy(), oi, od)
    assert int((idx[5] >= 0).sum()) == 3          # itself and both neighbours at exactly the radius
    with pytest.raises(RuntimeError):
        torch.ops.select_knn.select_knn(torch.as_tensor(c), torch.as_tensor(rs), m.cpu(), 4, 0.25, 0)
