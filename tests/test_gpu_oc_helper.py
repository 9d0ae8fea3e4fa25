"""oc_helper_matrices and its helper ops on the GPU: bit-exact against the CPU checker, the reference's
hand-written expectation, its stored matrices and the committed outputs of its compiled CPU code."""
import os

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def dev(a):
    return torch.tensor(np.asarray(a), dtype=torch.int64, device="cuda")


@pytest.fixture(scope="module")
def oc_golden():
    z = np.load(os.path.join(GOLDEN, "ref_oc_helper.npz"), allow_pickle=False)
    return z, sorted({k.split("/")[0] for k in z.files})


def run(a, rs, calc_m_not=True):
    from fastgraphcompute_amd import oc_helper_matrices
    M, M_not, nobj = oc_helper_matrices(dev(a), dev(rs), calc_m_not)
    assert M.dtype == torch.int64 and M_not.dtype == torch.int64 and M.is_cuda and M_not.is_cuda
    return M.cpu().numpy(), M_not.cpu().numpy(), nobj.cpu().numpy()


def test_hand_written_expectation(oracle):
    # tests/test_oc_helper.py:28-126 of the reference
    a = np.array([3, 7, 3, -1, -1, 3, 7, 1, 1, 0, 0, -1, 1, 1, -1, 3, -1, 19, 3, 2, -1, 19])
    rs = np.array([0, 15, 22])
    M, M_not, nobj = run(a, rs)
    np.testing.assert_array_equal(nobj, [4, 3])
    assert M.shape == (7, 4) and M_not.shape == (7, 15)
    M_exp = np.array([[0, 2, 5, -1], [1, 6, -1, -1], [7, 8, 12, 13], [9, 10, -1, -1],
                      [15, 18, -1, -1], [17, 21, -1, -1], [19, -1, -1, -1]])
    M_not_exp = np.array([
        [1, 3, 4, 6, 7, 8, 9, 10, 11, 12, 13, 14, -1, -1, -1],
        [0, 2, 3, 4, 5, 7, 8, 9, 10, 11, 12, 13, 14, -1, -1],
        [0, 1, 2, 3, 4, 5, 6, 9, 10, 11, 14, -1, -1, -1, -1],
        [0, 1, 2, 3, 4, 5, 6, 7, 8, 11, 12, 13, 14, -1, -1],
        [16, 17, 19, 20, 21, -1, -1, -1, -1, -1, -1, -1, -1, -1, -1],
        [15, 16, 18, 19, 20, -1, -1, -1, -1, -1, -1, -1, -1, -1, -1],
        [15, 16, 17, 18, 20, 21, -1, -1, -1, -1, -1, -1, -1, -1, -1]])
    got = oracle.oc_sort_rows(M, M_not)
    exp = oracle.oc_sort_rows(M_exp, M_not_exp)
    np.testing.assert_array_equal(got[0], exp[0])
    np.testing.assert_array_equal(got[1], exp[1])


def test_stored_matrices_of_the_reference(oracle, oc_golden):
    # tests/test_oc_helper.py:201-230 of the reference
    z, _ = oc_golden
    M, M_not, _ = run(z["stored/asso"], z["stored/row_splits"])
    M_exp = np.load(os.path.join(GOLDEN, "oc_helper_large_M.npy"), allow_pickle=False).astype(np.int64)
    M_not_exp = np.load(os.path.join(GOLDEN, "oc_helper_large_M_not.npy"), allow_pickle=False).astype(np.int64)
    got = oracle.oc_sort_rows(M, M_not)
    exp = oracle.oc_sort_rows(M_exp, M_not_exp)
    np.testing.assert_array_equal(got[0], exp[0])
    np.testing.assert_array_equal(got[1], exp[1])


def test_committed_reference_outputs(oc_golden):
    from fastgraphcompute_amd.extensions.oc_helper import max_same_valued_entries_per_row_split
    z, names = oc_golden
    for name in names:
        a, rs = z[name + "/asso"], z[name + "/row_splits"]
        M, M_not, nobj = run(a, rs)
        np.testing.assert_array_equal(M, z[name + "/M"], err_msg=name)          # same row order: (split, value)
        np.testing.assert_array_equal(M_not, z[name + "/M_not"], err_msg=name)
        np.testing.assert_array_equal(nobj, z[name + "/filter_objects_per_split"], err_msg=name)
        for flt, tag in ((True, "/filter"), (False, "/nofilter")):
            mx, g, no = max_same_valued_entries_per_row_split(dev(a), dev(rs), flt)
            np.testing.assert_array_equal(mx.cpu().numpy(), z[name + tag + "_max_per_split"], err_msg=name + tag)
            assert int(g) == int(z[name + tag + "_global_max"]) and g.is_cuda and g.dim() == 0
            np.testing.assert_array_equal(no.cpu().numpy(), z[name + tag + "_objects_per_split"], err_msg=name + tag)


@pytest.mark.parametrize("n,nval,splits,neg", [
    (100000, 999, [0, 1.0], 0.001),                    # the reference's large-scale case (test_oc_helper.py:177-183)
    (100000, 100, [0, 0.25, 0.5, 1.0], 0.01),          # test_oc_helper.py:234-240
    (50000, 49000, [0, 0.3, 1.0], 0.0),                # nearly every vertex its own object
    (30000, 3, [0, 0.5, 0.5, 0.9, 1.0], 0.5),          # few wide objects, an empty split, half noise
    (4097, 17, [0, 1.0], 0.1),                         # one vertex past a block of the compaction
    (70000, 40, [0] + [i / 70 for i in range(1, 71)], 0.2),   # many splits
])
def test_random_against_checker(oracle, n, nval, splits, neg):
    rng = np.random.default_rng(n + nval)
    a = rng.integers(0, nval, n)
    a[rng.random(n) < neg] = -1
    rs = np.array([int(round(f * n)) for f in splits])
    M, M_not, nobj = run(a, rs)
    Me, M_not_e, nobj_e = oracle.oc_helper_matrices(a, rs)
    np.testing.assert_array_equal(nobj, nobj_e)
    np.testing.assert_array_equal(M, Me)
    np.testing.assert_array_equal(M_not, M_not_e)


def test_values_beyond_32_bits_and_other_negatives(oracle):
    rng = np.random.default_rng(5)
    a = rng.integers(0, 50, 20000) * 987654321987 + 3
    a[rng.random(20000) < 0.1] = -1
    a[rng.random(20000) < 0.05] = -7           # any negative value forms no object
    rs = np.array([0, 5000, 20000])
    M, M_not, nobj = run(a, rs)
    Me, M_not_e, nobj_e = oracle.oc_helper_matrices(a, rs)
    np.testing.assert_array_equal(nobj, nobj_e)
    np.testing.assert_array_equal(M, Me)
    np.testing.assert_array_equal(M_not, M_not_e)
    a2 = np.array([2 ** 62, -2 ** 62, 5, 2 ** 62, 2 ** 31, 2 ** 32, 2 ** 32 - 1, 2 ** 32 - 2])
    M, M_not, nobj = run(a2, [0, 8])
    Me, M_not_e, nobj_e = oracle.oc_helper_matrices(a2, np.array([0, 8]))
    np.testing.assert_array_equal(M, Me)
    np.testing.assert_array_equal(M_not, M_not_e)


def test_without_m_not_and_degenerate_inputs(oracle):
    a = np.array([1, 1, 2, -1, 2, 2])
    M, M_not, nobj = run(a, [0, 6], calc_m_not=False)
    assert M_not.shape == (0, 0)           # as the reference's device op, oc_helper_cuda_kernel.cu:171-176
    np.testing.assert_array_equal(M, [[0, 1, -1], [2, 4, 5]])
    M, M_not, nobj = run(np.full(40, -1), [0, 10, 40])
    assert M.shape == (0, 0) and M_not.shape == (0, 30)
    np.testing.assert_array_equal(nobj, [0, 0])
    M, M_not, nobj = run(np.array([4]), [0, 1])
    np.testing.assert_array_equal(M, [[0]])
    np.testing.assert_array_equal(M_not, [[-1]])


def test_select_with_default_consistency():
    # tests/test_oc_helper.py:143-199 of the reference
    from fastgraphcompute_amd import oc_helper_matrices, select_with_default
    torch.manual_seed(3)
    a = torch.randint(0, 1000, (100000,), dtype=torch.int64) - 1
    a = a.cuda()
    rs = torch.tensor([0, a.numel()], dtype=torch.int64, device="cuda")
    M, M_not, _ = oc_helper_matrices(a, rs)
    for feat, dflt in ((a.unsqueeze(-1), -100), (a.float().unsqueeze(-1), -100.0),
                       (a.unsqueeze(-1).repeat(1, 10), -100)):
        sel = select_with_default(M, feat, dflt)
        assert sel.dtype == feat.dtype and sel.is_cuda
        ok = (sel == sel[:, 0:1]) | (sel == dflt)
        assert bool(ok.all())
    # M_not rows never contain the object's own vertices
    sel = select_with_default(M_not, a.unsqueeze(-1), -100)[:, :, 0]
    own = select_with_default(M, a.unsqueeze(-1), -100)[:, 0:1, 0]
    assert bool((sel != own).all())


def test_reference_op_with_caller_order(oracle):
    # torch.ops.oc_helper_cuda.oc_helper_cuda as oc_helper.py:209-218 of the reference calls it
    rng = np.random.default_rng(11)
    a = rng.integers(-2, 60, 9000)
    rs = np.array([0, 2000, 2000, 9000])
    uv, ur, gmax, lengths, max_len, nobj = oracle.oc_helper_inputs(a, rs, True)
    order = rng.permutation(uv.size)
    uv, ur = uv[order], ur[order]
    uv = np.concatenate([uv, [12345, -2]])          # a pair without vertices, and a negative value
    ur = np.concatenate([ur, [0, 2]])
    gmax = max(gmax, int((a[2000:] == -2).sum()))
    Me, M_not_e = oracle.oc_calc_m(a, uv, ur, rs, gmax, max_len)
    for calc_not in (True, False):
        M, M_not = torch.ops.oc_helper_cuda.oc_helper_cuda(dev(a), dev(uv), dev(ur), dev(rs), dev([gmax]),
                                                           dev([max_len]), calc_not)
        np.testing.assert_array_equal(M.cpu().numpy(), Me)
        if calc_not:
            np.testing.assert_array_equal(M_not.cpu().numpy(), M_not_e)
        else:
            assert tuple(M_not.shape) == (0, 0)
    with pytest.raises(RuntimeError):               # an object wider than the caller's M
        torch.ops.oc_helper_cuda.oc_helper_cuda(dev(a), dev(uv), dev(ur), dev(rs), dev([gmax - 1]), dev([max_len]),
                                                True)
    with pytest.raises(RuntimeError):
        torch.ops.oc_helper_cuda.oc_helper_cuda(dev(a), dev(uv), dev(ur), dev(rs), dev([gmax, 1]), dev([max_len]),
                                                True)


def test_argument_errors():
    from fastgraphcompute_amd import oc_helper_matrices
    a = torch.tensor([1, 1, 2], dtype=torch.int64, device="cuda")
    rs = torch.tensor([0, 3], dtype=torch.int64, device="cuda")
    errs = (RuntimeError, ValueError, AssertionError, torch.jit.Error)
    with pytest.raises(errs):
        oc_helper_matrices(a.int(), rs)
    with pytest.raises(errs):
        oc_helper_matrices(a, rs.int())
    with pytest.raises(errs):
        oc_helper_matrices(a.cpu(), rs.cpu())            # no CPU fallback
    with pytest.raises(errs):
        oc_helper_matrices(a, rs.cpu())
    with pytest.raises(errs):
        oc_helper_matrices(a, torch.tensor([0, 2], dtype=torch.int64, device="cuda"))
    with pytest.raises(errs):
        oc_helper_matrices(a, torch.tensor([0, 2, 1, 3], dtype=torch.int64, device="cuda"))


def test_scripted_module(oracle):
    from fastgraphcompute_amd.extensions.oc_helper import oc_helper_matrices

    class Wrap(torch.nn.Module):
        def forward(self, a, rs):
            M, M_not, n = oc_helper_matrices(a, rs)
            return M, M_not, n

    rng = np.random.default_rng(2)
    a = rng.integers(-1, 30, 5000)
    rs = np.array([0, 1000, 5000])
    m = torch.jit.script(Wrap())
    M, M_not, n = m(dev(a), dev(rs))
    Me, M_not_e, ne = oracle.oc_helper_matrices(a, rs)
    np.testing.assert_array_equal(M.cpu().numpy(), Me)
    np.testing.assert_array_equal(M_not.cpu().numpy(), M_not_e)
    np.testing.assert_array_equal(n.cpu().numpy(), ne)


def test_full_size_properties():
    """The benchmark shape (200 000 vertices, 4 row splits, 2 000 objects): properties that hold for any input."""
    from fastgraphcompute_amd import oc_helper_matrices
    from fastgraphcompute_amd.workloads import oc_workload
    a_np, rs_np = oc_workload()
    a, rs = dev(a_np), dev(rs_np)
    M, M_not, nobj = oc_helper_matrices(a, rs)
    U = M.shape[0]
    assert int(nobj.sum()) == U and M_not.shape == (U, int(np.diff(rs_np).max()))
    valid = M >= 0
    vals = torch.where(valid, a[M.clamp(min=0)], a[M[:, 0:1]].expand_as(M))
    assert bool((vals == vals[:, 0:1]).all()) and bool((vals[:, 0] >= 0).all())       # one truth index per row
    cnt = valid.sum(1)
    assert int(cnt.sum()) == int((a >= 0).sum())                                        # every object vertex once
    srt = torch.where(valid, M, torch.full_like(M, 2 ** 62))
    assert bool((srt[:, 1:] >= srt[:, :-1]).all())                                      # ascending, padding last
    split = torch.bucketize(M[:, 0], rs[1:], right=True)
    length = (rs[1:] - rs[:-1])[split]
    nvalid = (M_not >= 0).sum(1)
    assert bool((nvalid + cnt == length).all())                                         # M and M_not tile the split
    v = M_not >= 0
    assert bool((a[M_not.clamp(min=0)][v] != vals[:, 0:1].expand_as(M_not)[v]).all())
    inside = (M_not >= rs[split].unsqueeze(1)) & (M_not < rs[split + 1].unsqueeze(1))
    assert bool((inside | ~v).all())
    srt = torch.where(v, M_not, torch.full_like(M_not, 2 ** 62))
    assert bool((srt[:, 1:] >= srt[:, :-1]).all())
    assert int(M_not[v].sum()) == int(((rs[split] + rs[split + 1] - 1) * length // 2).sum()
                                      - torch.where(valid, M, torch.zeros_like(M)).sum())
