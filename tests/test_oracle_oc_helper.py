"""CPU tests: the object-condensation helper of the checker (oracle/) against the reference's hand-written
expectation, its stored matrices, the committed outputs of the reference's compiled CPU code, brute force - and,
where it has been built, against that compiled code directly."""
import os

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


@pytest.fixture(scope="module")
def oc_golden():
    z = np.load(os.path.join(GOLDEN, "ref_oc_helper.npz"), allow_pickle=False)
    return z, sorted({k.split("/")[0] for k in z.files})


def brute_matrices(a, rs):
    """The definition, element by element in Python (small inputs only)."""
    rows_m, rows_n = [], []
    nobj = []
    for r in range(len(rs) - 1):
        seg = range(rs[r], rs[r + 1])
        vals = sorted({int(a[i]) for i in seg if a[i] >= 0})
        nobj.append(len(vals))
        for v in vals:
            rows_m.append([i for i in seg if a[i] == v])
            rows_n.append([i for i in seg if a[i] != v])
    wm = max([len(x) for x in rows_m], default=0)
    wn = int(np.max(np.diff(rs)))
    M = np.array([x + [-1] * (wm - len(x)) for x in rows_m], dtype=np.int64).reshape(len(rows_m), wm)
    Mn = np.array([x + [-1] * (wn - len(x)) for x in rows_n], dtype=np.int64).reshape(len(rows_n), wn)
    return M, Mn, np.array(nobj, dtype=np.int64)


def test_hand_written_expectation(oracle):
    # tests/test_oc_helper.py:28-126 of the reference
    a = np.array([3, 7, 3, -1, -1, 3, 7, 1, 1, 0, 0, -1, 1, 1, -1, 3, -1, 19, 3, 2, -1, 19])
    rs = np.array([0, 15, 22])
    M, M_not, nobj = oracle.oc_helper_matrices(a, rs)
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
    # tests/test_oc_helper.py:201-230 of the reference; its input (torch.manual_seed(42), randint) is the
    # "stored" case of the fixture
    z, _ = oc_golden
    M, M_not, _ = oracle.oc_helper_matrices(z["stored/asso"], z["stored/row_splits"])
    M_exp = np.load(os.path.join(GOLDEN, "oc_helper_large_M.npy"), allow_pickle=False).astype(np.int64)
    M_not_exp = np.load(os.path.join(GOLDEN, "oc_helper_large_M_not.npy"), allow_pickle=False).astype(np.int64)
    got = oracle.oc_sort_rows(M, M_not)
    exp = oracle.oc_sort_rows(M_exp, M_not_exp)
    np.testing.assert_array_equal(got[0], exp[0])
    np.testing.assert_array_equal(got[1], exp[1])


def test_against_committed_reference_outputs(oracle, oc_golden):
    z, names = oc_golden
    assert len(names) >= 7
    for name in names:
        a, rs = z[name + "/asso"], z[name + "/row_splits"]
        uv, ur, gmax, lengths, max_len, nobj = oracle.oc_helper_inputs(a, rs, True)
        np.testing.assert_array_equal(uv, z[name + "/unique_idx"])
        np.testing.assert_array_equal(ur, z[name + "/unique_rs"])
        M, M_not = oracle.oc_calc_m(a, uv, ur, rs, gmax, max_len, True)
        np.testing.assert_array_equal(M, z[name + "/M"], err_msg=name)
        np.testing.assert_array_equal(M_not, z[name + "/M_not"], err_msg=name)
        for flt, tag in ((True, "/filter"), (False, "/nofilter")):
            mx, g, no = oracle.max_same_valued_entries_per_row_split(a, rs, flt)
            np.testing.assert_array_equal(mx, z[name + tag + "_max_per_split"], err_msg=name)
            assert g == int(z[name + tag + "_global_max"])
            np.testing.assert_array_equal(no, z[name + tag + "_objects_per_split"], err_msg=name)
        assert gmax == int(z[name + "/filter_global_max"])
        np.testing.assert_array_equal(nobj, z[name + "/filter_objects_per_split"])


def test_against_the_definition(oracle, oc_golden):
    z, names = oc_golden
    for name in names:
        a, rs = z[name + "/asso"], z[name + "/row_splits"]
        if a.size > 1200:
            a, rs = a[:1200], np.minimum(rs, 1200)
        M, M_not, nobj = oracle.oc_helper_matrices(a, rs)
        bm, bn, bo = brute_matrices(a, rs)
        np.testing.assert_array_equal(M, bm, err_msg=name)
        np.testing.assert_array_equal(M_not, bn, err_msg=name)
        np.testing.assert_array_equal(nobj, bo, err_msg=name)


def test_helper_known_answer(oracle):
    # tests/test_oc_helper_helper.py:113-131 of the reference (its torch.unique restatement, by hand)
    a = np.array([-1, -1, 2, 3, 3, 3, 8, 1, 0, 90, 2, 2, 4, 5, -1, -1, 2])
    rs = np.array([0, 9, 17])
    mx, g, no = oracle.max_same_valued_entries_per_row_split(a, rs, True)
    np.testing.assert_array_equal(mx, [3, 3])
    assert g == 3
    np.testing.assert_array_equal(no, [5, 4])
    mx, g, no = oracle.max_same_valued_entries_per_row_split(a, rs, False)
    np.testing.assert_array_equal(mx, [3, 3])
    np.testing.assert_array_equal(no, [6, 5])


def test_against_compiled_reference(oracle):
    if oracle.ref_lib() is None:
        pytest.skip("reference CPU code not built here")
    rng = np.random.default_rng(7)
    for n, nval, rs in ((500, 30, [0, 200, 500]), (2000, 300, [0, 0, 1500, 2000]), (64, 3, [0, 64])):
        a = rng.integers(-2, nval, n)
        rs = np.array(rs)
        for calc_not in (True, False):
            M, M_not, nobj = oracle.oc_helper_matrices(a, rs, calc_not)
            Mr, M_not_r, _ = oracle.oc_helper_matrices(a, rs, calc_not, use_ref=True)
            np.testing.assert_array_equal(M, Mr)
            if calc_not:
                np.testing.assert_array_equal(M_not, M_not_r)
        for flt in (True, False):
            got = oracle.max_same_valued_entries_per_row_split(a, rs, flt)
            ref = oracle.max_same_valued_entries_per_row_split(a, rs, flt, use_ref=True)
            np.testing.assert_array_equal(got[0], ref[0])
            assert got[1] == ref[1]
            np.testing.assert_array_equal(got[2], ref[2])
