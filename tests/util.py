"""Comparison helpers shared by the parity tests."""
import numpy as np

# tolerances of the parity contract
DIST_RTOL = 1e-5      # distsq and gradients: relative
TIE_RTOL = 1e-6       # neighbour sets may differ only between candidates this close in distance


def sort_rows(idx, dist):
    """Sort every row by (distance, index), keeping slot 0 (the query itself) first."""
    idx = np.asarray(idx)
    dist = np.asarray(dist)
    key = np.lexsort((idx[:, 1:], dist[:, 1:]), axis=1) if idx.shape[1] > 1 else None
    if key is None:
        return idx.copy(), dist.copy()
    si = np.concatenate([idx[:, :1], np.take_along_axis(idx[:, 1:], key, 1)], axis=1)
    sd = np.concatenate([dist[:, :1], np.take_along_axis(dist[:, 1:], key, 1)], axis=1)
    return si, sd


def assert_knn_equal(idx_a, dist_a, idx_b, dist_b, what=""):
    """Rows agree as sets: sorted distances within DIST_RTOL, and wherever the
    sorted indices differ the two candidates' distances tie within TIE_RTOL
    (relative) - the only freedom an exact kNN has."""
    ia, da = sort_rows(idx_a, dist_a)
    ib, db = sort_rows(idx_b, dist_b)
    assert ia.shape == ib.shape, what
    np.testing.assert_array_equal(ia[:, 0], ib[:, 0], err_msg=what + " slot 0")
    np.testing.assert_allclose(da, db, rtol=DIST_RTOL, atol=0, err_msg=what + " distances")
    np.testing.assert_array_equal(ia < 0, ib < 0, err_msg=what + " padding")
    diff = ia != ib
    if diff.any():
        # a differing slot is legitimate only inside a run of tied distances
        rows = np.unique(np.nonzero(diff)[0])
        for r in rows:
            sa, sb = set(ia[r].tolist()), set(ib[r].tolist())
            only_a, only_b = sa - sb, sb - sa
            kth = max(da[r].max(), db[r].max())
            for j in list(only_a) + list(only_b):
                src_i, src_d = (ia[r], da[r]) if j in only_a else (ib[r], db[r])
                dj = src_d[np.nonzero(src_i == j)[0][0]]
                assert abs(dj - kth) <= TIE_RTOL * max(kth, 1e-30), \
                    "%s row %d: neighbour %d (d2=%g) not a tie at the K-th distance %g" % (what, r, j, dj, kth)
            # same-set rows differing only in order must tie slot by slot
            if not only_a and not only_b:
                cols = np.nonzero(diff[r])[0]
                np.testing.assert_allclose(da[r, cols], db[r, cols], rtol=TIE_RTOL, atol=0)


def check_knn_properties(idx, dist, coords, row_splits, K, ascending=False):
    """Size-independent invariants of a kNN result (used at full benchmark sizes).  ascending: the rows were asked
    for by increasing distance (config.sorted_neighbours, or rows sorted by the caller)."""
    idx = np.asarray(idx)
    dist = np.asarray(dist)
    n = coords.shape[0]
    assert idx.shape == (n, K) and dist.shape == (n, K)
    np.testing.assert_array_equal(idx[:, 0], np.arange(n))
    assert np.all(dist[:, 0] == 0)
    ev = np.searchsorted(np.asarray(row_splits)[1:], np.arange(n), side="right")
    valid = idx >= 0
    nb_ev = np.where(valid, ev[np.clip(idx, 0, n - 1)], ev[:, None])
    assert np.all(nb_ev == ev[:, None]), "neighbour outside the query's event"
    # padding only where the event is smaller than K, and padded distances are 0
    sizes = np.diff(np.asarray(row_splits))[ev]
    np.testing.assert_array_equal(valid.sum(axis=1), np.minimum(sizes, K))
    assert np.all(dist[~valid] == 0)
    # empty slots only at the end of a row
    assert not np.any(~valid[:, :-1] & valid[:, 1:]), "a neighbour after an empty slot"
    if ascending:
        # slots 1.. ascending in distance over the valid part
        d = np.where(valid, dist, np.inf)
        with np.errstate(invalid="ignore"):
            dd = np.diff(d[:, 1:], axis=1)
        assert np.all((dd >= 0) | np.isnan(dd)), "row not sorted by distance"
    # no duplicate neighbours in a row
    s = np.sort(np.where(valid, idx, -np.arange(1, K + 1)[None, :]), axis=1)
    assert np.all(np.diff(s, axis=1) != 0), "duplicate neighbour"
