"""CPU tests pinning the checker's GravNet aggregation (oracle.gravnet_aggregate, gravnet_aggregate_torch,
gravnet_forward_torch) by what the mathematics of fastgraphcompute/gnn_ops.py:90-102 fixes, not by another
restatement: hand-computed known answers (tests/golden/gravnet_known_answers.json), closed-form special
cases that reduce to numpy.take + mean / max, a float64 definition written as plain loops, and finite
differences of that definition for the gradients.  Each check names the misreading it would catch."""
import json
import os

import numpy as np
import pytest
import torch

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def known():
    with open(os.path.join(GOLDEN, "gravnet_known_answers.json")) as f:
        return json.load(f)


def layer_weights():
    """Hand-set weights of the 'layer' case: x = [cx, cy, f0, f1]; space copies (cx, cy), propagate copies
    (f0, f1), the output layer is the identity on cat[x, fmean, fmax]."""
    sw = torch.zeros(2, 4)
    sw[0, 0] = sw[1, 1] = 1.0
    pw = torch.zeros(2, 4)
    pw[0, 2] = pw[1, 3] = 1.0
    return {"space_transformations.weight": sw, "space_transformations.bias": torch.zeros(2),
            "propagate_transformations.weight": pw, "propagate_transformations.bias": torch.zeros(2),
            "output_transformations.0.weight": torch.eye(8), "output_transformations.0.bias": torch.zeros(8)}


def definition_f64(idx, distsq, feat):
    """The aggregation as its definition reads, in float64 and plain loops (small inputs only)."""
    n, K = idx.shape
    P = feat.shape[1]
    fmean = np.zeros((n, P))
    fmax = np.zeros((n, P))
    for i in range(n):
        for p in range(P):
            vals = []
            for k in range(K):
                f = 0.0 if idx[i, k] == -1 else float(feat[idx[i, k], p])
                vals.append(f * np.exp(-10.0 * float(distsq[i, k])))
            fmean[i, p] = sum(vals) / K
            fmax[i, p] = max(vals)
    return fmean, fmax


# ------------------------------------------------------------------ hand-computed known answers
def test_weights_of_the_known_answers_are_what_the_file_says():
    # the table's d2 values are ln(2^j)/10: exp(-10 d2) must be the stated powers of 1/2
    a = known()["aggregate"]
    np.testing.assert_allclose(np.exp(-10.0 * np.array(a["distsq"])), np.array(a["weights"]), rtol=1e-14)
    # a misread exponent (-10 d instead of -10 d2, or another constant) does not give them
    assert abs(np.exp(-10.0 * np.sqrt(a["distsq"][0][1])) - 0.5) > 0.4
    assert abs(np.exp(-1.0 * a["distsq"][0][1]) - 0.5) > 0.4


def test_c_kernel_known_answers(oracle):
    a = known()["aggregate"]
    idx, d, f = np.array(a["idx"]), np.array(a["distsq"], np.float32), np.array(a["feat"], np.float32)
    fmean, fmax, am = oracle.gravnet_aggregate(idx, d, f)
    np.testing.assert_allclose(fmean, a["fmean"], rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(fmax, a["fmax"], rtol=1e-6, atol=1e-7)
    np.testing.assert_array_equal(am, a["argmax"])


def test_torch_composition_known_answers_forward_and_gradients(oracle):
    a = known()["aggregate"]
    idx = torch.tensor(a["idx"])
    d = torch.tensor(a["distsq"], dtype=torch.float32, requires_grad=True)
    f = torch.tensor(a["feat"], dtype=torch.float32, requires_grad=True)
    fmean, fmax = oracle.gravnet_aggregate_torch(idx, d, f)
    np.testing.assert_allclose(fmean.detach().numpy(), a["fmean"], rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(fmax.detach().numpy(), a["fmax"], rtol=1e-6, atol=1e-7)
    ((fmean * torch.tensor(a["grad_fmean"])).sum() + (fmax * torch.tensor(a["grad_fmax"])).sum()).backward()
    np.testing.assert_allclose(f.grad.numpy(), a["grad_feat"], rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(d.grad.numpy(), a["grad_distsq"], rtol=1e-5, atol=1e-5)


def test_layer_known_answers(oracle):
    c = known()["layer"]
    x = torch.tensor(c["x"], dtype=torch.float32)
    out, idx, dsq, space = oracle.gravnet_forward_torch(x, np.array(c["row_splits"]), layer_weights(), c["k"],
                                                        n_threads=1)
    idx, dsq = idx.numpy(), dsq.numpy()
    np.testing.assert_array_equal(idx[:, 0], np.arange(4))
    np.testing.assert_array_equal(np.sort(idx, 1), np.sort(np.array(c["neighbour_sets"]), 1))
    np.testing.assert_allclose(np.sort(dsq, 1), c["distsq_sorted"], rtol=1e-5, atol=1e-8)
    np.testing.assert_array_equal(space.numpy(), x[:, :2].numpy())
    expect = np.maximum(np.concatenate([np.array(c["x"]), np.array(c["fmean"]), np.array(c["fmax"])], 1), 0.0)
    np.testing.assert_allclose(out.detach().numpy(), expect, rtol=1e-5, atol=1e-6)


# ------------------------------------------------------------------ closed forms
def _random_case(seed, n=40, K=6, P=5, pad=True):
    rng = np.random.default_rng(seed)
    idx = rng.integers(0, n, (n, K))
    if pad:
        idx[rng.random((n, K)) < 0.25] = -1
        idx[3] = -1                                     # a row of padding only
    d = (rng.random((n, K)) * 0.3).astype(np.float32)
    f = rng.standard_normal((n, P)).astype(np.float32)
    return idx, d, f


def _both(oracle, idx, d, f):
    m1, x1, _ = oracle.gravnet_aggregate(idx, d, f)
    m2, x2 = oracle.gravnet_aggregate_torch(torch.from_numpy(idx), torch.from_numpy(d), torch.from_numpy(f))
    return (m1, x1), (m2.numpy(), x2.numpy())


def test_zero_distance_reduces_to_plain_mean_and_max(oracle):
    # all d2 = 0 and no padding: w = 1, so the result is numpy.take + mean / max over the slot axis
    idx, d, f = _random_case(1, pad=False)
    d[:] = 0
    g = np.take(f, idx, axis=0)                          # [n, K, P]
    for m, x in _both(oracle, idx, d, f):
        np.testing.assert_allclose(m, g.mean(1), rtol=1e-6, atol=1e-6)
        np.testing.assert_array_equal(x, g.max(1))


def test_k1_self_neighbour_returns_own_features(oracle):
    # K = 1, the only neighbour is the point itself at distance 0: fmean = fmax = own feature
    n, P = 30, 4
    f = np.random.default_rng(2).standard_normal((n, P)).astype(np.float32)
    idx = np.arange(n)[:, None]
    d = np.zeros((n, 1), np.float32)
    for m, x in _both(oracle, idx, d, f):
        np.testing.assert_array_equal(m, f)
        np.testing.assert_array_equal(x, f)


def test_uniform_weight_scales_linearly(oracle):
    # one common d2 for every slot: the result is exp(-10 d2) times the zero-distance result
    idx, d, f = _random_case(3, pad=False)
    d0 = np.zeros_like(d)
    d1 = np.full_like(d, 0.123)
    (m0, x0), _ = _both(oracle, idx, d0, f)
    s = np.exp(-1.23)
    fpos = np.abs(f)                                     # a positive scale commutes with max
    (mp0, xp0), _ = _both(oracle, idx, d0, fpos)
    for m, x in _both(oracle, idx, d1, fpos):
        np.testing.assert_allclose(m, s * mp0, rtol=2e-6)
        np.testing.assert_allclose(x, s * xp0, rtol=2e-6)
    for m, _x in _both(oracle, idx, d1, f):
        np.testing.assert_allclose(m, s * m0, rtol=1e-5, atol=1e-6)


def test_padding_counts_as_zero_and_mean_divides_by_k(oracle):
    # one valid neighbour with a negative feature among K slots: mean = f / K (not f / 1), max = 0 (the padding)
    K = 4
    f = np.array([[-2.0], [5.0]], np.float32)
    idx = np.array([[0, -1, -1, -1], [1, -1, -1, -1]])
    d = np.zeros((2, K), np.float32)
    for m, x in _both(oracle, idx, d, f):
        np.testing.assert_array_equal(m, [[-0.5], [1.25]])
        np.testing.assert_array_equal(x, [[0.0], [5.0]])


# ------------------------------------------------------------------ float64 definition and its finite differences
@pytest.mark.parametrize("seed", [11, 12])
def test_against_float64_definition(oracle, seed):
    idx, d, f = _random_case(seed, n=50, K=7, P=3)
    em, ex = definition_f64(idx, d, f)
    for m, x in _both(oracle, idx, d, f):
        np.testing.assert_allclose(m, em, rtol=1e-5, atol=1e-6)
        np.testing.assert_allclose(x, ex, rtol=1e-5, atol=1e-6)


def test_autograd_of_torch_composition_matches_finite_differences(oracle):
    # central differences of the float64 definition; the case has no ties between slot values, so max is smooth
    idx, d, f = _random_case(21, n=12, K=4, P=3)
    rng = np.random.default_rng(22)
    um, ux = rng.standard_normal((12, 3)), rng.standard_normal((12, 3))

    def loss(dd, ff):
        m, x = definition_f64(idx, dd, ff)
        return (m * um).sum() + (x * ux).sum()

    d64, f64 = d.astype(np.float64), f.astype(np.float64)
    h = 1e-6
    gd = np.zeros_like(d64)
    for i in range(d64.shape[0]):
        for k in range(d64.shape[1]):
            dp, dm = d64.copy(), d64.copy()
            dp[i, k] += h
            dm[i, k] -= h
            gd[i, k] = (loss(dp, f64) - loss(dm, f64)) / (2 * h)
    gf = np.zeros_like(f64)
    for i in range(f64.shape[0]):
        for p in range(f64.shape[1]):
            fp, fm = f64.copy(), f64.copy()
            fp[i, p] += h
            fm[i, p] -= h
            gf[i, p] = (loss(d64, fp) - loss(d64, fm)) / (2 * h)
    dt = torch.from_numpy(d64).requires_grad_(True)
    ft = torch.from_numpy(f64).requires_grad_(True)
    m, x = oracle.gravnet_aggregate_torch(torch.from_numpy(idx), dt, ft)
    ((m * torch.from_numpy(um)).sum() + (x * torch.from_numpy(ux)).sum()).backward()
    np.testing.assert_allclose(dt.grad.numpy(), gd, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(ft.grad.numpy(), gf, rtol=1e-5, atol=1e-6)


def test_layer_gradient_matches_finite_differences(oracle):
    # d(loss)/dx of the whole layer (projections, kNN distances, aggregation, output layer) against central
    # differences of a float64 evaluation built from the definition above and a brute-force neighbour search;
    # the neighbour sets are stable under the step (well-separated random points)
    rng = np.random.default_rng(31)
    n, C, S, P, k, O_ = 14, 5, 2, 3, 4, 6
    rs = np.array([0, 8, n])
    x = rng.standard_normal((n, C))
    W = {"space_transformations.weight": rng.standard_normal((S, C)) * 0.3,
         "space_transformations.bias": rng.standard_normal(S) * 0.1,
         "propagate_transformations.weight": rng.standard_normal((P, C)),
         "propagate_transformations.bias": rng.standard_normal(P),
         "output_transformations.0.weight": rng.standard_normal((O_, C + 2 * P)),
         "output_transformations.0.bias": rng.standard_normal(O_)}
    G = rng.standard_normal((n, O_))

    def forward64(xx):
        space = xx @ W["space_transformations.weight"].T + W["space_transformations.bias"]
        prop = xx @ W["propagate_transformations.weight"].T + W["propagate_transformations.bias"]
        idx = np.full((n, k), -1)
        dsq = np.zeros((n, k))
        for e in range(len(rs) - 1):
            lo, hi = rs[e], rs[e + 1]
            for i in range(lo, hi):
                dd = ((space[lo:hi] - space[i]) ** 2).sum(1)
                dd[i - lo] = -1.0                         # the point itself first
                o = np.argsort(dd, kind="stable")[:k]
                idx[i, :len(o)] = o + lo
                dsq[i, :len(o)] = np.maximum(dd[o], 0.0)
        m, mx = definition_f64(idx, dsq, prop)
        out = np.maximum(np.concatenate([xx, m, mx], 1) @ W["output_transformations.0.weight"].T
                         + W["output_transformations.0.bias"], 0.0)
        return (out * G).sum(), idx

    base, idx0 = forward64(x)
    h = 1e-6
    g = np.zeros_like(x)
    for i in range(n):
        for c in range(C):
            xp, xm = x.copy(), x.copy()
            xp[i, c] += h
            xm[i, c] -= h
            lp, ip = forward64(xp)
            lm, im = forward64(xm)
            assert np.array_equal(np.sort(ip, 1), np.sort(idx0, 1)) and np.array_equal(np.sort(im, 1), np.sort(idx0, 1))
            g[i, c] = (lp - lm) / (2 * h)
    xt = torch.from_numpy(x.astype(np.float32)).requires_grad_(True)
    wt = {kk: torch.from_numpy(v.astype(np.float32)) for kk, v in W.items()}
    out, idx, dsq, _ = oracle.gravnet_forward_torch(xt, rs, wt, k, n_threads=1)
    np.testing.assert_array_equal(np.sort(idx.numpy(), 1), np.sort(idx0, 1))
    (out * torch.from_numpy(G.astype(np.float32))).sum().backward()
    assert abs(float((out.detach().double() * torch.from_numpy(G)).sum()) - base) <= 1e-4 * max(1.0, abs(base))
    np.testing.assert_allclose(xt.grad.numpy(), g, rtol=2e-3, atol=2e-3 * np.abs(g).max())


# ------------------------------------------------------------------ the checks do catch the plausible misreadings
@pytest.mark.parametrize("mutation", ["exponent_on_d", "mean_over_valid", "nonzero_default", "last_max"])
def test_known_answers_reject_misreadings(mutation):
    """A deliberately wrong aggregation must fail the known answers (guards the table, not the checker)."""
    a = known()["aggregate"]
    idx, d, f = np.array(a["idx"]), np.array(a["distsq"]), np.array(a["feat"])
    n, K = idx.shape
    P = f.shape[1]
    fmean, fmax, am = np.zeros((n, P)), np.zeros((n, P)), np.zeros((n, P), int)
    for i in range(n):
        for p in range(P):
            vals = []
            for k in range(K):
                w = np.exp(-10.0 * (np.sqrt(d[i, k]) if mutation == "exponent_on_d" else d[i, k]))
                dflt = 1.0 if mutation == "nonzero_default" else 0.0
                vals.append((dflt if idx[i, k] == -1 else f[idx[i, k], p]) * w)
            nv = max(1, int((idx[i] != -1).sum()))
            fmean[i, p] = sum(vals) / (nv if mutation == "mean_over_valid" else K)
            fmax[i, p] = max(vals)
            am[i, p] = (K - 1 - int(np.argmax(vals[::-1]))) if mutation == "last_max" else int(np.argmax(vals))
    ok = (np.allclose(fmean, a["fmean"], rtol=1e-6) and np.allclose(fmax, a["fmax"], rtol=1e-6)
          and np.array_equal(am, a["argmax"]))
    assert not ok
