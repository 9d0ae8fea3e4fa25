"""The benchmark configurations at their full sizes on the GPU: size-independent
invariants, exhaustive-search checks on sampled queries, and full comparisons
with the CPU checker where that takes seconds."""
import numpy as np
import pytest
import torch

from tests.util import assert_knn_equal, check_knn_properties, DIST_RTOL

pytestmark = pytest.mark.gpu


def _brute_rows(coords, rs, queries, K):
    """float32 exhaustive search for the given query rows, same operation order as the kernels."""
    rs = np.asarray(rs)
    out_d = np.zeros((len(queries), K), np.float32)
    out_i = np.full((len(queries), K), -1, np.int64)
    for r, i in enumerate(queries):
        e = np.searchsorted(rs[1:], i, side="right")
        a, b = int(rs[e]), int(rs[e + 1])
        diff = coords[a:b] - coords[i]
        d2 = diff[:, 0] * diff[:, 0]
        for c in range(1, coords.shape[1]):
            d2 = d2 + diff[:, c] * diff[:, c]
        d2[i - a] = -1.0                      # the query itself first
        kk = min(K, b - a)
        part = np.argpartition(d2, kk - 1)[:kk]
        part = part[np.lexsort((part, d2[part]))]
        out_i[r, :kk] = part + a
        out_d[r, :kk] = np.maximum(d2[part], 0.0)
    return out_i, out_d


def _run(w):
    from fastgraphcompute_amd import binned_select_knn
    idx, dist = binned_select_knn(w["K"], torch.from_numpy(w["coords"]).cuda(),
                                  torch.from_numpy(w["row_splits"]).cuda())
    return idx.cpu().numpy(), dist.cpu().numpy()


def _sample_check(w, gi, gd, n_samples, seed):
    rng = np.random.default_rng(seed)
    q = np.sort(rng.choice(w["coords"].shape[0], n_samples, replace=False))
    bi, bd = _brute_rows(w["coords"], w["row_splits"], q, w["K"])
    assert_knn_equal(gi[q], gd[q], bi, bd, "sampled exhaustive search")


def _autograd_gradient_check(oracle, w, seed):
    """The backward that binned_select_knn's autograd runs (the sorted-space gradient kernel, fed by the search's
    own sorted neighbour rows) against the checker's gradient on the same neighbour rows, at full size."""
    from fastgraphcompute_amd import binned_select_knn
    coords = torch.from_numpy(w["coords"]).cuda().requires_grad_(True)
    idx, dist = binned_select_knn(w["K"], coords, torch.from_numpy(w["row_splits"]).cuda())
    up = w.get("grad_distsq")
    if up is None:
        up = np.random.default_rng(seed).standard_normal(tuple(dist.shape)).astype(np.float32)
    dist.backward(torch.from_numpy(up).cuda())
    got = coords.grad.cpu().numpy()
    gi = idx.cpu().numpy()
    exp = oracle.knn_grad(up, gi, w["coords"])
    scale = np.abs(exp).max()
    assert np.abs(got - exp).max() <= DIST_RTOL * scale
    assert np.abs(got.astype(np.float64).sum(axis=0)).max() <= 1e-3 * scale
    return gi, dist.detach().cpu().numpy()


def test_cfg4_full_forward_and_gradient(oracle):
    from fastgraphcompute_amd.workloads import cfg4_zipf_blobs
    from fastgraphcompute_amd.extensions import binned_select_knn_grad
    w = cfg4_zipf_blobs()
    gi, gd = _run(w)
    check_knn_properties(gi, gd, w["coords"], w["row_splits"], w["K"])
    _sample_check(w, gi, gd, 300, 4)
    # densest region: the queries with the smallest K-th distance
    dense = np.argsort(gd.max(axis=1))[:100]
    bi, bd = _brute_rows(w["coords"], w["row_splits"], np.sort(dense), w["K"])
    assert_knn_equal(gi[np.sort(dense)], gd[np.sort(dense)], bi, bd, "densest queries")
    # gradient: full comparison with the checker, plus translation invariance (the gradients sum to zero)
    x = torch.from_numpy(w["coords"]).cuda()
    it = torch.from_numpy(gi).cuda()
    g1 = torch.from_numpy(w["grad_distsq"]).cuda()
    got = binned_select_knn_grad(g1, it, x).cpu().numpy()
    exp = oracle.knn_grad(w["grad_distsq"], gi, w["coords"])
    scale = np.abs(exp).max()
    assert np.abs(got - exp).max() <= DIST_RTOL * scale
    assert np.abs(got.astype(np.float64).sum(axis=0)).max() <= 1e-3 * scale
    # the backward the benchmark times: autograd through the whole call (sorted-space kernel, 16-byte entries)
    ai, ad = _autograd_gradient_check(oracle, w, 0)
    np.testing.assert_array_equal(ai, gi)
    np.testing.assert_array_equal(ad, gd)
    # linearity in the upstream gradient
    g2 = torch.from_numpy(np.random.default_rng(5).standard_normal(g1.shape).astype(np.float32)).cuda()
    lin = binned_select_knn_grad(2.0 * g1 - 0.5 * g2, it, x).cpu().numpy()
    sep = 2.0 * got - 0.5 * binned_select_knn_grad(g2, it, x).cpu().numpy()
    assert np.abs(lin - sep).max() <= 2 * DIST_RTOL * np.abs(sep).max()


def test_cfg2_full_against_checker(oracle):
    from fastgraphcompute_amd.workloads import cfg2_blobs_4events
    w = cfg2_blobs_4events()
    gi, gd = _run(w)
    check_knn_properties(gi, gd, w["coords"], w["row_splits"], w["K"])
    oi, od = oracle.binned_select_knn(w["K"], w["coords"], w["row_splits"], n_threads=16)
    assert_knn_equal(gi, gd, oi, od)
    _autograd_gradient_check(oracle, w, 12)      # D = 4: the wide-entry variant of the sorted-space kernel


def test_cfg5_full_sampled(oracle):
    from fastgraphcompute_amd.workloads import cfg5_many_events_d8
    w = cfg5_many_events_d8()
    gi, gd = _run(w)
    check_knn_properties(gi, gd, w["coords"], w["row_splits"], w["K"])
    _sample_check(w, gi, gd, 400, 6)
    # D = 8, K = 100: the wide-entry gradient kernel where nearly every pair leaves the on-chip table
    # (both overflow paths), against the checker on all 50 M pairs
    _autograd_gradient_check(oracle, w, 15)


def test_cfg3_gravnet_full(oracle):
    from fastgraphcompute_amd.workloads import cfg3_gravnet
    from fastgraphcompute_amd.gnn_ops import GravNetOp, gravnet_aggregate
    w = cfg3_gravnet()
    torch.manual_seed(w["weight_seed"])
    op = GravNetOp(w["in_channels"], w["out_channels"], w["space_dimensions"], w["propagate_dimensions"], w["K"]).cuda()
    x = torch.from_numpy(w["x"]).cuda().requires_grad_(True)
    rs = torch.from_numpy(w["row_splits"]).cuda()
    out, idx, dsq, space = op(x, rs)
    (out * torch.from_numpy(w["out_grad"]).cuda()).sum().backward()
    n = w["x"].shape[0]
    assert out.shape == (n, 64) and idx.shape == (n, 40) and space.shape == (n, 4)
    assert torch.isfinite(out).all() and torch.isfinite(x.grad).all()
    for p in op.parameters():
        assert p.grad is not None and torch.isfinite(p.grad).all()
    ih, dh, sh = idx.cpu().numpy(), dsq.detach().cpu().numpy(), space.detach().cpu().numpy()
    check_knn_properties(ih, dh, sh, w["row_splits"], 40)
    q = np.sort(np.random.default_rng(7).choice(n, 200, replace=False))
    bi, bd = _brute_rows(sh, w["row_splits"], q, 40)
    assert_knn_equal(ih[q], dh[q], bi, bd, "GravNet learned space")
    # the fused aggregation on the full tensors against the checker's kernel
    prop = op.propagate_transformations(x).detach()
    fm, fx = gravnet_aggregate(idx, dsq.detach(), prop)
    cm, cx, _ = oracle.gravnet_aggregate(ih, dh, prop.cpu().numpy())
    assert np.abs(fm.cpu().numpy() - cm).max() <= DIST_RTOL * np.abs(cm).max()
    assert np.abs(fx.cpu().numpy() - cx).max() <= DIST_RTOL * np.abs(cx).max()


def test_cfg3_gravnet_backward_against_checker(oracle):
    """x.grad and the parameter gradients of the cfg3 layer against autograd through the checker's CPU layer
    (torch Linear, checker kNN and gradient, torch aggregation), on the first 2 x 12 000 points of the cfg3
    input with the cfg3 weights.  The learned coordinates differ in the last bits between the GPU and CPU
    products, so the comparison is at 2e-3 of each gradient's largest entry."""
    from fastgraphcompute_amd.workloads import cfg3_gravnet
    from fastgraphcompute_amd.gnn_ops import GravNetOp
    w = cfg3_gravnet()
    per = 12000
    half = w["x"].shape[0] // 2
    sel = np.concatenate([np.arange(per), half + np.arange(per)])
    x_h = torch.from_numpy(w["x"][sel].copy())
    g_h = torch.from_numpy(w["out_grad"][sel].copy())
    rs = np.array([0, per, 2 * per], dtype=np.int32)
    torch.manual_seed(w["weight_seed"])
    op = GravNetOp(w["in_channels"], w["out_channels"], w["space_dimensions"], w["propagate_dimensions"], w["K"])
    wt = {kk: v.detach().clone().requires_grad_(True) for kk, v in op.state_dict().items()}
    xr = x_h.clone().requires_grad_(True)
    out_r, idx_r, d_r, _ = oracle.gravnet_forward_torch(xr, rs, wt, w["K"], n_threads=16)
    (out_r * g_h).sum().backward()
    op = op.cuda()
    xg = x_h.cuda().requires_grad_(True)
    out, idx, dsq, _ = op(xg, torch.from_numpy(rs).cuda())
    (out * g_h.cuda()).sum().backward()

    def close(a, b, what, scale=None):
        a, b = a.detach().cpu().double(), b.detach().double()
        assert float((a - b).abs().max()) <= 2e-3 * (scale or float(b.abs().max())), what

    close(out, out_r, "out")
    close(torch.sort(dsq, 1).values, torch.sort(d_r, 1).values, "distsq")
    close(xg.grad, xr.grad, "x.grad")
    for name, p in op.named_parameters():
        # a bias gradient is the plain sum of the rows whose products with x give the weight gradient; for the
        # coordinate projection that sum is zero analytically (the distances do not change under a shift of
        # all points), so it is compared on the scale of its layer's weight gradient
        scale = float(wt[name.replace(".bias", ".weight")].grad.abs().max()) if name.endswith(".bias") else None
        close(p.grad, wt[name].grad, name, scale)


def test_more_than_2_31_output_entries():
    """36 M points with K = 64: 2.3e9 entries per output array, past every 32-bit offset.  Sampled exhaustive
    search on the device (first and last rows of each event included) and, for the gradient, translation
    invariance: the coordinate gradients of all points sum to zero."""
    from fastgraphcompute_amd import binned_select_knn
    free, _ = torch.cuda.mem_get_info()
    if free < 80 * 2 ** 30:
        pytest.skip("needs about 60 GB of device memory")
    n, K = 36_000_000, 64
    torch.manual_seed(7)
    coords = torch.rand((n, 3), device="cuda").requires_grad_(True)
    cut = n // 3
    rs = torch.tensor([0, cut, n], dtype=torch.int64, device="cuda")
    idx, dist = binned_select_knn(K, coords, rs)
    assert int((idx < 0).sum().item()) == 0
    c = coords.detach()
    g = torch.Generator().manual_seed(3)
    sample = torch.cat([torch.tensor([0, 1, cut - 1, cut, n - 2, n - 1]), torch.randint(0, n, (58,), generator=g)])
    for qi in sample.tolist():
        lo, hi = (0, cut) if qi < cut else (cut, n)
        d = ((c[lo:hi] - c[qi]) ** 2).sum(1)
        ref_d = torch.sort(torch.topk(d, K, largest=False).values).values
        got_d = torch.sort(dist[qi].detach()).values
        assert torch.allclose(got_d, ref_d, rtol=DIST_RTOL, atol=1e-12), qi
        row = idx[qi]
        assert row[0].item() == qi and row.min().item() >= lo and row.max().item() < hi, qi
        assert torch.allclose(((c[row] - c[qi]) ** 2).sum(1), dist[qi].detach(), rtol=DIST_RTOL, atol=1e-12), qi
    del d
    gd = torch.randn((n, K), device="cuda")
    (dist * gd).sum().backward()
    gr = coords.grad.double()
    assert (gr.sum(0).abs() / gr.abs().sum(0)).max().item() < 1e-6
    assert bool(coords.grad[-1000:].abs().sum(1).gt(0).all())


def _elementwise_error(got, exact64, abs_sum64):
    """Error of every element in units of what float32 summation can cost it: |got - exact| divided by
    (sum of |terms| * 2^-24).  A sum of t terms in any order stays below t such units (below about sqrt(t) typically),
    however much the terms cancel.  Returns (largest, 99.9th percentile)."""
    unit = abs_sum64 * 2.0 ** -24
    err = (got.double() - exact64).abs()
    assert bool((err[unit == 0] == 0).all()), "an element without terms must be exactly zero"
    ratio = (err / unit.clamp_min(1e-300))[unit > 0]
    return float(ratio.max()), float(torch.quantile(ratio[torch.randperm(ratio.numel(), device=ratio.device)[:4_000_000]], 0.999))


def test_cfg4_gradient_elementwise_error():
    """north_star asks for gradients 'within 1e-5 relative'.  With float atomics and upstream gradients of both signs
    an element of the gradient can be the small remainder of large terms, so the comparisons above are normwise
    (1e-5 of the gradient's largest entry).  This test adds the elementwise statement that can be made: every element
    of the timed backward (autograd path, sorted-space kernel) lies within a small multiple of the float32 summation
    unit of ITS OWN terms around the float64 value."""
    from fastgraphcompute_amd import binned_select_knn
    from fastgraphcompute_amd.workloads import cfg4_zipf_blobs
    w = cfg4_zipf_blobs()
    K = w["K"]
    x = torch.from_numpy(w["coords"]).cuda().requires_grad_(True)
    idx, dist = binned_select_knn(K, x, torch.from_numpy(w["row_splits"]).cuda())
    g = torch.from_numpy(w["grad_distsq"]).cuda()
    dist.backward(g)
    got = x.grad
    n, D = w["coords"].shape
    # float64 gradient and the sum of the absolute terms per element (binned_select_knn_grad_cpu.cpp:6-93):
    # pair (i, k) with neighbour j adds 2 g (x_i - x_j) to row i and subtracts it from row j
    xd = x.detach().double()
    exact = torch.zeros((n, D), dtype=torch.float64, device="cuda")
    abs_sum = torch.zeros((n, D), dtype=torch.float64, device="cuda")
    for k0 in range(0, K, 8):                      # 8 slots at a time: 8 M pairs x 3 doubles
        j = idx[:, k0:k0 + 8]
        valid = (j >= 0).unsqueeze(-1)
        t = 2.0 * g[:, k0:k0 + 8].double().unsqueeze(-1) * (xd.unsqueeze(1) - xd[j.clamp_min(0)]) * valid
        exact += t.sum(1)
        abs_sum += t.abs().sum(1)
        exact.index_add_(0, j.clamp_min(0).reshape(-1), -t.reshape(-1, D))
        abs_sum.index_add_(0, j.clamp_min(0).reshape(-1), t.abs().reshape(-1, D))
    worst, p999 = _elementwise_error(got, exact, abs_sum)
    print("cfg4 kNN gradient: elementwise error in float32 summation units: max %.1f, 99.9th percentile %.2f" % (worst, p999))
    assert p999 <= 4.0 and worst <= 16.0
    # and the normwise statement, against float64 this time
    assert float((got.double() - exact).abs().max()) <= DIST_RTOL * float(exact.abs().max())


def test_cfg3_aggregation_backward_full(oracle):
    """Both aggregation backward kernels on the FULL cfg3 tensors (300 000 rows, K = 40, 32 features; neighbour rows,
    distances and features as the GPU layer produces them, so no GEMM differences enter): the tile kernel that
    GravNetOp's backward runs (fgc_gravnet_aggregate_bwd_sorted_f32: 24-bit row arithmetic, 32-bit byte offsets and
    1024 buckets only a large input exercises) against the per-pair kernel, both against float64 sums elementwise, and
    against autograd through the checker's torch composition of gnn_ops.py:90-102 on one whole event."""
    import ctypes
    from fastgraphcompute_amd import _lib, _ops
    from fastgraphcompute_amd.workloads import cfg3_gravnet
    from fastgraphcompute_amd.gnn_ops import GravNetOp
    L = _lib.lib()
    w = cfg3_gravnet()
    K, P, S = w["K"], w["propagate_dimensions"], w["space_dimensions"]
    torch.manual_seed(w["weight_seed"])
    op = GravNetOp(w["in_channels"], w["out_channels"], S, P, K).cuda()
    x = torch.from_numpy(w["x"]).cuda()
    rs = torch.from_numpy(w["row_splits"]).cuda()
    with torch.no_grad():
        space = op.space_transformations(x).contiguous()
        feat = op.propagate_transformations(x).contiguous()
    n = x.shape[0]
    idx, dist, nbr, order = _ops._knn_forward(space, S, rs, K, None, None, 3, False, True)
    fm, fx = torch.empty((n, P), device="cuda"), torch.empty((n, P), device="cuda")
    am = torch.empty((n, P), dtype=torch.int32, device="cuda")
    st = _lib.stream_ptr()
    _lib.check(L.fgc_gravnet_aggregate_fwd_f32(_lib.ptr(idx), _lib.ptr(dist), _lib.ptr(feat), _lib.ptr(fm), _lib.ptr(fx),
                                               _lib.ptr(am), n, K, P, st))
    g = torch.from_numpy(np.random.default_rng(31).standard_normal((n, 2 * P)).astype(np.float32)).cuda()
    out = {}
    for name in ("pairs", "tiles"):
        gf = torch.zeros((n, P), device="cuda")
        gd = torch.full((n, K), 7.0, device="cuda")
        status = torch.zeros(4, dtype=torch.int32, device="cuda")
        if name == "pairs":
            rc = L.fgc_gravnet_aggregate_bwd_ld_f32(_lib.ptr(idx), _lib.ptr(dist), _lib.ptr(feat), P, n, _lib.ptr(am),
                                                    _lib.ptr(g), ctypes.c_void_p(g.data_ptr() + 4 * P), 2 * P,
                                                    _lib.ptr(gf), P, _lib.ptr(gd), n, K, P, _lib.ptr(status), st)
        else:
            rc = L.fgc_gravnet_aggregate_bwd_sorted_f32(_lib.ptr(nbr), _lib.ptr(order), _lib.ptr(dist), _lib.ptr(feat),
                                                        P, _lib.ptr(am), _lib.ptr(g),
                                                        ctypes.c_void_p(g.data_ptr() + 4 * P), 2 * P, _lib.ptr(gf), P,
                                                        _lib.ptr(gd), n, K, P, _lib.ptr(status), st)
        _lib.check(rc)
        torch.cuda.synchronize()
        assert int(status[0]) == 0
        out[name] = (gf, gd)
    assert torch.equal(out["tiles"][1], out["pairs"][1]), "grad_distsq: same operations in the same order"
    scale = float(out["pairs"][0].abs().max())
    assert float((out["tiles"][0] - out["pairs"][0]).abs().max()) <= DIST_RTOL * scale
    # float64 feature gradient and the sum of its absolute terms: pair (i, k) adds w (g_mean / K + [argmax == k] g_max)
    # to the row of its neighbour (gnn_ops.py:90-102)
    exact = torch.zeros((n, P), dtype=torch.float64, device="cuda")
    abs_sum = torch.zeros((n, P), dtype=torch.float64, device="cuda")
    gm, gx = g[:, :P].double(), g[:, P:].double()
    for k in range(K):
        j = idx[:, k]
        wk = torch.exp(-10.0 * dist[:, k].double()) * (j >= 0)
        c = wk.unsqueeze(1) * (gm / K + gx * (am == k))
        exact.index_add_(0, j.clamp_min(0), c)
        abs_sum.index_add_(0, j.clamp_min(0), c.abs())
    for name in ("tiles", "pairs"):
        worst, p999 = _elementwise_error(out[name][0], exact, abs_sum)
        # the weights are float32 expf results (2 units of relative error each): allow for them on top of the sums
        print("cfg3 aggregation backward (%s): elementwise error in float32 summation units: max %.1f, "
              "99.9th percentile %.2f" % (name, worst, p999))
        assert p999 <= 8.0 and worst <= 48.0
        assert float((out[name][0].double() - exact).abs().max()) <= DIST_RTOL * float(exact.abs().max())
    # one whole event (150 000 rows) against autograd through the checker's composition on the CPU
    a, b = int(w["row_splits"][0]), int(w["row_splits"][1])
    it = (idx[a:b] - a).cpu()
    it[idx[a:b].cpu() < 0] = -1
    dt = dist[a:b].cpu().requires_grad_(True)
    ft = feat[a:b].cpu().requires_grad_(True)
    tm, tx = oracle.gravnet_aggregate_torch(it, dt, ft)
    ((tm * g[a:b, :P].cpu()).sum() + (tx * g[a:b, P:].cpu()).sum()).backward()
    for name in ("tiles", "pairs"):
        gf, gd = out[name]
        assert float((gf[a:b].cpu() - ft.grad).abs().max()) <= DIST_RTOL * float(ft.grad.abs().max()), name
        assert float((gd[a:b].cpu() - dt.grad).abs().max()) <= DIST_RTOL * float(dt.grad.abs().max()), name
