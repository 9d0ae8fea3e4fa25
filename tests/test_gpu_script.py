"""TorchScript compatibility, as the reference's own tests check it
(tests/test_binned_select_knn.py:242-320, tests/test_bin_by_coordinates.py:84-109,
tests/test_gnn_ops.py:29-85,115-149): scripted == eager == saved-and-loaded."""
import io
from typing import Optional, Tuple

import pytest
import torch

from fastgraphcompute_amd import bin_by_coordinates, binned_select_knn

pytestmark = pytest.mark.gpu


class KnnModule(torch.nn.Module):
    def forward(self, K: int, coordinates: torch.Tensor, row_splits: torch.Tensor,
                direction: Optional[torch.Tensor] = None,
                n_bins: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
        return binned_select_knn(K, coordinates, row_splits, direction=direction, n_bins=n_bins)


class BinModule(torch.nn.Module):
    def forward(self, coordinates: torch.Tensor, row_splits: torch.Tensor, bin_width: torch.Tensor,
                nbins: torch.Tensor, return_all: bool
                ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
        return bin_by_coordinates(coordinates, row_splits, bin_width, nbins, return_all)


def _roundtrip(m):
    buf = io.BytesIO()
    torch.jit.save(m, buf)
    buf.seek(0)
    return torch.jit.load(buf)


def test_knn_module_scripts():
    import fastgraphcompute_amd  # noqa: F401
    torch.manual_seed(0)
    coords = torch.randn(100, 3, device="cuda")
    rs = torch.tensor([0, 50, 100], dtype=torch.int64, device="cuda")
    nb = torch.tensor(4, dtype=torch.int64, device="cuda")
    m = KnnModule().cuda()
    sm = torch.jit.script(m)
    lm = _roundtrip(sm)
    with torch.no_grad():
        ref = m(8, coords, rs, None, nb)
        for other in (sm(8, coords, rs, None, nb), lm(8, coords, rs, None, nb)):
            assert other[0].shape == (100, 8) and other[1].shape == (100, 8)
            assert torch.equal(ref[0], other[0]) and torch.equal(ref[1], other[1])
    # gradients flow through the scripted module
    c = coords.clone().requires_grad_(True)
    sm(8, c, rs, None, nb)[1].sum().backward()
    assert c.grad is not None and torch.isfinite(c.grad).all() and c.grad.abs().sum() > 0


def test_bin_by_coordinates_module_scripts():
    coords = torch.tensor([[0.1, 0.1], [2.5, 2.5], [4.9, 4.9]], device="cuda")
    rs = torch.tensor([0, 3], device="cuda")
    bw = torch.tensor([0.5], device="cuda")
    nb = torch.tensor([10, 10], device="cuda")
    m = BinModule()
    sm = torch.jit.script(m)
    with torch.no_grad():
        a = m(coords, rs, bw, nb, True)
        b = sm(coords, rs, bw, nb, True)
    assert len(a) == len(b) == 5
    for x, y in zip(a, b):
        assert x.shape == y.shape and torch.equal(x, y)


@pytest.mark.parametrize("C,P,k,S", [(8, 8, 8, 3), (12, 16, 32, 4)])
def test_gravnet_scripts_traces_and_reloads(C, P, k, S):
    from fastgraphcompute_amd.gnn_ops import GravNetOp
    torch.manual_seed(1)
    op = GravNetOp(C, 20, S, P, k).cuda().eval()
    x = torch.randn(100, C, device="cuda")
    rs = torch.tensor([0, 50, 80, 100], dtype=torch.int32, device="cuda")
    sop = torch.jit.script(op)
    lop = _roundtrip(sop)
    top = torch.jit.trace(op, (x, rs))
    with torch.no_grad():
        ref = op(x, rs)
        for other in (sop(x, rs), lop(x, rs), top(x, rs)):
            for a, b in zip(ref, other):
                assert a.shape == b.shape
                assert torch.allclose(a.float(), b.float(), atol=1e-6)
    xg = x.clone().requires_grad_(True)
    sop(xg, rs)[0].sum().backward()
    assert torch.isfinite(xg.grad).all()


def test_index_replacer_and_select_with_default_script():
    from fastgraphcompute_amd import index_replacer, select_with_default

    @torch.jit.script
    def both(idx: torch.Tensor, repl: torch.Tensor, feat: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
        return index_replacer(idx, repl), select_with_default(idx, feat, -1.5)

    idx = torch.randint(-1, 30, (40, 6), device="cuda")
    repl = torch.randperm(30, device="cuda")
    feat = torch.randn(30, 5, device="cuda", requires_grad=True)
    r, s = both(idx, repl, feat)
    assert torch.equal(r, torch.where(idx < 0, idx, repl[idx.clamp(min=0)]))
    exp = torch.where((idx == -1).unsqueeze(-1), torch.full((), -1.5, device="cuda"), feat[idx.clamp(min=0)])
    assert torch.equal(s, exp)
    # select_with_default is differentiable wrt the features, like the reference's tensor-op version
    g = torch.randn_like(s)
    (s * g).sum().backward()
    ga = feat.grad.clone()
    feat.grad = None
    (exp * g).sum().backward()
    assert torch.allclose(ga, feat.grad, atol=1e-6)
