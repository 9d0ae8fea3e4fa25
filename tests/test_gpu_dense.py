"""Weight-gradient kernel and the dense op of GravNetOp against float64 torch."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n,O,I", [(1, 1, 1), (7, 4, 64), (1000, 36, 64), (5001, 64, 128), (20000, 128, 128),
                                   (333, 33, 65), (4096, 10, 200), (64, 130, 3), (300000, 36, 64)])
def test_wgrad_against_float64(n, O, I):
    from fastgraphcompute_amd._ops import linear_wgrad
    g = torch.Generator(device="cpu").manual_seed(n + O + I)
    dy = torch.randn(n, O, generator=g)
    x = torch.randn(n, I, generator=g)
    gw, gb = linear_wgrad(dy.cuda(), x.cuda(), True)
    ref_w = dy.double().t() @ x.double()
    ref_b = dy.double().sum(0)
    # float32 accumulation over n terms: error relative to the sum of magnitudes, not to the (cancelling) sum
    scale_w = (dy.double().abs().t() @ x.double().abs()).clamp_min(1e-30)
    scale_b = dy.double().abs().sum(0).clamp_min(1e-30)
    assert float(((gw.cpu().double() - ref_w).abs() / scale_w).max()) < 1e-6
    assert float(((gb.cpu().double() - ref_b).abs() / scale_b).max()) < 1e-6
    gw2, gb2 = linear_wgrad(dy.cuda(), x.cuda(), False)
    assert gb2 is None and torch.equal(gw2, gw)            # fixed summation order: bit-reproducible


def test_wgrad_empty():
    from fastgraphcompute_amd._ops import linear_wgrad
    gw, gb = linear_wgrad(torch.zeros(0, 5, device="cuda"), torch.zeros(0, 7, device="cuda"))
    assert gw.shape == (5, 7) and float(gw.abs().sum()) == 0 and float(gb.abs().sum()) == 0


def test_dense_op_autograd_matches_linear():
    from fastgraphcompute_amd.gnn_ops import dense
    torch.manual_seed(5)
    lin = torch.nn.Linear(48, 20).cuda()
    x = torch.randn(3000, 48, device="cuda", requires_grad=True)
    go = torch.randn(3000, 20, device="cuda")
    y = dense(x, lin.weight, lin.bias)
    y.backward(go)
    got = (y.detach(), x.grad.clone(), lin.weight.grad.clone(), lin.bias.grad.clone())
    x.grad = None
    lin.zero_grad()
    y2 = lin(x)
    y2.backward(go)
    for a, b in zip(got, (y2.detach(), x.grad, lin.weight.grad, lin.bias.grad)):
        assert float((a - b).abs().max()) <= 2e-4 * float(b.abs().max())
    # without bias, and with an input that needs no gradient
    w = torch.randn(20, 48, device="cuda", requires_grad=True)
    y3 = dense(x.detach(), w, None)
    y3.sum().backward()
    assert float((w.grad - x.detach().sum(0).expand(20, 48)).abs().max()) < 1e-2


def test_gravnet_weight_gradients_against_float64():
    """All parameter gradients of one GravNetOp step against the same layer evaluated in float64 torch ops on the
    neighbour graph the GPU found."""
    from fastgraphcompute_amd.gnn_ops import GravNetOp
    torch.manual_seed(9)
    n, C, S, P, K = 6000, 24, 4, 16, 12
    op = GravNetOp(C, 20, S, P, K).cuda()
    x = torch.randn(n, C, device="cuda", requires_grad=True)
    rs = torch.tensor([0, 2500, n], device="cuda")
    go = torch.randn(n, 20, device="cuda")
    out, idx, dsq, space = op(x, rs)
    out.backward(go)
    got = {k: v.grad.double().cpu() for k, v in op.named_parameters()}
    gx = x.grad.double().cpu()

    xd = x.detach().double().cpu().requires_grad_(True)
    pd = {k: v.detach().double().cpu().requires_grad_(True) for k, v in op.named_parameters()}
    sp = xd @ pd["space_transformations.weight"].t() + pd["space_transformations.bias"]
    pr = xd @ pd["propagate_transformations.weight"].t() + pd["propagate_transformations.bias"]
    ii = idx.cpu()
    d2 = ((sp.unsqueeze(1) - sp[ii.clamp(min=0)]) ** 2).sum(-1)
    w = torch.exp(-10.0 * d2)
    f = pr[ii.clamp(min=0)] * (ii >= 0).unsqueeze(-1) * w.unsqueeze(-1)
    cat = torch.cat([xd, f.mean(1), f.max(1).values], dim=1)
    o = torch.relu(cat @ pd["output_transformations.0.weight"].t() + pd["output_transformations.0.bias"])
    o.backward(go.double().cpu())
    assert float((out.detach().double().cpu() - o.detach()).abs().max()) < 1e-4 * float(o.detach().abs().max())
    for k in got:
        ref = pd[k].grad
        # the space bias has no gradient at all (distances are translation invariant): measure its float32
        # noise against the gradient of the space weights
        scale = float(pd["space_transformations.weight"].grad.abs().max()) if k == "space_transformations.bias" \
            else float(ref.abs().max())
        assert float((got[k] - ref).abs().max()) < 2e-4 * scale, k
    assert float((gx - xd.grad).abs().max()) < 2e-4 * float(xd.grad.abs().max())


def test_use_dense_layers_keeps_results_and_parameters():
    """A model with its nn.Linear layers swapped for Dense ones: same parameters (shared), outputs and gradients."""
    from fastgraphcompute_amd.gnn_ops import Dense, use_dense_layers
    torch.manual_seed(3)
    model = torch.nn.Sequential(torch.nn.Linear(16, 40), torch.nn.ReLU(),
                                torch.nn.Sequential(torch.nn.Linear(40, 40, bias=False), torch.nn.Tanh()),
                                torch.nn.Linear(40, 3)).cuda()
    x = torch.randn(5000, 16, device="cuda")
    params = list(model.parameters())
    out = model(x)
    out.square().sum().backward()
    ref = [p.grad.clone() for p in params]
    model.zero_grad()
    state = {k: v.clone() for k, v in model.state_dict().items()}
    assert use_dense_layers(model) is model
    assert isinstance(model[0], Dense) and isinstance(model[2][0], Dense) and isinstance(model[3], Dense)
    assert all(a is b for a, b in zip(params, model.parameters()))          # the very same parameter tensors
    assert list(model.state_dict().keys()) == list(state.keys())
    out2 = model(x)
    assert float((out2 - out).abs().max()) <= 1e-5 * float(out.abs().max())
    out2.square().sum().backward()
    for p, r in zip(params, ref):
        assert float((p.grad - r).abs().max()) <= 2e-4 * float(r.abs().max())
    scripted = torch.jit.script(model)
    assert float((scripted(x) - out).abs().max()) <= 1e-5 * float(out.abs().max())
