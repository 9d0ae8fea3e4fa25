"""The C-ABI calls allocate nothing, never synchronise and clear memory with kernels, so a whole forward can be
captured into a HIP graph.  Every replay is compared with an eager call on the same input, with eager work and
synchronisations between the replays."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_forward_captured_in_a_graph_replays_correctly():
    from fastgraphcompute_amd import _lib, binned_select_knn
    from fastgraphcompute_amd._ops import choose_search_grid
    L = _lib.lib()
    n, D, K = 20000, 3, 16
    rs_host = torch.tensor([0, 8000, n], dtype=torch.int64)
    rs = rs_host.cuda()
    nbd, nb1 = choose_search_grid(rs_host, D, 3)
    nb = _lib.host_i64([nb1] * nbd)
    rsa = _lib.host_i64(rs_host.tolist())
    ws_bytes = L.fgc_binned_select_knn_workspace_bytes(n, D, nbd, nb, 3, K)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda")
    status = torch.zeros(4, dtype=torch.int32, device="cuda")
    coords = torch.rand(n, D, device="cuda")
    idx = torch.empty((n, K), dtype=torch.int64, device="cuda")
    dist = torch.empty((n, K), dtype=torch.float32, device="cuda")

    def enqueue():
        _lib.check(L.fgc_binned_select_knn_f32(_lib.ptr(coords), n, D, _lib.ptr(rs), rsa, 3, K, nbd, nb, None,
                                               _lib.KNN_ANY_ORDER,       # the row order binned_select_knn asks for
                                               _lib.ptr(idx), _lib.ptr(dist), _lib.ptr(status), None, _lib.ptr(ws),
                                               ws_bytes, _lib.stream_ptr()))

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        enqueue()                                   # warm-up on the capture stream
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=side):
        enqueue()
    gen = torch.Generator(device="cuda").manual_seed(5)
    for rep in range(4):
        coords.copy_(torch.rand(n, D, device="cuda", generator=gen) * (rep + 1))   # new input, same buffers
        g.replay()
        torch.cuda.synchronize()
        got_i, got_d = idx.clone(), dist.clone()
        ref_i, ref_d = binned_select_knn(K, coords.clone(), rs)                      # eager work in between
        torch.cuda.synchronize()
        assert torch.equal(got_d, ref_d), "replay %d: distances differ" % rep
        assert torch.equal(got_i, ref_i), "replay %d: indices differ" % rep
        assert int(status[0]) & (_lib.ST_NONFINITE | _lib.ST_BAD_RANGE) == 0
