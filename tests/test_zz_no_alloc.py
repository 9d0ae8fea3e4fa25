"""fgc_binned_select_knn_noalloc_f32 (the entry point that allocates nothing: its workspace is a fixed array in
the library's own device memory) against fgc_binned_select_knn_f32 with a caller's workspace, through the C ABI:
two calls in a row, the second with a smaller input, so that the second call runs on the leftovers of the first.
Results must be bit-identical (same kernels, same order of operations).  Collected last on purpose."""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _call(L, lib, noalloc, coords, rs_host, K, nbd, nb, direction=None, tf_compat=0):
    dev = coords.device
    n, D = coords.shape
    rs_dev = torch.tensor(rs_host, dtype=torch.int64, device=dev)
    rs_arr, nb_arr = lib.host_i64(rs_host), lib.host_i64(nb)
    idx = torch.full((n, K), -7, dtype=torch.int64, device=dev)
    dist = torch.full((n, K), -7.0, dtype=torch.float32, device=dev)
    status = torch.zeros(4, dtype=torch.int32, device=dev)
    st = lib.stream_ptr()
    if noalloc:
        rc = L.fgc_binned_select_knn_noalloc_f32(lib.ptr(coords), n, D, lib.ptr(rs_dev), rs_arr, len(rs_host), K, nbd,
                                                 nb_arr, lib.ptr(direction), tf_compat, lib.ptr(idx), lib.ptr(dist),
                                                 lib.ptr(status), st)
    else:
        ws_bytes = L.fgc_binned_select_knn_workspace_bytes(n, D, nbd, nb_arr, len(rs_host), K)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
        rc = L.fgc_binned_select_knn_f32(lib.ptr(coords), n, D, lib.ptr(rs_dev), rs_arr, len(rs_host), K, nbd, nb_arr,
                                         lib.ptr(direction), tf_compat, lib.ptr(idx), lib.ptr(dist), lib.ptr(status),
                                         None, lib.ptr(ws), ws_bytes, st)
    torch.cuda.synchronize()
    return rc, idx.cpu().numpy(), dist.cpu().numpy(), status.cpu().numpy()


def test_noalloc_matches_workspace_entry_point_twice_in_a_row(oracle):
    from fastgraphcompute_amd import _lib
    from fastgraphcompute_amd.workloads import cfg4_zipf_blobs, cfg2_blobs_4events
    from tests.util import assert_knn_equal
    L = _lib.lib()
    # first call: 200 000 clustered points in one event, K = 64
    w = cfg4_zipf_blobs(0.2)
    c1 = torch.from_numpy(w["coords"]).cuda()
    rs1 = [int(v) for v in w["row_splits"]]
    rc, i1, d1, s1 = _call(L, _lib, True, c1, rs1, 64, 3, [6, 6, 6])
    assert rc == 0
    rc, ei1, ed1, es1 = _call(L, _lib, False, c1, rs1, 64, 3, [6, 6, 6])
    assert rc == 0
    np.testing.assert_array_equal(i1, ei1)
    np.testing.assert_array_equal(d1, ed1)
    np.testing.assert_array_equal(s1, es1)
    # second call, smaller and of another shape (4 events, 4 coordinates, K = 40, a direction array): it runs on
    # whatever the first call left in the fixed array
    w = cfg2_blobs_4events(0.1)
    c2 = torch.from_numpy(w["coords"]).cuda()
    rs2 = [int(v) for v in w["row_splits"]]
    direction = torch.from_numpy(np.random.default_rng(5).integers(0, 4, c2.shape[0])).cuda()
    rc, i2, d2, s2 = _call(L, _lib, True, c2, rs2, 40, 3, [3, 3, 3], direction)
    assert rc == 0
    rc, ei2, ed2, es2 = _call(L, _lib, False, c2, rs2, 40, 3, [3, 3, 3], direction)
    assert rc == 0
    np.testing.assert_array_equal(i2, ei2)
    np.testing.assert_array_equal(d2, ed2)
    np.testing.assert_array_equal(s2, es2)
    # and both against the CPU checker
    oi, od = oracle.binned_select_knn(64, c1.cpu().numpy(), np.array(rs1), n_threads=16)
    assert_knn_equal(i1, d1, oi, od, "first call")
    oi, od = oracle.binned_select_knn(40, c2.cpu().numpy(), np.array(rs2), direction=direction.cpu().numpy(),
                                      n_threads=16)
    assert_knn_equal(i2, d2, oi, od, "second call")


def test_noalloc_rejects_inputs_beyond_its_fixed_scratch():
    from fastgraphcompute_amd import _lib
    L = _lib.lib()
    n, D, K = 3_000_000, 3, 8
    nb = _lib.host_i64([10, 10, 10])
    assert L.fgc_binned_select_knn_workspace_bytes(n, D, 3, nb, 2, K) > (32 << 20)
    coords = torch.zeros((n, D), device="cuda")
    idx = torch.full((n, K), -7, dtype=torch.int64, device="cuda")
    dist = torch.empty((n, K), device="cuda")
    rs = torch.tensor([0, n], device="cuda")
    status = torch.zeros(4, dtype=torch.int32, device="cuda")
    rc = L.fgc_binned_select_knn_noalloc_f32(_lib.ptr(coords), n, D, _lib.ptr(rs), _lib.host_i64([0, n]), 2, K, 3, nb,
                                             None, 0, _lib.ptr(idx), _lib.ptr(dist), _lib.ptr(status),
                                             _lib.stream_ptr())
    torch.cuda.synchronize()
    assert rc == -4
    assert b"FGC_NOALLOC_SCRATCH_BYTES" in L.fgc_error_string(rc)
    with pytest.raises(RuntimeError, match="scratch"):
        _lib.check(rc)
    assert int((idx != -7).sum().item()) == 0          # nothing was launched


def test_noalloc_allocates_nothing_and_can_be_captured():
    """After fgc_noalloc_init (the scratch address looked up ahead of time) the entry point leaves the device's free
    memory unchanged, and it can be captured into a HIP graph: every replay, with eager work and synchronisations in
    between, equals the eager call on the same input."""
    from fastgraphcompute_amd import _lib
    L = _lib.lib()
    assert L.fgc_noalloc_init() == 0
    n, D, K = 30000, 3, 24
    rs_host = [0, 11000, n]
    rs = torch.tensor(rs_host, dtype=torch.int64, device="cuda")
    rsa, nb = _lib.host_i64(rs_host), _lib.host_i64([4, 4, 4])
    coords = torch.rand(n, D, device="cuda")
    idx = torch.empty((n, K), dtype=torch.int64, device="cuda")
    dist = torch.empty((n, K), dtype=torch.float32, device="cuda")
    status = torch.zeros(4, dtype=torch.int32, device="cuda")

    def enqueue():
        _lib.check(L.fgc_binned_select_knn_noalloc_f32(_lib.ptr(coords), n, D, _lib.ptr(rs), rsa, 3, K, 3, nb, None, 0,
                                                       _lib.ptr(idx), _lib.ptr(dist), _lib.ptr(status),
                                                       _lib.stream_ptr()))

    enqueue()
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    enqueue()
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before, "the call changed the device's free memory"
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=side):
        enqueue()
    ws_bytes = L.fgc_binned_select_knn_workspace_bytes(n, D, 3, nb, 3, K)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda")
    ref_i, ref_d = torch.empty_like(idx), torch.empty_like(dist)
    gen = torch.Generator(device="cuda").manual_seed(9)
    for rep in range(3):
        coords.copy_(torch.rand(n, D, device="cuda", generator=gen) * (rep + 1))
        g.replay()
        torch.cuda.synchronize()
        got_i, got_d = idx.clone(), dist.clone()
        _lib.check(L.fgc_binned_select_knn_f32(_lib.ptr(coords), n, D, _lib.ptr(rs), rsa, 3, K, 3, nb, None, 0,
                                               _lib.ptr(ref_i), _lib.ptr(ref_d), _lib.ptr(status), None, _lib.ptr(ws),
                                               ws_bytes, _lib.stream_ptr()))              # eager work in between
        torch.cuda.synchronize()
        assert torch.equal(got_d, ref_d) and torch.equal(got_i, ref_i), "replay %d differs" % rep
