"""CPU tests of the C-ABI library (loads, exports every declared symbol,
rejects bad arguments before touching a device) and of the host-side logic."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "fgc_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fgc_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from fastgraphcompute_amd import _lib
    L = _lib.lib()
    names = _declared_symbols()
    assert len(names) >= 12
    for nm in names:
        assert hasattr(L, nm), nm
    assert set(names) == set(_lib.SIGNATURES.keys())
    assert L.fgc_version() >= 100
    assert b"binning dimensions" in L.fgc_error_string(-3)


def test_argument_validation_without_device():
    from fastgraphcompute_amd import _lib
    L = _lib.lib()
    fake = ctypes.c_void_p(4096)
    nb = _lib.host_i64([10, 10, 10])
    rs = _lib.host_i64([0, 100])
    ws = L.fgc_binned_select_knn_workspace_bytes(100, 3, 3, nb, 2, 8)
    assert ws > 0

    def call(n=100, D=3, K=8, nbd=3, rs_=rs, n_rs=2, ws_bytes=ws, nb_=nb):
        return L.fgc_binned_knn_search_f32(n, D, rs_, n_rs, K, nbd, nb_, 0, 0, fake, fake, None, None, fake, ws_bytes, None)
    assert call(K=0) == -1 and call(K=1025) == -1
    assert call(nbd=1) == -3 and call(nbd=6) == -3 and call(D=2, nbd=3) == -3
    assert call(rs_=_lib.host_i64([0, 99])) == -1            # row splits do not end at n_vert
    assert call(rs_=_lib.host_i64([0, 120, 100]), n_rs=3) == -1
    assert call(ws_bytes=16) == -2
    assert call(nb_=_lib.host_i64([0, 10, 10])) == -1
    assert call(n=0, rs_=_lib.host_i64([0, 0])) == 0          # empty input is a no-op
    assert L.fgc_index_replacer_i64(fake, fake, fake, -1, 4, None) == -1
    assert L.fgc_binned_select_knn_grad_f32(fake, fake, fake, fake, 10, 0, 3, None, None, None) == -1
    assert L.fgc_gravnet_aggregate_fwd_f32(fake, fake, fake, fake, fake, None, 10, 4, 0, None) == -1


def test_host_wrappers_reject_cpu_tensors_and_bad_arguments():
    import fastgraphcompute_amd as fgc
    with pytest.raises(RuntimeError):
        fgc.binned_select_knn(3, torch.rand(10, 3), torch.tensor([0, 10]))
    # the wrapper is a scripted function like the reference's: its ValueErrors surface as torch.jit.Error,
    # a RuntimeError
    with pytest.raises((ValueError, RuntimeError, torch.jit.Error)):
        fgc.binned_select_knn(3, torch.rand(10, 0), torch.tensor([0, 10]))
    with pytest.raises((ValueError, RuntimeError, torch.jit.Error)):
        fgc.binned_select_knn(3, torch.rand(10, 3), torch.tensor([0, 10]), max_bin_dims=0)
    with pytest.raises(RuntimeError):
        fgc.bin_by_coordinates(torch.rand(10, 3), torch.tensor([0, 10]), n_bins=4)
    with pytest.raises((AssertionError, RuntimeError, torch.jit.Error)):
        fgc.index_replacer(torch.zeros(3, dtype=torch.int32), torch.zeros(3, dtype=torch.int64))
    with pytest.raises((RuntimeError, torch.jit.Error)):          # no CPU fallback
        fgc.oc_helper_matrices(torch.tensor([1, 1, 2]), torch.tensor([0, 3]))
    with pytest.raises(RuntimeError):
        fgc.extensions.oc_helper.max_same_valued_entries_per_row_split(torch.tensor([1, 1, 2]), torch.tensor([0, 3]),
                                                                       True)


def test_n_bins_heuristic_host():
    from fastgraphcompute_amd.extensions.binned_select_knn import calculate_optimal_bins
    from fastgraphcompute_amd.workloads import cfg5_many_events_d8
    t = lambda v: torch.tensor(v, dtype=torch.int64)
    assert calculate_optimal_bins(t([0, 6000, 10000]), 16, 3) == 18
    assert calculate_optimal_bins(t([0, 50000, 100000, 150000, 200000]), 40, 3) == 30
    assert calculate_optimal_bins(t([0, 1000000]), 64, 3) == 30
    assert calculate_optimal_bins(torch.from_numpy(cfg5_many_events_d8()["row_splits"]).long(), 100, 3) == 13
    assert calculate_optimal_bins(t([0, 3333, 5000, 10000]), 50, 3) == 11
    assert calculate_optimal_bins(t([0, 50, 100]), 8, 3) == 5


def test_own_search_grid_host():
    from fastgraphcompute_amd.workloads import cfg5_many_events_d8
    from fastgraphcompute_amd._ops import choose_search_grid
    t = lambda v: torch.tensor(v, dtype=torch.int64)
    assert choose_search_grid(t([0, 1000000]), 3, 3) == (3, 10)          # ~150 chunks of 64 points per bin row
    assert choose_search_grid(t([0, 50000, 100000, 150000, 200000]), 4, 3) == (4, 1)
    assert choose_search_grid(t([0, 200000]), 4, 3) == (4, 2)
    assert choose_search_grid(torch.from_numpy(cfg5_many_events_d8()["row_splits"]).long(), 8, 3) == (5, 1)
    assert choose_search_grid(t([0, 1000000]), 6, 3) == (5, 2)
    assert choose_search_grid(t([0, 6000, 10000]), 3, 3) == (3, 1)
    assert choose_search_grid(t([0, 10]), 2, 3) == (2, 1)
    assert choose_search_grid(t([0, 100000000]), 2, 2) == (2, 30)       # capped


def test_workloads_are_deterministic():
    from fastgraphcompute_amd import workloads
    a, b = workloads.cfg4_zipf_blobs(0.01), workloads.cfg4_zipf_blobs(0.01)
    assert a["coords"].dtype.name == "float32" and (a["coords"] == b["coords"]).all()
    w5 = workloads.cfg5_many_events_d8()
    assert w5["row_splits"][-1] == 500000 and len(w5["row_splits"]) == 65 and w5["coords"].shape == (500000, 8)
    assert workloads.cfg2_blobs_4events(0.1)["coords"].shape == (20000, 4)


def test_gravnet_module_state_dict_names():
    from fastgraphcompute_amd.gnn_ops import GravNetOp
    op = GravNetOp(8, 6, 3, 5, 4)
    assert set(op.state_dict().keys()) == {
        "space_transformations.weight", "space_transformations.bias", "propagate_transformations.weight",
        "propagate_transformations.bias", "output_transformations.0.weight", "output_transformations.0.bias"}
    assert op.output_transformations[0].in_features == 8 + 2 * 5


def test_ops_are_registered_and_wrappers_script():
    import fastgraphcompute_amd  # noqa: F401
    from fastgraphcompute_amd.gnn_ops import GravNetOp
    # the reference's dispatcher surface (same namespaces, names and schemas)
    s = str(torch.ops.fastgraphcompute_custom_ops.binned_select_knn_autograd.default._schema)
    assert "Tensor coords, Tensor row_splits, int K, Tensor? direction, Tensor? n_bins, int max_bin_dims, " \
           "bool torch_compatible_indices" in s
    assert "Tensor? bin_width, Tensor? n_bins, bool calc_n_per_bin, bool pre_normalized" in \
        str(torch.ops.bin_by_coordinates.bin_by_coordinates.default._schema)
    assert torch.ops.index_replacer.index_replacer is not None
    assert torch.ops.binned_select_knn_grad.binned_select_knn_grad is not None
    # scripting compiles without a device
    sm = torch.jit.script(GravNetOp(8, 6, 3, 5, 4))
    assert "gravnet_layer_core" in str(sm.code) and "dense_split" in str(sm.code)


def test_integration_shim_compiles_against_the_header():
    """The reference-side binding shown in the repository's integration notes (the C++ a maintainer would put behind
    BinnedKNNAutograd and the *_cuda_fn symbols) is compiled, syntax only, against include/fgc_hip.h and the torch
    headers: argument counts and types of every call must match the header."""
    import shutil
    import subprocess
    import tempfile
    import torch.utils.cpp_extension as ce
    if shutil.which("g++") is None:
        pytest.skip("no g++")
    text = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    blocks = re.findall(r"```cpp\n(.*?)```", text, flags=re.S)
    assert blocks, "the integration notes hold no C++ block"
    src = "\n".join(blocks)
    for fn in ("fgc_binned_select_knn_f32", "fgc_binned_select_knn_grad_f32", "fgc_index_replacer_i64",
               "fgc_bin_points_f32"):
        assert fn in src, fn
    with tempfile.TemporaryDirectory() as tmp:
        path = os.path.join(tmp, "shim.cpp")
        with open(path, "w") as f:
            f.write(src)
        cmd = ["g++", "-std=c++17", "-fsyntax-only", "-D__HIP_PLATFORM_AMD__", "-DUSE_ROCM",
               "-I", os.path.join(ROOT, "include"), "-I", "/opt/rocm/include", "-I", "/usr/include/python3.10"]
        for inc in ce.include_paths():
            cmd += ["-I", inc]
        r = subprocess.run(cmd + [path], capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-4000:]


def test_tile_backward_predicate_and_entry_point_agree():
    """GravNetOp's backward asks fgc_gravnet_aggregate_bwd_sorted_supported before it takes the tile kernel; the
    entry point must reject (FGC_ESHAPE, nothing launched) exactly the shapes the predicate turns down - among them
    layers of 2^24 points and more, which fit this GPU - and name the general entry point in its message."""
    import ctypes
    from fastgraphcompute_amd import _lib
    L = _lib.lib()
    p = ctypes.c_void_p(4096)
    assert b"general entry point" in L.fgc_error_string(-5)
    cases = [(100, 40, 32, 32, 32), (100, 64, 64, 64, 64), (100, 65, 32, 32, 32), (100, 40, 8, 8, 8), (100, 40, 65, 65, 65),
             ((1 << 24) - 1, 40, 32, 32, 32), (1 << 24, 40, 32, 32, 32), (20_000_000, 40, 32, 32, 32),
             (1 << 23, 40, 32, 128, 32), (1 << 23, 40, 32, 32, 128), (1000, 40, 32, 1 << 22, 32), (0, 40, 32, 32, 32)]
    for n, K, P, ldf, ldg in cases:
        ok = L.fgc_gravnet_aggregate_bwd_sorted_supported(n, K, P, ldf, ldg)
        if ok and n > 0:
            continue          # a supported shape would launch: only the rejections can be tried without a GPU
        rc = L.fgc_gravnet_aggregate_bwd_sorted_f32(p, p, p, p, ldf, p, p, p, P, p, ldg, p, n, K, P, None, None)
        assert (rc == -5) == (not ok), (n, K, P, ldf, ldg, ok, rc)
    assert L.fgc_gravnet_aggregate_bwd_sorted_supported(1 << 24, 40, 32, 32, 32) == 0
    assert L.fgc_gravnet_aggregate_bwd_sorted_supported((1 << 24) - 1, 40, 32, 32, 32) == 1
