"""The `fastgraphcompute` import path: the import lines of the reference's own tests and benchmark scripts, typed
as they stand there, must resolve to this implementation (same objects as `fastgraphcompute_amd`, nothing imported
twice)."""
import subprocess
import sys

import pytest


def test_reference_import_lines_resolve():
    # tests/test_bin_by_coordinates.py:5-6
    import fastgraphcompute.extensions
    from fastgraphcompute import bin_by_coordinates
    # tests/test_binned_select_knn.py:6,295
    from fastgraphcompute import binned_select_knn
    from fastgraphcompute.extensions.binned_select_knn import binned_select_knn as bsk2
    # tests/test_gnn_ops.py:4
    from fastgraphcompute.gnn_ops import GravNetOp
    # tests/test_index_replacer.py:6
    from fastgraphcompute import index_replacer
    # tests/test_oc_helper.py:5
    from fastgraphcompute import oc_helper_matrices, select_with_default
    # tests/test_torch_geometric_interface.py:3
    from fastgraphcompute.torch_geometric_interface import row_splits_from_strict_batch, strict_batch_from_row_splits
    # performance/oc_helper_helper.py:6
    from fastgraphcompute.extensions.oc_helper import max_same_valued_entries_per_row_split
    import fastgraphcompute
    import fastgraphcompute_amd
    from fastgraphcompute_amd.gnn_ops import GravNetOp as G2
    assert binned_select_knn is bsk2 is fastgraphcompute_amd.binned_select_knn
    assert bin_by_coordinates is fastgraphcompute_amd.bin_by_coordinates
    assert index_replacer is fastgraphcompute_amd.index_replacer
    assert oc_helper_matrices is fastgraphcompute_amd.oc_helper_matrices
    assert select_with_default is fastgraphcompute_amd.select_with_default
    assert GravNetOp is G2
    assert fastgraphcompute.extensions is fastgraphcompute_amd.extensions
    assert set(fastgraphcompute.extensions.__all__) >= {"bin_by_coordinates", "binned_select_knn", "index_replacer",
                                                        "oc_helper_matrices", "select_with_default"}
    assert callable(row_splits_from_strict_batch) and callable(strict_batch_from_row_splits)
    assert callable(max_same_valued_entries_per_row_split)


def test_alias_first_in_a_fresh_process():
    # importing the alias before (or without) the implementation package must work too
    code = ("from fastgraphcompute.gnn_ops import GravNetOp\n"
            "from fastgraphcompute import binned_select_knn\n"
            "import fastgraphcompute_amd\n"
            "assert binned_select_knn is fastgraphcompute_amd.binned_select_knn\n"
            "op = GravNetOp(8, 8, 3, 4, 5)\n"
            "assert sorted(op.state_dict()) == ['output_transformations.0.bias', 'output_transformations.0.weight',"
            " 'propagate_transformations.bias', 'propagate_transformations.weight', 'space_transformations.bias',"
            " 'space_transformations.weight']\n"
            "print('ok')\n")
    import os
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, "-c", code], cwd=root, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and r.stdout.strip().endswith("ok"), r.stderr[-2000:]


@pytest.mark.gpu
def test_reference_style_call_through_the_alias():
    # the shape of tests/test_binned_select_knn.py:97-123 of the reference: random points, two events, the result
    # against torch.cdist + topk
    import torch
    from fastgraphcompute import binned_select_knn
    torch.manual_seed(45)
    coords = torch.rand(1000, 3, device="cuda")
    row_splits = torch.tensor([0, 400, 1000], dtype=torch.int32, device="cuda")
    idx, distsq = binned_select_knn(5, coords, row_splits)
    for a, b in ((0, 400), (400, 1000)):
        d = torch.cdist(coords[a:b], coords[a:b]) ** 2
        ref = torch.topk(d, 5, largest=False).values
        assert torch.allclose(torch.sort(distsq[a:b], 1).values, torch.sort(ref, 1).values, atol=1e-6)
        assert int(idx[a:b].min()) >= a and int(idx[a:b].max()) < b
