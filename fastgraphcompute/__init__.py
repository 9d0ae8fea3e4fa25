"""Import-path alias: `fastgraphcompute` resolves to the MI355X implementation in `fastgraphcompute_amd`.

Code written against the reference package (fastgraphcompute/__init__.py:5-8, extensions/__init__.py:1-14)
- `from fastgraphcompute import binned_select_knn`, `from fastgraphcompute.gnn_ops import GravNetOp`,
`import fastgraphcompute.extensions`, `from fastgraphcompute.extensions.binned_select_knn import ...` - runs
unmodified: every sub-module name below is bound to the *same* module object as its `fastgraphcompute_amd`
counterpart (nothing is imported twice, so the torch ops are registered once).  The object-condensation loss
(`fastgraphcompute.object_condensation`) is not part of this package."""
import importlib
import sys

import fastgraphcompute_amd as _impl

_SUBMODULES = (
    "extensions",
    "extensions.bin_by_coordinates",
    "extensions.binned_select_knn",
    "extensions.index_replacer",
    "extensions.oc_helper",
    "extensions.select_knn",
    "gnn_ops",
    "torch_geometric_interface",
    "config",
)
for _name in _SUBMODULES:
    sys.modules[__name__ + "." + _name] = importlib.import_module("fastgraphcompute_amd." + _name)

extensions = sys.modules[__name__ + ".extensions"]
gnn_ops = sys.modules[__name__ + ".gnn_ops"]
torch_geometric_interface = sys.modules[__name__ + ".torch_geometric_interface"]
config = _impl.config

for _name in ("bin_by_coordinates", "binned_select_knn", "index_replacer", "oc_helper_matrices",
              "select_with_default"):
    globals()[_name] = getattr(_impl, _name)

__version__ = _impl.__version__
__all__ = ["bin_by_coordinates", "binned_select_knn", "index_replacer", "oc_helper_matrices",
           "select_with_default", "extensions", "gnn_ops", "torch_geometric_interface", "config"]
