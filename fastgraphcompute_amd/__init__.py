"""fastgraphcompute_amd - MI355X-native graph-building path of FastGraphCompute.

Drop-in for the reference package's binning / kNN / GravNet entry points
(fastgraphcompute/__init__.py:5-8): `import fastgraphcompute_amd as fastgraphcompute`.
All compute runs in hand-written HIP kernels (libfgc_hip.so); tensors must live
on the GPU.
"""
from .extensions.oc_helper import oc_helper_matrices, select_with_default
from .extensions.binned_select_knn import binned_select_knn
from .extensions.index_replacer import index_replacer
from .extensions.bin_by_coordinates import bin_by_coordinates
from . import config

__version__ = "0.1.0"
