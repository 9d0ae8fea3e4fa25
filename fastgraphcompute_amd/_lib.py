"""ctypes binding of libfgc_hip.so (the C ABI declared in include/fgc_hip.h).

There is no fallback: if the shared library is missing, or a tensor is not on
a HIP device, the call raises.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libfgc_hip.so")
_lib = None

c_i64p = ctypes.POINTER(ctypes.c_int64)
_vp, _i32, _i64, _f32, _sz = ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64, ctypes.c_float, ctypes.c_size_t

# name -> (restype, argtypes); must list every symbol of include/fgc_hip.h
SIGNATURES = {
    "fgc_version": (ctypes.c_int, []),
    "fgc_error_string": (ctypes.c_char_p, [ctypes.c_int]),
    "fgc_bin_geometry_workspace_bytes": (_sz, [_i64]),
    "fgc_bin_geometry_f32": (ctypes.c_int, [_vp, _i64, _i32, _i32, _i32, c_i64p, _i32, _f32, _i32, _vp, _vp,
                                            _vp, _sz, _vp]),
    "fgc_bin_points_f32": (ctypes.c_int, [_vp, _i64, _i32, _i32, _vp, _vp, _i32, c_i64p, _vp, _vp, _vp, _vp, _vp]),
    "fgc_binned_select_knn_workspace_bytes": (_sz, [_i64, _i32, _i32, c_i64p, _i32, _i32]),
    "fgc_binned_select_knn_f32": (ctypes.c_int, [_vp, _i64, _i32, _vp, c_i64p, _i32, _i32, _i32, c_i64p, _vp,
                                                 _i32, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "fgc_binned_select_knn_noalloc_f32": (ctypes.c_int, [_vp, _i64, _i32, _vp, c_i64p, _i32, _i32, _i32, c_i64p, _vp,
                                                         _i32, _vp, _vp, _vp, _vp]),
    "fgc_binned_knn_prepare_f32": (ctypes.c_int, [_vp, _i64, _i32, _vp, c_i64p, _i32, _i32, _i32, c_i64p, _vp, _vp,
                                                  _vp, _sz, _vp]),
    "fgc_binned_knn_prepare_ld_f32": (ctypes.c_int, [_vp, _i64, _i32, _i32, _vp, c_i64p, _i32, _i32, _i32, c_i64p, _vp,
                                                     _vp, _vp, _sz, _vp]),
    "fgc_binned_knn_search_f32": (ctypes.c_int, [_i64, _i32, c_i64p, _i32, _i32, _i32, c_i64p, _i32, _i32, _vp,
                                                 _vp, _vp, _vp, _vp, _sz, _vp]),
    "fgc_binned_select_knn_grad_sorted_workspace_bytes": (ctypes.c_size_t, [_i64, _i32]),
    "fgc_binned_select_knn_grad_sorted_f32": (ctypes.c_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i32, _i32, _vp, _vp, _sz,
                                                             _vp]),
    "fgc_binned_select_knn_grad_sorted_ld_f32": (ctypes.c_int, [_vp, _vp, _vp, _i32, _vp, _vp, _i32, _i64, _i32, _i32,
                                                                _vp, _vp, _sz, _vp]),
    "fgc_gravnet_aggregate_fwd_ld_f32": (ctypes.c_int, [_vp, _vp, _vp, _i32, _i64, _vp, _vp, _i32, _vp, _i64, _i32,
                                                        _i32, _vp, _vp]),
    "fgc_gravnet_aggregate_bwd_ld_f32": (ctypes.c_int, [_vp, _vp, _vp, _i32, _i64, _vp, _vp, _vp, _i32, _vp, _i32,
                                                        _vp, _i64, _i32, _i32, _vp, _vp]),
    "fgc_noalloc_init": (ctypes.c_int, []),
    "fgc_gravnet_aggregate_bwd_sorted_supported": (ctypes.c_int, [_i64, _i32, _i32, _i32, _i32]),
    "fgc_gravnet_aggregate_bwd_sorted_f32": (ctypes.c_int, [_vp, _vp, _vp, _vp, _i32, _vp, _vp, _vp, _i32, _vp, _i32,
                                                            _vp, _i64, _i32, _i32, _vp, _vp]),
    "fgc_index_replacer_i64": (ctypes.c_int, [_vp, _vp, _vp, _i64, _i64, _vp]),
    "fgc_binned_select_knn_grad_f32": (ctypes.c_int, [_vp, _vp, _vp, _vp, _i64, _i32, _i32, _vp, _vp, _vp]),
    "fgc_binned_knn_export_order_i32": (ctypes.c_int, [_i64, _i32, c_i64p, _i32, _i32, _i32, c_i64p, _i32, _vp, _sz,
                                                       _vp, _vp]),
    "fgc_select_with_default_f32": (ctypes.c_int, [_vp, _vp, _vp, _i64, _i32, _i32, _i64, _f32, _vp]),
    "fgc_select_with_default_b64": (ctypes.c_int, [_vp, _vp, _vp, _i64, _i32, _i32, _i64, ctypes.c_uint64, _vp]),
    "fgc_gravnet_aggregate_fwd_f32": (ctypes.c_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i32, _i32, _vp]),
    "fgc_gravnet_aggregate_bwd_f32": (ctypes.c_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i32, _i32,
                                                     _vp]),
    "fgc_select_knn_f32": (ctypes.c_int, [_vp, _i64, _i32, _vp, _vp, _i32, _i32, ctypes.c_double, _i32, _vp, _vp, _vp,
                                          _vp, _vp, ctypes.c_size_t, _vp]),
    "fgc_linear_wgrad_workspace_bytes": (ctypes.c_size_t, [_i64, _i32, _i32]),
    "fgc_linear_wgrad_f32": (ctypes.c_int, [_vp, _vp, _i64, _i32, _i32, _vp, _vp, _vp, ctypes.c_size_t, _vp]),
    "fgc_oc_helper_workspace_bytes": (ctypes.c_size_t, [_i64]),
    "fgc_oc_helper_objects_i64": (ctypes.c_int, [_vp, _i64, _vp, _i32, _i32, _i32, _vp, _vp, _vp, _vp,
                                                 ctypes.c_size_t, _vp]),
    "fgc_oc_helper_fill_i64": (ctypes.c_int, [_i64, _vp, _i32, _i64, _i64, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _vp,
                                              _vp, _vp, ctypes.c_size_t, _vp]),
}

ST_NONFINITE, ST_CLAMPED, ST_BAD_RANGE, ST_BAD_INDEX, ST_OC_TRUNCATED = 1, 2, 4, 8, 16
KNN_TF_COMPAT, KNN_ANY_ORDER, KNN_NO_MATRIX, KNN_FORCE_MATRIX = 1, 2, 4, 8   # bits of the kNN entry points' tf_compat argument


def lib():
    """Load libfgc_hip.so once; raise if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "fastgraphcompute_amd: %s is missing - build it with "
                "`python fastgraphcompute_amd/csrc/build.py` (hipcc, gfx950); there is no CPU fallback" % LIB_PATH)
        l = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(l, name)
            fn.restype = res
            fn.argtypes = args
        _lib = l
    return _lib


def check(rc):
    if rc != 0:
        msg = lib().fgc_error_string(rc).decode()
        if rc == -3:
            raise ValueError(msg)
        raise RuntimeError("fastgraphcompute_amd: %s (code %d)" % (msg, rc))


def require_device(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("fastgraphcompute_amd runs on MI355X (HIP) tensors only; got a %s tensor and "
                               "there is no CPU fallback" % t.device)


def stream_ptr():
    """The current HIP stream of the current device as a void pointer."""
    raw = getattr(torch._C, "_cuda_getCurrentRawStream", None)
    if raw is not None:         # (what torch.cuda.current_stream().cuda_stream returns, without building a Stream object)
        return ctypes.c_void_p(raw(torch.cuda.current_device()))
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


class on_device:
    """`with on_device(dev):` makes `dev` the current device like torch.cuda.device(dev), but does nothing at all when it
    already is (the usual case, and a few microseconds per call on the small-input path)."""
    __slots__ = ("ctx",)

    def __init__(self, dev):
        idx = dev.index if isinstance(dev, torch.device) else int(dev)
        self.ctx = None if (idx is None or idx == torch.cuda.current_device()) else torch.cuda.device(idx)

    def __enter__(self):
        if self.ctx is not None:
            self.ctx.__enter__()
        return self

    def __exit__(self, *exc):
        if self.ctx is not None:
            return self.ctx.__exit__(*exc)
        return False


def ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


def host_i64(values):
    arr = (ctypes.c_int64 * len(values))(*[int(v) for v in values])
    return arr
