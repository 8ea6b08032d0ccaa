"""Loads the native libraries of this package.

* ``libpca_neighbors.so`` -- HIP kernels behind the C ABI declared in
  ``include/pca_neighbors.h`` (bound with ctypes as :data:`capi`).
* ``_torch_ops.so`` -- registers ``torch.ops.torch_cluster.knn`` /
  ``radius`` / ``nearest`` / ``fps`` / ``cuda_version``, the operators the reference package loads from
  its per-operator shared objects (``torch_cluster/__init__.py:8-21``).

There is no fallback: if a library is missing the import fails and says how to
build it.
"""
import ctypes
import os

import torch  # first: the HIP runtime PyTorch ships must be the one in use

_HERE = os.path.dirname(os.path.abspath(__file__))
CAPI_PATH = os.path.join(_HERE, "libpca_neighbors.so")
TORCH_OPS_PATH = os.path.join(_HERE, "_torch_ops.so")

_BUILD_HINT = ("build it with `python pytorch_cluster_amd/build.py` "
               "(or `python -c 'import __graft_entry__ as g; g.build()'`)")

PCA_F32, PCA_F64, PCA_F16, PCA_BF16 = 0, 1, 2, 3
PCA_EDGES_DROP_SELF, PCA_EDGES_X_FIRST, PCA_SEGMENTS_BY_ID = 1, 2, 4
PCA_FIXED_SCRATCH_BYTES = 32 << 20

_vp = ctypes.c_void_p
_i64 = ctypes.c_int64

# name -> (restype, argtypes); mirrors include/pca_neighbors.h
C_ABI = {
    "pca_abi_version": (ctypes.c_int, []),
    "pca_status_string": (ctypes.c_char_p, [ctypes.c_int]),
    "pca_last_error": (ctypes.c_char_p, []),
    "pca_time_next_search": (ctypes.c_int, [_vp, _vp]),
    "pca_report_examples": (ctypes.c_int, [_vp]),
    "pca_knn_workspace_bytes": (ctypes.c_size_t,
                                [_i64, _i64, _i64, _i64, _i64, ctypes.c_int]),
    "pca_knn": (ctypes.c_int,
                [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64,
                 ctypes.c_int, ctypes.c_int, ctypes.c_int, _vp, _vp, _vp, _vp,
                 ctypes.c_size_t, _vp]),
    "pca_segment_pointers": (ctypes.c_int,
                             [_vp, _i64, _vp, _i64, _i64, _vp, _vp, _vp]),
    "pca_knn_fixed_scratch": (ctypes.c_int,
                              [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64,
                               _i64, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                               _vp, _vp, _vp, _vp]),
    "pca_knn_binned_workspace_bytes": (ctypes.c_size_t,
                                       [_i64, _i64, _i64, _i64, _i64]),
    "pca_knn_binned": (ctypes.c_int,
                       [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64,
                        ctypes.c_int, _vp, _vp, _vp, _vp, ctypes.c_size_t,
                        _vp]),
    "pca_radius_slots": (_i64, [_i64, _i64]),
    "pca_radius_workspace_bytes": (ctypes.c_size_t,
                                   [_i64, _i64, _i64, _i64, _i64,
                                    ctypes.c_int]),
    "pca_radius": (ctypes.c_int,
                   [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64,
                    ctypes.c_double, _i64, ctypes.c_int, ctypes.c_int,
                    ctypes.c_int, _vp, _vp, _vp, ctypes.c_size_t, _vp]),
    "pca_radius_binned_workspace_bytes": (ctypes.c_size_t,
                                          [_i64, _i64, _i64, _i64, _i64]),
    "pca_radius_binned": (ctypes.c_int,
                          [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64,
                           ctypes.c_double, _i64, ctypes.c_int, ctypes.c_int,
                           _vp, _vp, _vp, ctypes.c_size_t, _vp]),
    "pca_nearest_workspace_bytes": (ctypes.c_size_t,
                                    [_i64, _i64, _i64, _i64, ctypes.c_int]),
    "pca_nearest": (ctypes.c_int,
                    [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, ctypes.c_int,
                     _vp, _vp, ctypes.c_size_t, _vp]),
    "pca_nearest_binned_workspace_bytes": (ctypes.c_size_t,
                                           [_i64, _i64, _i64, _i64]),
    "pca_nearest_binned": (ctypes.c_int,
                           [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp,
                            _vp, ctypes.c_size_t, _vp]),
    "pca_host_last_error": (ctypes.c_char_p, []),
    "pca_knn_host": (ctypes.c_int,
                     [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64,
                      ctypes.c_int, ctypes.c_int, ctypes.c_int, _vp, _vp,
                      _vp]),
    "pca_radius_host": (ctypes.c_int,
                        [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64,
                         ctypes.c_double, _i64, ctypes.c_int, ctypes.c_int,
                         ctypes.c_int, ctypes.c_int, _vp, _vp]),
    "pca_fps_host": (ctypes.c_int,
                     [_vp, _vp, _vp, _vp, _i64, _i64, _i64, ctypes.c_int,
                      ctypes.c_int, _vp]),
    "pca_nearest_host": (ctypes.c_int,
                         [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64,
                          ctypes.c_int, ctypes.c_int, _vp]),
    "pca_fps_workspace_bytes": (ctypes.c_size_t,
                                [_i64, _i64, _i64, _i64, ctypes.c_int]),
    "pca_fps": (ctypes.c_int,
                [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, ctypes.c_int,
                 _vp, _vp, ctypes.c_size_t, _vp]),
}


def load_capi():
    if not os.path.exists(CAPI_PATH):
        raise ImportError("%s is missing; %s" % (CAPI_PATH, _BUILD_HINT))
    lib = ctypes.CDLL(CAPI_PATH, mode=ctypes.RTLD_GLOBAL)
    for name, (restype, argtypes) in C_ABI.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    return lib


def load_torch_ops():
    if not os.path.exists(TORCH_OPS_PATH):
        raise ImportError("%s is missing; %s" % (TORCH_OPS_PATH, _BUILD_HINT))
    torch.ops.load_library(TORCH_OPS_PATH)


capi = load_capi()
load_torch_ops()
