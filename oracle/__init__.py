"""TEST INFRASTRUCTURE ONLY.

CPU checker for the kNN / radius neighbour-search path.  Only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import this package; the product (``pytorch_cluster_amd``) never does.

Layers (reference file:line each one follows):

* ``knn_op`` / ``radius_op``: the operator as the reference's GPU build
  computes it -- host wrapper ``csrc/cuda/knn_cuda.cu:86-135`` /
  ``csrc/cuda/radius_cuda.cu:44-96`` around the kernels restated in
  ``neighbors_oracle.c``.
* ``knn`` / ``knn_graph`` / ``radius`` / ``radius_graph``: the Python entry
  points ``torch_cluster/knn.py:6-82,85-144`` and
  ``torch_cluster/radius.py:6-88,91-148`` restated with numpy
  (``searchsorted`` in place of ``bucketize``).
* ``ref_knn`` / ``ref_radius``: the reference's own CPU operators
  (``csrc/cpu/knn_cpu.cpp:7-105``, ``csrc/cpu/radius_cpu.cpp:7-117``) compiled
  from the reference sources into ``oracle/_ref`` when those are available.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_REF_PATH = os.path.join(_HERE, "_ref", "libref_cpu.so")

_i64p = ctypes.POINTER(ctypes.c_int64)
_DTYPE_CODE = {np.dtype(np.float32): 0, np.dtype(np.float64): 1}


def build(with_ref=True):
    """Compiles the C restatement and, when the reference sources are present,
    the reference's CPU operators."""
    subprocess.check_call(["make", "-C", _HERE, "oracle"])
    if with_ref and os.path.isdir("/root/reference/csrc"):
        subprocess.check_call(["make", "-C", _HERE, "ref"])


_lib = None


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build(with_ref=False)
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.oracle_compact.restype = ctypes.c_int64
    return _lib


def _ptr(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _as_points(a):
    a = np.asarray(a)
    if a.dtype not in _DTYPE_CODE:
        raise TypeError(f"oracle supports float32/float64, got {a.dtype}")
    if a.ndim != 2:
        raise RuntimeError("Input mismatch")
    return np.ascontiguousarray(a)


def _as_ptr(p):
    if p is None:
        return None
    p = np.ascontiguousarray(np.asarray(p), dtype=np.int64)
    if p.ndim != 1:
        raise RuntimeError("Input mismatch")
    return p


def _suffix(dtype):
    return "f32" if dtype == np.float32 else "f64"


def _scalar(dtype, v):
    return ctypes.c_float(v) if dtype == np.float32 else ctypes.c_double(v)


def knn_dense(x, y, ptr_x, ptr_y, k, cosine=False, fma_mode=1):
    """The kernel's raw output: (col [m,k] int64, -1 padded; dist [m,k])."""
    lib = _load()
    x, y = _as_points(x), _as_points(y)
    if x.shape[1] != y.shape[1] or x.dtype != y.dtype:
        raise RuntimeError("Input mismatch")
    ptr_x, ptr_y = _as_ptr(ptr_x), _as_ptr(ptr_y)
    if (ptr_x is None) != (ptr_y is None):
        # the host wrapper fills a missing one with [0, N]; then the lengths
        # must agree
        if ptr_x is None:
            ptr_x = np.array([0, x.shape[0]], dtype=np.int64)
        else:
            ptr_y = np.array([0, y.shape[0]], dtype=np.int64)
    if ptr_x is not None and ptr_x.size != ptr_y.size:
        raise RuntimeError("Input mismatch")
    nseg = 1 if ptr_x is None else ptr_x.size - 1
    m = y.shape[0]
    row = np.empty(m * k, dtype=np.int64)
    col = np.empty(m * k, dtype=np.int64)
    dist = np.empty(m * k, dtype=x.dtype)
    fn = getattr(lib, "oracle_knn_dense_" + _suffix(x.dtype))
    rc = fn(_ptr(x), _ptr(y), _ptr(ptr_x), _ptr(ptr_y),
            ctypes.c_int64(x.shape[0]), ctypes.c_int64(m),
            ctypes.c_int64(x.shape[1]), ctypes.c_int64(nseg),
            ctypes.c_int64(k), ctypes.c_int(int(cosine)),
            ctypes.c_int(int(fma_mode)), _ptr(row), _ptr(col), _ptr(dist))
    if rc != 0:
        raise RuntimeError("oracle_knn_dense failed")
    return row.reshape(m, k), col.reshape(m, k), dist.reshape(m, k)


def _compact(row, col, mask_src):
    lib = _load()
    slots = row.size
    e = lib.oracle_compact(_ptr(row), _ptr(col), _ptr(mask_src),
                           ctypes.c_int64(slots), None, ctypes.c_int64(0))
    out = np.empty((2, e), dtype=np.int64)
    lib.oracle_compact(_ptr(row), _ptr(col), _ptr(mask_src),
                       ctypes.c_int64(slots), _ptr(out), ctypes.c_int64(e))
    return out


def knn_op(x, y, ptr_x, ptr_y, k, cosine=False, num_workers=1, fma_mode=1):
    """``torch_cluster::knn`` as the GPU build computes it; numpy in/out."""
    if k > 100:
        raise RuntimeError("`k` needs to smaller than or equal to 100")
    row, col, _ = knn_dense(x, y, ptr_x, ptr_y, k, cosine, fma_mode)
    row = np.ascontiguousarray(row.reshape(-1))
    col = np.ascontiguousarray(col.reshape(-1))
    return _compact(row, col, col)


def radius_dense(x, y, ptr_x, ptr_y, r, max_num_neighbors,
                 ignore_same_index=False, fma_mode=1):
    """Raw slot arrays (col [m,max] int64, -1 padded) and per-query scan
    lengths."""
    lib = _load()
    x, y = _as_points(x), _as_points(y)
    if x.shape[1] != y.shape[1] or x.dtype != y.dtype:
        raise RuntimeError("Input mismatch")
    ptr_x, ptr_y = _as_ptr(ptr_x), _as_ptr(ptr_y)
    if (ptr_x is None) != (ptr_y is None):
        if ptr_x is None:
            ptr_x = np.array([0, x.shape[0]], dtype=np.int64)
        else:
            ptr_y = np.array([0, y.shape[0]], dtype=np.int64)
    if ptr_x is not None and ptr_x.size != ptr_y.size:
        raise RuntimeError("Input mismatch")
    nseg = 1 if ptr_x is None else ptr_x.size - 1
    m = y.shape[0]
    row = np.empty(m * max_num_neighbors, dtype=np.int64)
    col = np.empty(m * max_num_neighbors, dtype=np.int64)
    scanned = np.empty(m, dtype=np.int64)
    # r * r in double, narrowed to the element type at the launch
    r2 = x.dtype.type(float(r) * float(r))
    fn = getattr(lib, "oracle_radius_dense_" + _suffix(x.dtype))
    rc = fn(_ptr(x), _ptr(y), _ptr(ptr_x), _ptr(ptr_y),
            ctypes.c_int64(x.shape[0]), ctypes.c_int64(m),
            ctypes.c_int64(x.shape[1]), ctypes.c_int64(nseg),
            _scalar(x.dtype, float(r2)), ctypes.c_int64(max_num_neighbors),
            ctypes.c_int(int(ignore_same_index)), ctypes.c_int(int(fma_mode)),
            _ptr(row), _ptr(col), _ptr(scanned))
    if rc != 0:
        raise RuntimeError("oracle_radius_dense failed")
    return (row.reshape(m, max_num_neighbors),
            col.reshape(m, max_num_neighbors), scanned)


def radius_op(x, y, ptr_x, ptr_y, r, max_num_neighbors, num_workers=1,
              ignore_same_index=False, fma_mode=1):
    """``torch_cluster::radius`` as the GPU build computes it."""
    row, col, _ = radius_dense(x, y, ptr_x, ptr_y, r, max_num_neighbors,
                               ignore_same_index, fma_mode)
    row = np.ascontiguousarray(row.reshape(-1))
    col = np.ascontiguousarray(col.reshape(-1))
    return _compact(row, col, row)


# --------------------------------------------------------------------------
# 16-bit element types (bit patterns as uint16; kind 0 = fp16, 1 = bf16)
# --------------------------------------------------------------------------

def _as_bits(a):
    a = np.ascontiguousarray(a)
    if a.dtype == np.float16:
        a = a.view(np.uint16)
    if a.dtype != np.uint16 or a.ndim != 2:
        raise TypeError("expected a 2-D uint16 / float16 array")
    return a


def round16(v, kind):
    lib = _load()
    lib.oracle_round16.restype = ctypes.c_float
    return float(lib.oracle_round16(ctypes.c_float(float(v)),
                                    ctypes.c_int(kind)))


def knn_op16(x_bits, y_bits, ptr_x, ptr_y, k, cosine=False, kind=0):
    """``torch_cluster::knn`` for fp16 / bf16 points as the GPU build computes
    it (c10::Half / c10::BFloat16 arithmetic); returns ([2, E], dist [E])."""
    lib = _load()
    if k > 100:
        raise RuntimeError("`k` needs to smaller than or equal to 100")
    x, y = _as_bits(x_bits), _as_bits(y_bits)
    ptr_x, ptr_y = _as_ptr(ptr_x), _as_ptr(ptr_y)
    nseg = 1 if ptr_x is None else ptr_x.size - 1
    m = y.shape[0]
    row = np.empty(m * k, dtype=np.int64)
    col = np.empty(m * k, dtype=np.int64)
    dist = np.empty(m * k, dtype=np.float32)
    rc = lib.oracle_knn_dense_16(
        _ptr(x), _ptr(y), _ptr(ptr_x), _ptr(ptr_y), ctypes.c_int64(x.shape[0]),
        ctypes.c_int64(m), ctypes.c_int64(x.shape[1]), ctypes.c_int64(nseg),
        ctypes.c_int64(k), ctypes.c_int(int(cosine)), ctypes.c_int(kind),
        _ptr(row), _ptr(col), _ptr(dist))
    if rc != 0:
        raise RuntimeError("oracle_knn_dense_16 failed")
    return _compact(row, col, col), dist[col != -1]


def radius_op16(x_bits, y_bits, ptr_x, ptr_y, r, max_num_neighbors,
                ignore_same_index=False, kind=0):
    """``torch_cluster::radius`` for fp16 / bf16 points."""
    lib = _load()
    x, y = _as_bits(x_bits), _as_bits(y_bits)
    ptr_x, ptr_y = _as_ptr(ptr_x), _as_ptr(ptr_y)
    nseg = 1 if ptr_x is None else ptr_x.size - 1
    m = y.shape[0]
    row = np.empty(m * max_num_neighbors, dtype=np.int64)
    col = np.empty(m * max_num_neighbors, dtype=np.int64)
    # (scalar_t)(r * r): double -> float -> 16 bits
    r2 = round16(np.float32(float(r) * float(r)), kind)
    rc = lib.oracle_radius_dense_16(
        _ptr(x), _ptr(y), _ptr(ptr_x), _ptr(ptr_y), ctypes.c_int64(x.shape[0]),
        ctypes.c_int64(m), ctypes.c_int64(x.shape[1]), ctypes.c_int64(nseg),
        ctypes.c_float(r2), ctypes.c_int64(max_num_neighbors),
        ctypes.c_int(int(ignore_same_index)), ctypes.c_int(kind), _ptr(row),
        _ptr(col))
    if rc != 0:
        raise RuntimeError("oracle_radius_dense_16 failed")
    return _compact(row, col, row)


# --------------------------------------------------------------------------
# nearest (csrc/cuda/nearest_cuda.cu, torch_cluster/nearest.py)
# --------------------------------------------------------------------------

def nearest_op(x, y, ptr_x, ptr_y, fma_mode=1):
    """``torch_cluster::nearest`` (csrc/cuda/nearest_cuda.cu:68-94): for every
    row of ``x`` the row of ``y`` of its example that is nearest.  ``x``/``y``
    float32 or float64 arrays, or uint16 / float16 arrays for IEEE half."""
    lib = _load()
    x, y = np.ascontiguousarray(x), np.ascontiguousarray(y)
    # x.view({x.size(0), -1}) (:76-77)
    x = x.reshape(x.shape[0], -1)
    y = y.reshape(y.shape[0], -1)
    if x.dtype != y.dtype or x.shape[1] != y.shape[1]:
        raise RuntimeError("Input mismatch")
    ptr_x, ptr_y = _as_ptr(ptr_x), _as_ptr(ptr_y)
    nseg = ptr_x.size - 1
    out = np.empty(x.shape[0], dtype=np.int64)
    if x.dtype == np.float16:
        x, y = x.view(np.uint16), y.view(np.uint16)
    if x.dtype == np.uint16:
        fn, mode = lib.oracle_nearest_16, 0
    elif x.dtype in _DTYPE_CODE:
        fn, mode = getattr(lib, "oracle_nearest_" + _suffix(x.dtype)), fma_mode
    else:
        raise TypeError(f"oracle nearest: unsupported dtype {x.dtype}")
    rc = fn(_ptr(x), _ptr(y), _ptr(ptr_x), _ptr(ptr_y),
            ctypes.c_int64(x.shape[0]), ctypes.c_int64(y.shape[0]),
            ctypes.c_int64(x.shape[1]), ctypes.c_int64(nseg),
            ctypes.c_int(int(mode)), _ptr(out))
    if rc != 0:
        raise RuntimeError("a row of x lies in no example of ptr_x")
    return out


def _counts_to_ptr(batch):
    """torch_cluster/nearest.py:57-63: scatter_add of ones, then cumsum."""
    batch = np.asarray(batch, dtype=np.int64)
    batch_size = int(batch.max()) + 1
    deg = np.bincount(batch, minlength=batch_size)
    return np.concatenate([[0], np.cumsum(deg)]).astype(np.int64)


def nearest(x, y, batch_x=None, batch_y=None, fma_mode=1):
    """The GPU branch of torch_cluster/nearest.py:7-91."""
    x, y = np.asarray(x), np.asarray(y)
    x = x.reshape(-1, 1) if x.ndim == 1 else x
    y = y.reshape(-1, 1) if y.ndim == 1 else y
    assert x.shape[1] == y.shape[1]
    if batch_x is not None and (np.diff(np.asarray(batch_x)) < 0).any():
        raise ValueError("'batch_x' is not sorted")
    if batch_y is not None and (np.diff(np.asarray(batch_y)) < 0).any():
        raise ValueError("'batch_y' is not sorted")
    if batch_x is not None:
        assert x.shape[0] == np.asarray(batch_x).size
        ptr_x = _counts_to_ptr(batch_x)
    else:
        ptr_x = np.array([0, x.shape[0]], dtype=np.int64)
    if batch_y is not None:
        assert y.shape[0] == np.asarray(batch_y).size
        ptr_y = _counts_to_ptr(batch_y)
    else:
        ptr_y = np.array([0, y.shape[0]], dtype=np.int64)
    # an example that is non-empty in x must be non-empty in y (:80-86);
    # torch.equal is False for different shapes
    nonempty_x = np.diff(ptr_x) > 0
    nonempty_y = np.diff(ptr_y) > 0
    if nonempty_x.shape != nonempty_y.shape or \
            not np.array_equal(nonempty_x, nonempty_y):
        raise ValueError("Some batch indices occur in 'batch_x' "
                         "that do not occur in 'batch_y'")
    return nearest_op(x, y, ptr_x, ptr_y, fma_mode)


# --------------------------------------------------------------------------
# fps (csrc/cuda/fps_cuda.cu, torch_cluster/fps.py)
# --------------------------------------------------------------------------

def fps_out_ptr(ptr, ratio, dtype):
    """csrc/cuda/fps_cuda.cu:80-83: samples per example = ceil(deg * ratio)
    evaluated in the ratio's element type (``dtype``), then the running sum
    with a leading zero.  ``ratio``: scalar or one value per example."""
    ptr = np.asarray(ptr, dtype=np.int64)
    deg = np.diff(ptr)
    ratio = np.asarray(ratio, dtype=dtype)
    with np.errstate(over="ignore"):
        per = np.ceil(deg.astype(dtype) * ratio).astype(np.int64)
    return np.concatenate([[0], np.cumsum(per)]).astype(np.int64)


def fps_op(src, ptr, ratio, start=None, fma_mode=1):
    """``torch_cluster::fps`` (csrc/cuda/fps_cuda.cu:68-109) with
    ``random_start=False``, or with the given start offsets per example.
    ``src`` float32 / float64 / float16 (or uint16 bit patterns of halves)."""
    lib = _load()
    src = np.ascontiguousarray(src)
    src = src.reshape(src.shape[0], -1)
    ptr = _as_ptr(ptr)
    nseg = ptr.size - 1
    if src.dtype == np.uint16:
        ratio_dtype = np.float16
    else:
        ratio_dtype = src.dtype
    out_ptr = fps_out_ptr(ptr, ratio, ratio_dtype)
    if start is None:
        start = np.zeros(nseg, dtype=np.int64)
    start = np.ascontiguousarray(start, dtype=np.int64)
    out = np.empty(int(out_ptr[-1]), dtype=np.int64)
    if src.dtype == np.float16:
        src = src.view(np.uint16)
    if src.dtype == np.uint16:
        fn, mode = lib.oracle_fps_16, 0
    elif src.dtype in _DTYPE_CODE:
        fn, mode = getattr(lib, "oracle_fps_" + _suffix(src.dtype)), fma_mode
    else:
        raise TypeError(f"oracle fps: unsupported dtype {src.dtype}")
    rc = fn(_ptr(src), _ptr(ptr), _ptr(out_ptr), _ptr(start),
            ctypes.c_int64(src.shape[0]), ctypes.c_int64(src.shape[1]),
            ctypes.c_int64(nseg), ctypes.c_int(int(mode)), _ptr(out))
    if rc != 0:
        raise RuntimeError("oracle_fps failed")
    return out


def fps(src, batch=None, ratio=None, random_start=True, batch_size=None,
        ptr=None, fma_mode=1):
    """torch_cluster/fps.py:35-108 (random_start must be False here: the
    reference draws its start rows from the device's generator)."""
    assert not random_start, "the oracle has no random start"
    src = np.asarray(src)
    if ratio is None:
        ratio = 0.5
    if ptr is not None:
        return fps_op(src, np.asarray(ptr), ratio, None, fma_mode)
    if batch is not None:
        batch = np.asarray(batch)
        assert src.shape[0] == batch.size
        if batch_size is None:
            batch_size = int(batch.max()) + 1
        deg = np.bincount(batch, minlength=batch_size)
        ptr_vec = np.concatenate([[0], np.cumsum(deg)]).astype(np.int64)
    else:
        ptr_vec = np.array([0, src.shape[0]], dtype=np.int64)
    return fps_op(src, ptr_vec, ratio, None, fma_mode)


# --------------------------------------------------------------------------
# Python entry points (torch_cluster/knn.py, torch_cluster/radius.py)
# --------------------------------------------------------------------------

def _prologue(x, y, batch_x, batch_y, batch_size):
    """torch_cluster/knn.py:58-79 == torch_cluster/radius.py:62-84."""
    x, y = np.asarray(x), np.asarray(y)
    x = x.reshape(-1, 1) if x.ndim == 1 else x
    y = y.reshape(-1, 1) if y.ndim == 1 else y
    if batch_size is None:
        batch_size = 1
        if batch_x is not None:
            assert x.shape[0] == np.asarray(batch_x).size
            batch_size = int(np.max(batch_x)) + 1
        if batch_y is not None:
            assert y.shape[0] == np.asarray(batch_y).size
            batch_size = max(batch_size, int(np.max(batch_y)) + 1)
    assert batch_size > 0
    ptr_x = ptr_y = None
    if batch_size > 1:
        assert batch_x is not None
        assert batch_y is not None
        arange = np.arange(batch_size + 1)
        # torch.bucketize(arange, batch) with right=False: first position i
        # with batch[i] >= value
        ptr_x = np.searchsorted(np.asarray(batch_x), arange, side="left")
        ptr_y = np.searchsorted(np.asarray(batch_y), arange, side="left")
    return x, y, ptr_x, ptr_y


def knn(x, y, k, batch_x=None, batch_y=None, cosine=False, num_workers=1,
        batch_size=None, fma_mode=1):
    """torch_cluster/knn.py:6-82."""
    if np.asarray(x).size == 0 or np.asarray(y).size == 0:
        return np.empty((2, 0), dtype=np.int64)
    x, y, ptr_x, ptr_y = _prologue(x, y, batch_x, batch_y, batch_size)
    return knn_op(x, y, ptr_x, ptr_y, k, cosine, num_workers, fma_mode)


def knn_graph(x, k, batch=None, loop=False, flow="source_to_target",
              cosine=False, num_workers=1, batch_size=None, fma_mode=1):
    """torch_cluster/knn.py:85-144."""
    assert flow in ["source_to_target", "target_to_source"]
    edge_index = knn(x, x, k if loop else k + 1, batch, batch, cosine,
                     num_workers, batch_size, fma_mode)
    if flow == "source_to_target":
        row, col = edge_index[1], edge_index[0]
    else:
        row, col = edge_index[0], edge_index[1]
    if not loop:
        mask = row != col
        row, col = row[mask], col[mask]
    return np.stack([row, col], axis=0)


def radius(x, y, r, batch_x=None, batch_y=None, max_num_neighbors=32,
           num_workers=1, batch_size=None, ignore_same_index=False,
           fma_mode=1):
    """torch_cluster/radius.py:6-88."""
    if np.asarray(x).size == 0 or np.asarray(y).size == 0:
        return np.empty((2, 0), dtype=np.int64)
    x, y, ptr_x, ptr_y = _prologue(x, y, batch_x, batch_y, batch_size)
    return radius_op(x, y, ptr_x, ptr_y, r, max_num_neighbors, num_workers,
                     ignore_same_index, fma_mode)


def radius_graph(x, r, batch=None, loop=False, max_num_neighbors=32,
                 flow="source_to_target", num_workers=1, batch_size=None,
                 fma_mode=1):
    """torch_cluster/radius.py:91-148."""
    assert flow in ["source_to_target", "target_to_source"]
    edge_index = radius(x, x, r, batch, batch, max_num_neighbors, num_workers,
                        batch_size, not loop, fma_mode)
    if flow == "source_to_target":
        row, col = edge_index[1], edge_index[0]
    else:
        row, col = edge_index[0], edge_index[1]
    return np.stack([row, col], axis=0)


# --------------------------------------------------------------------------
# The reference's own CPU operators (oracle/_ref)
# --------------------------------------------------------------------------

_ref = None


def have_ref():
    return os.path.exists(_REF_PATH)


def _load_ref():
    global _ref
    if _ref is None:
        import torch  # noqa: F401  (libref_cpu.so links libtorch_cpu)
        _ref = ctypes.CDLL(_REF_PATH)
        _ref.ref_knn_cpu.restype = ctypes.c_int64
        _ref.ref_radius_cpu.restype = ctypes.c_int64
    return _ref


def ref_knn(x, y, ptr_x, ptr_y, k):
    """csrc/cpu/knn_cpu.cpp:7-105 -> [2, E] int64 (row 0 = y, row 1 = x)."""
    lib = _load_ref()
    x, y = _as_points(x), _as_points(y)
    ptr_x, ptr_y = _as_ptr(ptr_x), _as_ptr(ptr_y)
    nseg = 0 if ptr_x is None else ptr_x.size - 1
    cap = y.shape[0] * k
    out = np.empty(2 * cap, dtype=np.int64)
    e = lib.ref_knn_cpu(_ptr(x), _ptr(y), _ptr(ptr_x), _ptr(ptr_y),
                        ctypes.c_int64(x.shape[0]), ctypes.c_int64(y.shape[0]),
                        ctypes.c_int64(x.shape[1]), ctypes.c_int64(nseg),
                        ctypes.c_int64(k), ctypes.c_int(_DTYPE_CODE[x.dtype]),
                        _ptr(out), ctypes.c_int64(cap))
    if e < 0:
        raise RuntimeError("reference knn_cpu raised")
    return out[:2 * e].reshape(2, e).copy()


def ref_radius(x, y, ptr_x, ptr_y, r, max_num_neighbors,
               ignore_same_index=False):
    """csrc/cpu/radius_cpu.cpp:7-117 -> [2, E] int64."""
    lib = _load_ref()
    x, y = _as_points(x), _as_points(y)
    ptr_x, ptr_y = _as_ptr(ptr_x), _as_ptr(ptr_y)
    nseg = 0 if ptr_x is None else ptr_x.size - 1
    cap = y.shape[0] * max_num_neighbors
    out = np.empty(2 * cap, dtype=np.int64)
    e = lib.ref_radius_cpu(_ptr(x), _ptr(y), _ptr(ptr_x), _ptr(ptr_y),
                           ctypes.c_int64(x.shape[0]),
                           ctypes.c_int64(y.shape[0]),
                           ctypes.c_int64(x.shape[1]), ctypes.c_int64(nseg),
                           ctypes.c_double(float(r)),
                           ctypes.c_int64(max_num_neighbors),
                           ctypes.c_int(int(ignore_same_index)),
                           ctypes.c_int(_DTYPE_CODE[x.dtype]), _ptr(out),
                           ctypes.c_int64(cap))
    if e < 0:
        raise RuntimeError("reference radius_cpu raised")
    return out[:2 * e].reshape(2, e).copy()


def ref_fps(src, ptr, ratio):
    """The reference's CPU operator ``fps_cpu`` (csrc/cpu/fps_cpu.cpp:13-68),
    first row of every example as start."""
    lib = _load_ref()
    src = _as_points(src)
    ptr = _as_ptr(ptr)
    out = np.empty(src.shape[0] + ptr.size, dtype=np.int64)
    lib.ref_fps_cpu.restype = ctypes.c_int64
    count = lib.ref_fps_cpu(_ptr(src), _ptr(ptr), ctypes.c_int64(src.shape[0]),
                            ctypes.c_int64(src.shape[1]),
                            ctypes.c_int64(ptr.size - 1),
                            ctypes.c_double(float(ratio)),
                            ctypes.c_int(_DTYPE_CODE[src.dtype]),
                            _ptr(out), ctypes.c_int64(out.size))
    if count < 0:
        raise RuntimeError("ref_fps_cpu failed")
    return out[:count].copy()
