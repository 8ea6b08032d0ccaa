"""ctypes binding of the C ABI (``include/pca_neighbors.h``) for torch tensors.

The TorchScript operators go through the same entry points from C++; this
module lets Python call them directly -- with the per-edge distances, on an
explicit stream, or without the final host read of the edge count.
"""
import ctypes
from typing import Optional, Tuple

import torch

from ._native import (PCA_BF16, PCA_EDGES_DROP_SELF, PCA_EDGES_X_FIRST, PCA_F16,
                      PCA_SEGMENTS_BY_ID,
                      PCA_F32, PCA_F64, capi)

_DTYPE_CODE = {torch.float32: PCA_F32, torch.float64: PCA_F64,
               torch.float16: PCA_F16, torch.bfloat16: PCA_BF16}


class PcaError(RuntimeError):
    def __init__(self, status: int):
        detail = capi.pca_last_error().decode()
        text = detail or capi.pca_status_string(status).decode()
        super().__init__(text)
        self.status = status


def _check(status: int):
    if status != 0:
        raise PcaError(status)


def _dev_ptr(t: Optional[torch.Tensor]):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _stream_handle(stream: Optional[torch.cuda.Stream], device):
    s = stream if stream is not None else torch.cuda.current_stream(device)
    return ctypes.c_void_p(s.cuda_stream)


def _segments(ptr_x, ptr_y, ids_examples: int = 0):
    """(ptr_x, ptr_y, number of segments); with ``ids_examples`` > 0 the two
    tensors are the rows' sorted example ids (``PCA_SEGMENTS_BY_ID``)."""
    if ptr_x is None and ptr_y is None:
        return None, None, 1
    assert ptr_x is not None and ptr_y is not None
    assert ptr_x.dtype == torch.long and ptr_y.dtype == torch.long
    assert ptr_x.is_contiguous() and ptr_y.is_contiguous()
    if ids_examples > 0:
        return ptr_x, ptr_y, ids_examples
    assert ptr_x.numel() == ptr_y.numel()
    return ptr_x, ptr_y, ptr_x.numel() - 1


def _edge_flags(drop_self: bool, x_first: bool, by_id: bool = False) -> int:
    return ((PCA_EDGES_DROP_SELF if drop_self else 0)
            | (PCA_EDGES_X_FIRST if x_first else 0)
            | (PCA_SEGMENTS_BY_ID if by_id else 0))


def segment_pointers(ids_x, ids_y, num_segments: int, stream=None):
    """``pca_segment_pointers``: (ptr_x, ptr_y), ``num_segments + 1`` entries
    each, of two sorted example-id vectors."""
    assert ids_x.is_cuda and ids_x.dtype == torch.long
    assert ids_y.is_cuda and ids_y.dtype == torch.long
    ptr_x = torch.empty(num_segments + 1, dtype=torch.long,
                        device=ids_x.device)
    ptr_y = torch.empty_like(ptr_x)
    _check(capi.pca_segment_pointers(
        _dev_ptr(ids_x), ids_x.numel(), _dev_ptr(ids_y), ids_y.numel(),
        num_segments, _dev_ptr(ptr_x), _dev_ptr(ptr_y),
        _stream_handle(stream, ids_x.device)))
    return ptr_x, ptr_y


def knn_launch(x, y, ptr_x, ptr_y, k: int, cosine: bool = False,
               want_dist: bool = False, stream=None, drop_self: bool = False,
               x_first: bool = False, binned: bool = False,
               fixed_scratch: bool = False, ids_examples: int = 0):
    """Queues ``pca_knn`` (``binned``: ``pca_knn_binned``; ``fixed_scratch``:
    ``pca_knn_fixed_scratch``, no workspace); returns (edges buffer [2*m*k],
    num_edges [1] on the device, dist buffer or None, workspace or None).
    ``ids_examples`` > 0: ``ptr_x`` / ``ptr_y`` are the rows' sorted example
    ids, that many examples.  Nothing is synchronised."""
    assert x.is_cuda and y.is_cuda and x.is_contiguous() and y.is_contiguous()
    assert x.dtype == y.dtype and x.dtype in _DTYPE_CODE
    dtype = _DTYPE_CODE[x.dtype]
    n, d = x.shape
    m = y.shape[0]
    ptr_x, ptr_y, nseg = _segments(ptr_x, ptr_y, ids_examples)
    by_id = ids_examples > 0
    assert not (by_id and binned)
    edges = torch.empty(max(2 * m * max(k, 0), 1), dtype=torch.long,
                        device=x.device)
    num_edges = torch.empty(1, dtype=torch.long, device=x.device)
    dist = (torch.empty(max(m * max(k, 0), 1), dtype=torch.float32,
                        device=x.device) if want_dist else None)
    if fixed_scratch:
        assert not binned
        _check(capi.pca_knn_fixed_scratch(
            _dev_ptr(x), _dev_ptr(y), _dev_ptr(ptr_x), _dev_ptr(ptr_y), n, m,
            d, nseg, k, int(cosine), dtype,
            _edge_flags(drop_self, x_first, by_id),
            _dev_ptr(edges), _dev_ptr(num_edges), _dev_ptr(dist),
            _stream_handle(stream, x.device)))
        return edges, num_edges, dist, None
    if binned:
        assert dtype == 0 and not cosine
        ws_bytes = capi.pca_knn_binned_workspace_bytes(n, m, d, nseg, k)
    else:
        ws_bytes = capi.pca_knn_workspace_bytes(n, m, d, nseg, k, dtype)
    if ws_bytes == 0:
        # let the entry point produce the precise error
        ws_bytes = 256
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device)
    if binned:
        _check(capi.pca_knn_binned(_dev_ptr(x), _dev_ptr(y), _dev_ptr(ptr_x),
                                   _dev_ptr(ptr_y), n, m, d, nseg, k,
                                   _edge_flags(drop_self, x_first),
                                   _dev_ptr(edges), _dev_ptr(num_edges),
                                   _dev_ptr(dist), _dev_ptr(ws), ws_bytes,
                                   _stream_handle(stream, x.device)))
        return edges, num_edges, dist, ws
    _check(capi.pca_knn(_dev_ptr(x), _dev_ptr(y), _dev_ptr(ptr_x),
                        _dev_ptr(ptr_y), n, m, d, nseg, k, int(cosine),
                        dtype, _edge_flags(drop_self, x_first, by_id),
                        _dev_ptr(edges), _dev_ptr(num_edges),
                        _dev_ptr(dist), _dev_ptr(ws), ws_bytes,
                        _stream_handle(stream, x.device)))
    return edges, num_edges, dist, ws


def knn_edges(x, y, ptr_x=None, ptr_y=None, k: int = 1, cosine: bool = False,
              want_dist: bool = False, stream=None, drop_self: bool = False,
              x_first: bool = False, binned: bool = False,
              fixed_scratch: bool = False, ids_examples: int = 0
              ) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """``[2, E]`` edges (and the ``[E]`` distances when asked for)."""
    edges, num_edges, dist, _ws = knn_launch(x, y, ptr_x, ptr_y, k, cosine,
                                             want_dist, stream, drop_self,
                                             x_first, binned, fixed_scratch,
                                             ids_examples)
    e = int(num_edges.item())
    out = edges[:2 * e].view(2, e)
    return out, (dist[:e] if dist is not None else None)


def radius_launch(x, y, ptr_x, ptr_y, r: float, max_num_neighbors: int,
                  ignore_same_index: bool = False, stream=None,
                  x_first: bool = False, binned: bool = False,
                  ids_examples: int = 0):
    assert x.is_cuda and y.is_cuda and x.is_contiguous() and y.is_contiguous()
    assert x.dtype == y.dtype and x.dtype in _DTYPE_CODE
    dtype = _DTYPE_CODE[x.dtype]
    n, d = x.shape
    m = y.shape[0]
    ptr_x, ptr_y, nseg = _segments(ptr_x, ptr_y, ids_examples)
    by_id = ids_examples > 0
    assert not (by_id and binned)
    if binned:
        assert dtype == 0
        ws_bytes = capi.pca_radius_binned_workspace_bytes(
            n, m, d, nseg, max_num_neighbors)
    else:
        ws_bytes = capi.pca_radius_workspace_bytes(n, m, d, nseg,
                                                   max_num_neighbors, dtype)
    if ws_bytes == 0:
        ws_bytes = 256
    slots = capi.pca_radius_slots(n, max_num_neighbors)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device)
    edges = torch.empty(max(2 * m * slots, 1), dtype=torch.long,
                        device=x.device)
    num_edges = torch.empty(1, dtype=torch.long, device=x.device)
    if binned:
        _check(capi.pca_radius_binned(
            _dev_ptr(x), _dev_ptr(y), _dev_ptr(ptr_x), _dev_ptr(ptr_y), n, m,
            d, nseg, float(r), max_num_neighbors, int(ignore_same_index),
            _edge_flags(False, x_first), _dev_ptr(edges), _dev_ptr(num_edges),
            _dev_ptr(ws), ws_bytes, _stream_handle(stream, x.device)))
        return edges, num_edges, ws
    _check(capi.pca_radius(_dev_ptr(x), _dev_ptr(y), _dev_ptr(ptr_x),
                           _dev_ptr(ptr_y), n, m, d, nseg, float(r),
                           max_num_neighbors, int(ignore_same_index), dtype,
                           _edge_flags(False, x_first, by_id),
                           _dev_ptr(edges), _dev_ptr(num_edges), _dev_ptr(ws),
                           ws_bytes, _stream_handle(stream, x.device)))
    return edges, num_edges, ws


def radius_edges(x, y, ptr_x=None, ptr_y=None, r: float = 1.0,
                 max_num_neighbors: int = 32, ignore_same_index: bool = False,
                 stream=None, x_first: bool = False,
                 binned: bool = False, ids_examples: int = 0) -> torch.Tensor:
    edges, num_edges, _ws = radius_launch(x, y, ptr_x, ptr_y, r,
                                          max_num_neighbors,
                                          ignore_same_index, stream, x_first,
                                          binned, ids_examples)
    e = int(num_edges.item())
    return edges[:2 * e].view(2, e)


def nearest_launch(x, y, ptr_x=None, ptr_y=None, stream=None,
                   binned: bool = False):
    """Queues ``pca_nearest``: for every row of ``x`` the nearest row of ``y``
    of the same segment.  Returns (out [n] int64, workspace); nothing is
    synchronised."""
    assert x.is_cuda and y.is_cuda and x.is_contiguous() and y.is_contiguous()
    assert x.dtype == y.dtype and x.dtype in _DTYPE_CODE
    dtype = _DTYPE_CODE[x.dtype]
    n, d = x.shape
    m = y.shape[0]
    ptr_x, ptr_y, nseg = _segments(ptr_x, ptr_y)
    if binned:
        assert dtype == 0
        ws_bytes = capi.pca_nearest_binned_workspace_bytes(n, m, d, nseg)
    else:
        ws_bytes = capi.pca_nearest_workspace_bytes(n, m, d, nseg, dtype)
    if ws_bytes == 0:
        ws_bytes = 256
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device)
    out = torch.empty(n, dtype=torch.long, device=x.device)
    if binned:
        _check(capi.pca_nearest_binned(
            _dev_ptr(x), _dev_ptr(y), _dev_ptr(ptr_x), _dev_ptr(ptr_y), n, m,
            d, nseg, _dev_ptr(out), _dev_ptr(ws), ws_bytes,
            _stream_handle(stream, x.device)))
        return out, ws
    _check(capi.pca_nearest(_dev_ptr(x), _dev_ptr(y), _dev_ptr(ptr_x),
                            _dev_ptr(ptr_y), n, m, d, nseg, dtype,
                            _dev_ptr(out), _dev_ptr(ws), ws_bytes,
                            _stream_handle(stream, x.device)))
    return out, ws


def nearest_rows(x, y, ptr_x=None, ptr_y=None, stream=None,
                 binned: bool = False) -> torch.Tensor:
    return nearest_launch(x, y, ptr_x, ptr_y, stream, binned)[0]


def fps_launch(src, ptr, out_ptr, num_samples: int, start=None,
               max_segment_rows: int = 0, stream=None):
    """Queues ``pca_fps``.  ``out_ptr``: int64 ``[B + 1]`` output positions on
    the device, ``num_samples`` = its last entry (known to the caller).
    Returns (out [num_samples] int64, workspace); nothing is synchronised."""
    assert src.is_cuda and src.is_contiguous() and src.dtype in _DTYPE_CODE
    assert ptr.dtype == torch.long and out_ptr.dtype == torch.long
    dtype = _DTYPE_CODE[src.dtype]
    n, d = src.shape
    nseg = ptr.numel() - 1
    ws_bytes = capi.pca_fps_workspace_bytes(n, d, nseg, max_segment_rows,
                                            dtype)
    if ws_bytes == 0:
        ws_bytes = 256
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=src.device)
    out = torch.empty(num_samples, dtype=torch.long, device=src.device)
    _check(capi.pca_fps(_dev_ptr(src), _dev_ptr(ptr), _dev_ptr(out_ptr),
                        _dev_ptr(start), n, d, nseg, max_segment_rows, dtype,
                        _dev_ptr(out), _dev_ptr(ws), ws_bytes,
                        _stream_handle(stream, src.device)))
    return out, ws
