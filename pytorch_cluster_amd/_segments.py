"""Host-side prologue shared by ``knn`` and ``radius``.

The reference repeats this block in both wrappers
(``torch_cluster/knn.py:58-79``, ``torch_cluster/radius.py:62-84``): make the
point matrices 2-D and contiguous, find the number of examples, and turn the
sorted batch vectors into CSR pointers.  Everything here is
``torch.jit.script``-able.
"""
from typing import Optional, Tuple

import torch


def as_points(t: torch.Tensor) -> torch.Tensor:
    """``[N]`` -> ``[N, 1]``; returns a contiguous ``[N, F]`` matrix."""
    if t.dim() == 1:
        t = t.view(-1, 1)
    return t.contiguous()


def check_ids(x: torch.Tensor, y: torch.Tensor, batch_x: torch.Tensor,
              batch_y: torch.Tensor) -> None:
    """The size checks of the reference's wrappers
    (``torch_cluster/knn.py:66,71``)."""
    assert x.size(0) == batch_x.numel()
    assert y.size(0) == batch_y.numel()


def examples_or_unknown(batch_size: Optional[int]) -> int:
    """``batch_size`` for the operators that take example ids: -1 stands for
    "not known" (the operator then starts with the number of examples of the
    previous call and checks it against the ids on the device)."""
    if batch_size is None:
        return -1
    return batch_size


def num_examples(x: torch.Tensor, y: torch.Tensor,
                 batch_x: Optional[torch.Tensor],
                 batch_y: Optional[torch.Tensor],
                 batch_size: Optional[int]) -> int:
    """Number of examples B (CPU tensors, and GPU calls that go through
    pointers).  Without ``batch_size`` it is read from the LAST entry of each
    batch vector: the vectors must be sorted (as the reference requires,
    ``torch_cluster/knn.py:27-29``), so that is the largest -- one 8-byte read
    each instead of the reference's ``batch.max()`` reductions
    (``torch_cluster/knn.py:62-72``).  An unsorted vector is not detected."""
    if batch_size is not None:
        assert batch_size > 0
        return batch_size
    b = 1
    if batch_x is not None:
        assert x.size(0) == batch_x.numel()
        b = int(batch_x[-1]) + 1
    if batch_y is not None:
        assert y.size(0) == batch_y.numel()
        b = max(b, int(batch_y[-1]) + 1)
    assert b > 0
    return b


def segment_pointers(
    x: torch.Tensor, y: torch.Tensor, batch_x: Optional[torch.Tensor],
    batch_y: Optional[torch.Tensor], batch_size: Optional[int]
) -> Tuple[Optional[torch.Tensor], Optional[torch.Tensor]]:
    """CSR pointers ``[B + 1]`` of both sorted batch vectors, or
    ``(None, None)`` for a single example: ``ptr[b]`` is the first row whose
    example id is ``>= b`` (examples without rows get empty segments)."""
    b = num_examples(x, y, batch_x, batch_y, batch_size)
    if b <= 1:
        return None, None
    assert batch_x is not None
    assert batch_y is not None
    ids = torch.arange(b + 1, device=x.device)
    return torch.bucketize(ids, batch_x), torch.bucketize(ids, batch_y)


def graph_pointers(x: torch.Tensor, batch: Optional[torch.Tensor],
                   batch_size: Optional[int]) -> Optional[torch.Tensor]:
    """:func:`segment_pointers` of a graph entry point, where both sides are
    the same rows: one pointer array, computed once."""
    b = num_examples(x, x, batch, None, batch_size)
    if b <= 1:
        return None
    assert batch is not None
    return torch.bucketize(torch.arange(b + 1, device=x.device), batch)


def batch_pointers(rows: torch.Tensor, batch: torch.Tensor,
                   batch_size: Optional[int]) -> torch.Tensor:
    """CSR pointers ``[B + 1]`` of one sorted batch vector (always an array,
    also for a single example).  Without ``batch_size`` the number of examples
    is read from the vector's LAST entry (sorted: its largest), which is one
    8-byte read instead of a reduction over the vector."""
    assert rows.size(0) == batch.numel()
    b = batch_size
    if b is None:
        b = int(batch[-1]) + 1 if batch.numel() > 0 else 1
    return torch.bucketize(torch.arange(b + 1, device=rows.device), batch)
