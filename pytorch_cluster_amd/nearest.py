"""``nearest``: drop-in for ``torch_cluster.nearest``
(reference: ``torch_cluster/nearest.py:7-91``, the ``x.is_cuda`` branch).

Same signature, argument checks and errors.  The search itself is
``torch.ops.torch_cluster.nearest``, registered by this package's native
library.  CPU tensors take the same checks and the same operator, which
searches them on host threads with the result contract of the GPU kernel
(the reference normalises them per example and calls scipy's ``vq``,
``torch_cluster/nearest.py:93-124``; its operator rejects CPU tensors,
``csrc/nearest.cpp:33``).

The reference reads from the device five times before it calls the operator
(two sortedness tests, two ``batch.max()``, one comparison of the non-empty
examples).  Here the same facts come back in two reads: the last entries of
the batch vectors (their maxima if they are sorted) size the pointer arrays,
and one vector of three flags carries the outcome of all three checks.
"""
from typing import Optional

import torch


def _unsorted(batch: Optional[torch.Tensor], like: torch.Tensor) -> torch.Tensor:
    """0-d bool tensor: the batch vector decreases somewhere."""
    if batch is None or batch.numel() < 2:
        return torch.zeros((), dtype=torch.bool, device=like.device)
    return (batch[1:] < batch[:-1]).any()


def _pointers(batch: Optional[torch.Tensor], rows: torch.Tensor,
              batch_size: int) -> torch.Tensor:
    """``[B + 1]`` CSR pointers of a sorted batch vector: ``ptr[b]`` is the
    first row whose example id is ``>= b`` -- the running sum of the counts
    per example that the reference forms (``torch_cluster/nearest.py:55-63``)."""
    if batch is None:
        return torch.tensor([0, rows.size(0)], device=rows.device)
    ids = torch.arange(batch_size + 1, device=rows.device)
    return torch.bucketize(ids, batch)


def nearest(
    x: torch.Tensor,
    y: torch.Tensor,
    batch_x: Optional[torch.Tensor] = None,
    batch_y: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    r"""For each row of ``x`` the row of ``y`` of the same example that is
    nearest to it (squared Euclidean distance).

    Args:
        x: ``[N, F]`` rows to be assigned.
        y: ``[M, F]`` rows they are assigned to.
        batch_x: sorted ``[N]`` vector assigning each row of ``x`` to an
            example.
        batch_y: the same for ``y``; an example with rows in ``x`` must have
            rows in ``y``.

    Returns ``[N]`` int64 row numbers of ``y``.
    """
    x = x.view(-1, 1) if x.dim() == 1 else x
    y = y.view(-1, 1) if y.dim() == 1 else y
    assert x.size(1) == y.size(1)
    if batch_x is not None:
        assert x.size(0) == batch_x.numel()
    if batch_y is not None:
        assert y.size(0) == batch_y.numel()

    # first read: the number of examples on each side (the last entry of a
    # sorted vector is its maximum; if it is not sorted the check below fails
    # before the pointers are used)
    size_x, size_y = 1, 1
    lasts = []
    if batch_x is not None and batch_x.numel() > 0:
        lasts.append(batch_x[-1])
    if batch_y is not None and batch_y.numel() > 0:
        lasts.append(batch_y[-1])
    if len(lasts) > 0:
        values = torch.stack(lasts).tolist()
        if batch_x is not None and batch_x.numel() > 0:
            size_x = int(values[0]) + 1
        if batch_y is not None and batch_y.numel() > 0:
            size_y = int(values[-1]) + 1
    bad_sizes = size_x < 1 or size_y < 1

    ptr_x = _pointers(batch_x, x, max(size_x, 1))
    ptr_y = _pointers(batch_y, y, max(size_y, 1))

    # second read: the three checks of the reference, in its order
    if ptr_x.numel() == ptr_y.numel():
        mismatch = (((ptr_x[1:] - ptr_x[:-1]) > 0)
                    != ((ptr_y[1:] - ptr_y[:-1]) > 0)).any()
    else:
        mismatch = torch.ones((), dtype=torch.bool, device=x.device)
    flags = torch.stack([_unsorted(batch_x, x), _unsorted(batch_y, y),
                         mismatch]).tolist()
    if flags[0]:
        raise ValueError("'batch_x' is not sorted")
    if flags[1]:
        raise ValueError("'batch_y' is not sorted")
    if flags[2] or bad_sizes:
        raise ValueError("Some batch indices occur in 'batch_x' "
                         "that do not occur in 'batch_y'")

    return torch.ops.torch_cluster.nearest(x, y, ptr_x, ptr_y)
