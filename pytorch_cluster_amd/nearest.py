"""``nearest``: drop-in for ``torch_cluster.nearest`` on GPU tensors
(reference: ``torch_cluster/nearest.py:7-91``, the ``x.is_cuda`` branch).

Same signature, argument checks and errors.  The search itself is
``torch.ops.torch_cluster.nearest``, registered by this package's native
library; the reference's route for CPU tensors (scipy's ``vq``,
``torch_cluster/nearest.py:93-124``) has no counterpart here: the operator
rejects them ("No CPU version supported", as ``csrc/nearest.cpp:33``).
"""
from typing import Optional

import torch


def _pointers(batch: Optional[torch.Tensor], rows: torch.Tensor) -> torch.Tensor:
    """``[B + 1]`` CSR pointers of a sorted batch vector: counts per example,
    then their running sum (``torch_cluster/nearest.py:55-63``)."""
    if batch is None:
        return torch.tensor([0, rows.size(0)], device=rows.device)
    assert rows.size(0) == batch.numel()
    batch_size = int(batch.max()) + 1
    deg = rows.new_zeros(batch_size, dtype=torch.long)
    deg.scatter_add_(0, batch, torch.ones_like(batch))
    ptr = deg.new_zeros(batch_size + 1)
    torch.cumsum(deg, 0, out=ptr[1:])
    return ptr


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

    if batch_x is not None and (batch_x[1:] - batch_x[:-1] < 0).any():
        raise ValueError("'batch_x' is not sorted")
    if batch_y is not None and (batch_y[1:] - batch_y[:-1] < 0).any():
        raise ValueError("'batch_y' is not sorted")

    ptr_x = _pointers(batch_x, x)
    ptr_y = _pointers(batch_y, y)

    nonempty_x = (ptr_x[1:] - ptr_x[:-1]) > 0
    nonempty_y = (ptr_y[1:] - ptr_y[:-1]) > 0
    if not torch.equal(nonempty_x, nonempty_y):
        raise ValueError("Some batch indices occur in 'batch_x' "
                         "that do not occur in 'batch_y'")

    return torch.ops.torch_cluster.nearest(x, y, ptr_x, ptr_y)
