"""MI355X-native neighbour search behind the ``torch_cluster`` operator API.

``knn``, ``knn_graph``, ``radius``, ``radius_graph``, ``nearest`` and ``fps``
are drop-ins for the functions of the same name in ``torch_cluster``;
importing this package registers ``torch.ops.torch_cluster.knn`` / ``radius``
/ ``nearest`` / ``fps``.
"""
from . import _native  # noqa: F401  (loads the native libraries or raises)
from .fps import fps
from .knn import knn, knn_graph
from .nearest import nearest
from .radius import radius, radius_graph

import torch as _torch

__version__ = "0.1.0"


def set_search_strategy(name: str) -> None:
    """How ``knn`` / ``knn_graph`` (Euclidean, k <= 64) and ``radius`` /
    ``radius_graph`` (at most 64 neighbours per query) search fp32 points of
    up to 3 dimensions: ``"scan"`` looks at every row of the example,
    ``"binned"`` orders the rows along a space-filling curve first and looks
    only at rows near the query, ``"auto"`` (the default) bins when its
    estimate of the two costs says so (from some ten thousand rows per example
    on, unless the queries are few).  Same edges either way; binning wins on large
    examples.  Process-wide; the environment variable
    ``PCA_SEARCH_STRATEGY`` sets the initial value.  No counterpart in the
    reference."""
    _torch.ops.pytorch_cluster_amd.set_search_strategy(name)


def get_search_strategy() -> str:
    return _torch.ops.pytorch_cluster_amd.get_search_strategy()


__all__ = ["knn", "knn_graph", "radius", "radius_graph", "nearest", "fps",
           "set_search_strategy", "get_search_strategy", "__version__"]
