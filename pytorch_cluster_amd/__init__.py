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

__version__ = "0.1.0"

__all__ = ["knn", "knn_graph", "radius", "radius_graph", "nearest", "fps",
           "__version__"]
