"""Build-time helpers around the search path: data, graphs, sampling, router
construction, SVD and the recall metric.

These stand in for ``pilot_ann/utils`` of the reference.  The reference builds
its graphs with faiss (``pilot_ann/utils/graphs.py:15-20,52-56``), which is a
third-party dependency that is not part of the reference's sources; the
builders here produce the same *format* (padded CSR, ``-1`` fill, global ids,
empty rows for unsampled nodes) with their own construction, and every random
choice takes a seed.
"""
from .recall import recall
from .svd import svd
from .graphs import (knn_graph, graph_init, subgraph_init, graph_sampling,
                     connect_graph, reachable)
from .router import router_init
from .synth import gaussian_mixture, brute_force_topk
from .layout import locality_order
from .search import search_simple
from .loader import DataLoader

__all__ = [
    'recall', 'svd', 'knn_graph', 'graph_init', 'subgraph_init',
    'graph_sampling', 'connect_graph', 'reachable', 'router_init', 'gaussian_mixture', 'brute_force_topk',
    'locality_order', 'search_simple', 'DataLoader',
]
