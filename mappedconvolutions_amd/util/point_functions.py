"""k-nearest-neighbour wrapper (reference: layers/util/point_functions.py:7-18)."""
from .. import _C


def knn(ref, query, k):
    """ref [B, D, M], query [B, D, N] (points are columns), k neighbours.

    Returns (idx [B, k, N] int64, dist [B, k, N]): for each query the k nearest
    reference points, closest first.  Indices are 1-based (1..M), which is what
    the reference's kernel emits although its docstring says otherwise.
    """
    return _C.knn_forward(ref, query, k)
