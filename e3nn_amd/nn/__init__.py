from .edges import DstSortedEdges  # noqa: F401
