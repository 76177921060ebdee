"""Oracle: edge gather + destination scatter-sum.  TEST INFRASTRUCTURE ONLY.

Follows the three lines of the reference's message-passing step
(e3nn/nn/models/v2106/points_convolution.py:13-17 ``scatter`` and :105-106
``tp(node_features[edge_src], edge_attr, weight)`` then ``scatter(..., edge_dst, N)``).
"""
import numpy as np

from .tensor_product import tp_forward


def gather(node_x, edge_src):
    # torch advanced indexing: negative indices wrap, out-of-range raises
    edge_src = np.asarray(edge_src)
    n = node_x.shape[0]
    if edge_src.size and (edge_src.min() < -n or edge_src.max() >= n):
        raise IndexError("index out of range")
    return node_x[edge_src]


def scatter(src, index, dim_size):
    # zeros(dim_size, F).scatter_add_(0, index[:, None].expand_as(src), src); rows are
    # accumulated in edge order (np.add.at is sequential), nodes with no edge stay 0
    index = np.asarray(index)
    if index.size and (index.min() < 0 or index.max() >= dim_size):
        raise IndexError("index out of range")
    out = np.zeros((dim_size, src.shape[1]), dtype=src.dtype)
    np.add.at(out, index, src)
    return out


def tp_gather_scatter(spec, node_x, edge_attr, weight, edge_src, edge_dst, num_nodes, dtype=np.float64):
    msg = tp_forward(spec, gather(np.asarray(node_x, dtype=dtype), edge_src), edge_attr, weight, dtype=dtype)
    return scatter(msg, edge_dst, num_nodes)
