"""Edge lists grouped by destination node, the preprocessing of the fused scatter-sum.

The message-passing step of the reference is
``scatter(tp(node_features[edge_src], edge_attr, weight), edge_dst, dim_size=N)``
(e3nn/nn/models/v2106/points_convolution.py:13-17,105-106).  The fused kernel needs the
edges of each destination to be contiguous: ``DstSortedEdges`` validates both index
arrays once and builds the row pointers and the stable permutation on the GPU.
"""
import ctypes
import os

import torch

from .. import _lib


class DstSortedEdges:
    """``edge_src[e] -> edge_dst[e]`` for ``e < E``, grouped by ``edge_dst``.

    ``edge_src`` indexes rows of the node-feature table like torch advanced indexing
    (values in ``[-num_src_nodes, num_src_nodes)``, negative ones wrap); ``edge_dst``
    follows ``scatter_add_`` (values in ``[0, num_nodes)``).  Out-of-range values raise
    ``IndexError``.  int32 and int64 indices give identical results.

    ``locality_order``: the fused kernel may walk the output rows in the order of their smallest source row, which
    puts rows with overlapping source sets next to each other (their gathers then hit L2) whatever the node
    numbering; the results do not change by a bit.  ``"auto"`` (default) keeps that order when the graph shows
    neighbourhood structure (``locality_score``: fraction of rows that agree with their successor in their two
    smallest sources, at least 2 %), ``True`` / ``False`` force it on / off.
    """

    def transposed(self) -> "DstSortedEdges":
        """The same edges with source and destination exchanged (grouped by ``edge_src``); the backward
        pass with respect to the node features scatters onto the sources.  Built once, cached."""
        if self._transposed is None:
            # the sources become scatter destinations, which do not wrap: negative source indices (valid for the
            # gather, like torch advanced indexing) are normalised first
            src = torch.where(self.edge_src < 0, self.edge_src + self.num_src_nodes, self.edge_src)
            self._transposed = DstSortedEdges(self.edge_dst, src, self.num_src_nodes, self.num_nodes, self._locality_order)
            self._transposed._transposed = self
        return self._transposed

    @property
    def src_rows(self) -> torch.Tensor:
        """``edge_src`` in the order of the destination-sorted list (int32, negative values wrapped): the fused
        kernels read it sequentially, where ``edge_src[perm[k]]`` costs them a cache line per edge.  Built on first
        use, once per graph."""
        if self._src_rows is None and self.num_edges > 0 and os.environ.get("E3X_SRC_ROWS", "1") != "0":
            dev = self.edge_src.device
            rows = torch.empty(self.num_edges, dtype=torch.int32, device=dev)
            with torch.cuda.device(dev):
                _lib.check(
                    _lib.lib().e3x_src_rows_build(
                        _lib.ptr(self.edge_src), self.edge_src.element_size() * 8, _lib.ptr(self.perm), self.num_edges,
                        self.num_src_nodes, _lib.ptr(rows), _lib.stream_ptr(dev),
                    )  # fmt: skip
                )
            self._src_rows = rows
        return self._src_rows

    def __init__(self, edge_src: torch.Tensor, edge_dst: torch.Tensor, num_nodes: int, num_src_nodes: int = None,
                 locality_order="auto"):
        self._transposed = None
        self._src_rows = None
        self._locality_order = locality_order
        if not (edge_src.is_cuda and edge_dst.is_cuda):
            raise RuntimeError("DstSortedEdges needs index tensors on the GPU")
        if edge_src.dtype not in (torch.int32, torch.int64) or edge_dst.dtype not in (torch.int32, torch.int64):
            raise TypeError("edge indices must be int32 or int64")
        if edge_src.ndim != 1 or edge_src.shape != edge_dst.shape:
            raise ValueError("edge_src and edge_dst must be 1-D tensors of the same length")
        self.num_nodes = int(num_nodes)
        self.num_src_nodes = int(num_nodes if num_src_nodes is None else num_src_nodes)
        self.edge_src = edge_src.contiguous()
        self.edge_dst = edge_dst.contiguous()
        self.num_edges = E = edge_src.numel()
        dev = edge_src.device
        L = _lib.lib()
        with torch.cuda.device(dev):
            st = _lib.stream_ptr(dev)
            _lib.check(L.e3x_index_check(_lib.ptr(self.edge_src), self.edge_src.element_size() * 8, E, self.num_src_nodes, st))
            self.rowptr = torch.empty(self.num_nodes + 1, dtype=torch.int32, device=dev)
            self.perm = torch.empty(E, dtype=torch.int32, device=dev)
            ws_bytes = L.e3x_csr_workspace_bytes(E, self.num_nodes)
            ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
            _lib.check(
                L.e3x_csr_build(
                    _lib.ptr(self.edge_dst), self.edge_dst.element_size() * 8, E, self.num_nodes, _lib.ptr(self.rowptr),
                    _lib.ptr(self.perm), _lib.ptr(ws), ws_bytes, st,
                )  # fmt: skip
            )
            # rows that share their smallest source are processed next to each other (they share most of their
            # sources, which then sit in L2): locality taken from the graph, not from the caller's node numbering
            self.row_order = None
            if locality_order and self.num_nodes > 0:
                self.row_order = torch.empty(self.num_nodes, dtype=torch.int32, device=dev)
                ws_bytes = L.e3x_row_order_workspace_bytes(self.num_nodes)
                ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
                pairs = ctypes.c_int32(0)
                _lib.check(
                    L.e3x_row_order_build(
                        _lib.ptr(self.edge_src), self.edge_src.element_size() * 8, _lib.ptr(self.rowptr), _lib.ptr(self.perm),
                        E, self.num_nodes, self.num_src_nodes, _lib.ptr(self.row_order), ctypes.byref(pairs), _lib.ptr(ws),
                        ws_bytes, st,
                    )  # fmt: skip
                )
                # rows that follow each other in the order and agree in their two smallest sources: next to nothing
                # on a graph without neighbourhood structure, where the order would only scatter the rows
                self.locality_score = pairs.value / self.num_nodes
                if locality_order == "auto" and self.locality_score < 0.02:
                    self.row_order = None

