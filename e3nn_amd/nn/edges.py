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

    def in_sorted_order(self, *edge_tensors):
        """Per-edge tensors ``[E, ...]`` rewritten in the order of the destination-sorted list (row ``k`` of a result is
        row ``perm[k]`` of the argument; differentiable).  Together with :meth:`sorted` this moves the permutation out
        of the message kernels: done once per graph for the edge attributes and the inputs of the radial network, every
        layer then produces and consumes its per-edge weights in the order the kernels walk them, a row's weights
        being one contiguous run instead of scattered rows."""
        if self.walk_perm is None:
            return edge_tensors if len(edge_tensors) != 1 else edge_tensors[0]
        out = tuple(t.index_select(0, self.perm) for t in edge_tensors)
        return out if len(out) != 1 else out[0]

    def sorted(self) -> "DstSortedEdges":
        """The same graph with its edge list held in destination order: edge ``k`` is edge ``perm[k]`` of this list, so
        the kernels read per-edge tensors by position.  Shares the row pointers, the row order and the source rows;
        nothing is sorted again.  Per-edge tensors go with it through :meth:`in_sorted_order`."""
        if self.walk_perm is None:
            return self
        if self._sorted is None:
            other = object.__new__(DstSortedEdges)
            other.__dict__.update(self.__dict__)
            src = self.src_rows if self.src_rows is not None else torch.where(self.edge_src < 0, self.edge_src + self.num_src_nodes, self.edge_src).index_select(0, self.perm).int()
            other.edge_src, other.edge_dst = src, self.edge_dst.index_select(0, self.perm)
            other._src_rows, other.walk_perm = src, None
            other.perm = torch.arange(self.num_edges, dtype=torch.int32, device=src.device)
            other._transposed, other._sorted = None, other
            self._sorted = other
        return self._sorted

    def __init__(self, edge_src: torch.Tensor, edge_dst: torch.Tensor, num_nodes: int, num_src_nodes: int = None,
                 locality_order="auto"):
        self._transposed = None
        self._sorted = None
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
            # A list that is already grouped by destination (what neighbour searches emit: torch_cluster's
            # radius_graph, which the reference's models call, returns its pairs sorted by the query node) is walked
            # by position: the stable sort is then the identity and the kernels are handed no permutation, so that
            # per-edge rows are read as one contiguous run per destination.
            self.walk_perm = self.perm
            if E > 1 and bool((self.edge_dst[1:] >= self.edge_dst[:-1]).all()):
                self.walk_perm = None
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

