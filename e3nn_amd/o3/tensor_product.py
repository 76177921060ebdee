"""Tensor product with parametrised paths, evaluated by instruction-set-specialised HIP kernels.

Public behaviour of the reference's ``e3nn.o3.TensorProduct``
(e3nn/o3/_tensor_product/_tensor_product.py:196-609) and
``e3nn.o3.FullyConnectedTensorProduct`` (e3nn/o3/_tensor_product/_sub.py:10-68) for the
``uvu`` and ``uvw`` connection modes: constructor arguments, normalisation of the path
weights, weight bookkeeping, ``output_mask``, ``forward`` with broadcasting of the batch
dimensions, weight views.  Where the reference generates an fx graph of einsums per
instruction set (``_codegen.py:24-395``), this module asks the C library for a plan: one
fused kernel specialised to the instruction set.

``forward_gather_scatter`` is additive: the message-passing step
``scatter(tp(x[edge_src], edge_attr, w), edge_dst, N)`` in one kernel.
"""
import ctypes
import warnings
from collections import namedtuple
from math import prod, sqrt
from typing import List, Optional, Union

import torch

from .. import _lib, get_optimization_defaults
from .irreps import Irreps

Instruction = namedtuple(
    "Instruction", ["i_in1", "i_in2", "i_out", "connection_mode", "has_weight", "path_weight", "path_shape"]
)

_MODES = ["uvw", "uvu", "uvv", "uuw", "uuu", "uvuv", "uvu<v", "u<vw"]
_KERNEL_MODES = {"uvw": 0, "uvu": 1, "uvv": 2, "uuw": 3, "uuu": 4, "uvuv": 5, "uvu<v": 6, "u<vw": 7}  # E3X_MODE_*
_DTYPES = {torch.float32: _lib.F32, torch.bfloat16: _lib.BF16}


def _path_shape(mode, m1, m2, mo):
    return {
        "uvw": (m1, m2, mo),
        "uvu": (m1, m2),
        "uvv": (m1, m2),
        "uuw": (m1, mo),
        "uuu": (m1,),
        "uvuv": (m1, m2),
        "uvu<v": (m1 * (m2 - 1) // 2,),
        "u<vw": (m1 * (m2 - 1) // 2, mo),
    }[mode]


def _num_elements(mode, m1, m2):
    return {
        "uvw": m1 * m2,
        "uvu": m2,
        "uvv": m1,
        "uuw": m1,
        "uuu": 1,
        "uvuv": 1,
        "uvu<v": 1,
        "u<vw": m1 * (m2 - 1) // 2,
    }[mode]


class _Plan:
    """Owner of one ``e3x_plan`` handle: a fused kernel specialised to one instruction set."""

    def __init__(self, irreps_in1, irreps_in2, irreps_out, instructions, shared_weights: bool, dtype: torch.dtype):
        """``instructions``: tuples ``(i_in1, i_in2, i_out, mode, has_weight, path_weight)``, path weights final."""
        L = _lib.lib()
        mk = lambda irreps: (_lib.Irrep * max(1, len(irreps)))(*[_lib.Irrep(mul, ir.l, ir.p) for mul, ir in irreps])  # noqa: E731
        in1, in2, out = mk(irreps_in1), mk(irreps_in2), mk(irreps_out)
        ins = (_lib.Instruction * max(1, len(instructions)))(
            *[_lib.Instruction(a, b, c, _KERNEL_MODES[mode], int(hw), pw) for a, b, c, mode, hw, pw in instructions]
        )
        desc = _lib.TpDesc(
            len(irreps_in1), len(irreps_in2), len(irreps_out), len(instructions), in1, in2, out, ins,
            int(shared_weights), _DTYPES[dtype],
        )  # fmt: skip
        handle = _lib.c_void_p()
        _lib.check(L.e3x_tp_plan_create(ctypes.byref(desc), ctypes.byref(handle)))
        self.handle = handle
        self.shared_weights = bool(shared_weights)
        wn, fam, key = ctypes.c_int64(), ctypes.c_char_p(), ctypes.c_char_p()
        _lib.check(L.e3x_tp_plan_info(handle, ctypes.byref(wn), None, None, None, ctypes.byref(fam), ctypes.byref(key)))
        self.weight_numel, self.family, self.key = wn.value, fam.value.decode(), key.value.decode()
        self.out_dim, self.in2_dim = irreps_out.dim, irreps_in2.dim
        self.arithmetic = L.e3x_tp_plan_arithmetic(handle, 0).decode()  # which instruction forms the products
        self._fused_grad_w = None  # whether the plan has the message-step backward kernel; asked on first use

    def __del__(self):
        try:
            if self.handle:
                _lib.lib().e3x_tp_plan_destroy(self.handle)
                self.handle = None
        except Exception:
            pass

    def forward(self, x1, x2, w):
        Z = x1.shape[0]
        out = torch.empty(Z, self.out_dim, dtype=x1.dtype, device=x1.device)
        ws_bytes = _lib.lib().e3x_tp_forward_workspace_bytes(self.handle)
        ws = None
        if ws_bytes:
            # scratch for the weights repacked for the matrix cores; the kernel reads rows with 16-byte loads
            ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x1.device)
            x1, x2 = (t if t.data_ptr() % 16 == 0 else t.clone() for t in (x1, x2))
        if self.family == "uvw_node":
            # rows and weights are read with 16-byte loads
            x1, w = (t if t.data_ptr() % 16 == 0 else t.clone() for t in (x1, w))
        with torch.cuda.device(x1.device):
            _lib.check(
                _lib.lib().e3x_tp_forward_ws(
                    self.handle, _lib.ptr(x1), _lib.ptr(x2), _lib.ptr(w), _lib.ptr(out), Z,
                    _lib.ptr(ws) if ws is not None else None, ws_bytes, _lib.stream_ptr(x1.device),
                )
            )
        return out

    def gather_scatter(self, table, edge_attr, w, gather_idx, edges, num_table_rows):
        """``out[n] = sum_{e: edges groups e under n} TP(table[gather_idx[e]], edge_attr[e], w[e])``."""
        out = torch.empty(edges.num_nodes, self.out_dim, dtype=table.dtype, device=table.device)
        L = _lib.lib()
        with torch.cuda.device(table.device):
            # scratch of the matrix-core message kernel (the node table in operand order); 0 for every other plan
            ws_bytes = L.e3x_tp_gather_scatter_workspace_bytes(self.handle, num_table_rows)
            ws = torch.empty(ws_bytes, dtype=torch.uint8, device=table.device) if ws_bytes else None
            _lib.check(
                L.e3x_tp_gather_scatter_ws(
                    self.handle, _lib.ptr(table), _lib.ptr(edge_attr), _lib.ptr(w), _lib.ptr(gather_idx),
                    gather_idx.element_size() * 8, _lib.ptr(edges.rowptr), _lib.ptr(edges.walk_perm), _lib.ptr(edges.row_order),
                    _lib.ptr(edges.src_rows if gather_idx is edges.edge_src else None),
                    _lib.ptr(out), edges.num_edges, num_table_rows, edges.num_nodes, _lib.ptr(ws), ws_bytes,
                    _lib.stream_ptr(table.device),
                )  # fmt: skip
            )
        return out

    def gather_scatter_sh(self, table, edge_vec, w, gather_idx, edges, num_table_rows, normalize, normalization):
        """``gather_scatter`` with ``edge_attr`` = the spherical harmonics of ``edge_vec[E, 3]``, formed in the kernel;
        None when the plan's second input is not ``0e + 1o + ...`` up to ``l <= 3``."""
        L = _lib.lib()
        rc = L.e3x_tp_plan_prepare_gather_scatter_sh(self.handle, int(bool(normalize)), normalization)
        if rc == _lib.ERR_INVALID:
            return None
        _lib.check(rc)
        out = torch.empty(edges.num_nodes, self.out_dim, dtype=table.dtype, device=table.device)
        with torch.cuda.device(table.device):
            _lib.check(
                L.e3x_tp_gather_scatter_sh(
                    self.handle, _lib.ptr(table), _lib.ptr(edge_vec), _lib.ptr(w), _lib.ptr(gather_idx),
                    gather_idx.element_size() * 8, _lib.ptr(edges.rowptr), _lib.ptr(edges.walk_perm), _lib.ptr(edges.row_order),
                    _lib.ptr(edges.src_rows if gather_idx is edges.edge_src else None),
                    _lib.ptr(out), edges.num_edges, num_table_rows, edges.num_nodes, int(bool(normalize)), normalization,
                    _lib.stream_ptr(table.device),
                )  # fmt: skip
            )
        return out

    def gather_scatter_grad_w(self, table, edge_attr, w, row_x, gather_idx, edges, want_x2=False):
        """On the transposed plan of a message step: ``(gather_scatter(table, ...), grad_w[E, weight_numel],
        grad_edge_attr or None)`` from one kernel, ``row_x`` being the forward input rows of the nodes that ``edges``
        groups by; None when the plan does not fit that kernel."""
        L = _lib.lib()
        if self._fused_grad_w is None:
            rc = L.e3x_tp_plan_prepare_gather_scatter_grad_w(self.handle)
            if rc != _lib.ERR_INVALID:
                _lib.check(rc)
            self._fused_grad_w = rc != _lib.ERR_INVALID
        if not self._fused_grad_w:
            return None
        out = torch.empty(edges.num_nodes, self.out_dim, dtype=table.dtype, device=table.device)
        grad_w = torch.empty(edges.num_edges, self.weight_numel, dtype=table.dtype, device=table.device)
        grad_x2 = torch.empty_like(edge_attr) if want_x2 else None
        with torch.cuda.device(table.device):
            _lib.check(
                L.e3x_tp_gather_scatter_grad_w(
                    self.handle, _lib.ptr(table), _lib.ptr(edge_attr), _lib.ptr(w), _lib.ptr(row_x), _lib.ptr(gather_idx),
                    gather_idx.element_size() * 8, _lib.ptr(edges.rowptr), _lib.ptr(edges.walk_perm), _lib.ptr(edges.row_order),
                    _lib.ptr(edges.src_rows if gather_idx is edges.edge_src else None),
                    _lib.ptr(out), _lib.ptr(grad_w), _lib.ptr(grad_x2), edges.num_edges, table.shape[0], edges.num_nodes,
                    _lib.stream_ptr(table.device),
                )  # fmt: skip
            )
        return out, grad_w, grad_x2

    def gather_scatter_radial(self, table, edge_attr, edge_scalars, w1, w2, act_kind, act_cst, variance_in, variance_out,
                              gather_idx, edges, num_table_rows):
        """``gather_scatter`` with the per-edge weights computed in the kernel by the two-layer network
        ``(edge_scalars, w1, w2)``; returns None when the library does not take this instruction set or network."""
        out = torch.empty(edges.num_nodes, self.out_dim, dtype=table.dtype, device=table.device)
        with torch.cuda.device(table.device):
            rc = _lib.lib().e3x_tp_gather_scatter_radial(
                self.handle, _lib.ptr(table), _lib.ptr(edge_attr), _lib.ptr(edge_scalars), _lib.ptr(w1), _lib.ptr(w2),
                w1.shape[0], w1.shape[1], act_kind, act_cst, float(variance_in), float(variance_out), _lib.ptr(gather_idx),
                gather_idx.element_size() * 8, _lib.ptr(edges.rowptr), _lib.ptr(edges.walk_perm), _lib.ptr(out), edges.num_edges,
                num_table_rows, edges.num_nodes, _lib.stream_ptr(table.device),
            )  # fmt: skip
        if rc == _lib.ERR_INVALID:
            return None
        _lib.check(rc)
        return out

    @property
    def arithmetic_weight_gradient(self):
        """Instruction of the matrix-core ``uvw`` weight gradient; "" before that kernel has been built."""
        return _lib.lib().e3x_tp_plan_arithmetic(self.handle, 1).decode()

    def backward_w_uvw(self, x1, x2, grad_out, shared_weights):
        shape = (self.weight_numel,) if shared_weights else (x1.shape[0], self.weight_numel)
        gw = torch.empty(shape, dtype=x1.dtype, device=x1.device)
        # the matrix-core kernel reads rows with 16-byte loads
        x1, x2, grad_out = (t if t.data_ptr() % 16 == 0 else t.clone() for t in (x1, x2, grad_out))
        with torch.cuda.device(x1.device):
            _lib.check(
                _lib.lib().e3x_tp_backward_w_uvw(
                    self.handle, _lib.ptr(x1), _lib.ptr(x2), _lib.ptr(grad_out), _lib.ptr(gw), x1.shape[0],
                    _lib.stream_ptr(x1.device),
                )
            )
        return gw

    def backward_w_x2(self, x1, x2, w, grad_out, src, dst, want_w, want_x2, num_edges):
        """``x2`` may be None when only ``want_x2`` is set (the weight gradient alone reads it), per-sample ``w`` when
        only ``want_w`` is."""
        gw_shape = (self.weight_numel,) if self.shared_weights else (num_edges, self.weight_numel)
        gw = torch.empty(gw_shape, dtype=x1.dtype, device=x1.device) if want_w else None
        gx2 = torch.empty(num_edges, self.in2_dim, dtype=x1.dtype, device=x1.device) if want_x2 else None
        if w is None and self.shared_weights and self.weight_numel:
            w = x1.new_zeros(self.weight_numel)
        bits = src.element_size() * 8 if src is not None else 64
        with torch.cuda.device(x1.device):
            _lib.check(
                _lib.lib().e3x_tp_backward_w_x2(
                    self.handle, _lib.ptr(x1), _lib.ptr(x2), _lib.ptr(w), _lib.ptr(grad_out), _lib.ptr(src), _lib.ptr(dst),
                    bits, _lib.ptr(gw), _lib.ptr(gx2), num_edges, x1.shape[0], grad_out.shape[0], _lib.stream_ptr(x1.device),
                )  # fmt: skip
            )
        return gw, gx2


def _w3j_swap_sign(tp, t):
    # exchanging two indices of the real Wigner 3j tensor multiplies it by (-1)^(l1 + l2 + l3)
    l = tp.irreps_in1[t.i_in1].ir.l + tp.irreps_in2[t.i_in2].ir.l + tp.irreps_out[t.i_out].ir.l
    return -1.0 if l % 2 else 1.0


def _permuted_weights(tp, w, perm):
    """Per-instruction ``[..., U, V, W]`` weight blocks of a ``uvw`` product with their last three axes permuted: one
    gather along the weight axis through an index list built once per product, permutation and device."""
    if tp.weight_numel == 0:
        return w
    key = ("weight permutation", perm, w.device)  # kept with the plans: dropped by copies and pickles alike
    index = tp._plans.get(key)
    if index is None:
        blocks, offset = [], 0
        for t in tp.instructions:
            if t.has_weight:
                n = prod(t.path_shape)
                blocks.append(torch.arange(offset, offset + n).view(t.path_shape).permute(*perm).reshape(-1))
                offset += n
        index = tp._plans[key] = torch.cat(blocks).to(w.device)
    return w.index_select(-1, index)


# ---------------------------------------------------------------------------------------------------- autograd
# The product is trilinear, so F(x1, x2, w, g) = <g, tp(x1, x2, w)> is linear in each of its four slots.  The product
# itself is dF/dg and its three gradients are dF/dx1, dF/dx2, dF/dw, each a function of the other three slots; and the
# derivative of any of these four maps with respect to one of ITS arguments, contracted with a cotangent c, is again
# one of the four maps, evaluated with c in the slot that the differentiated map stands for.  The family is closed, so
# one autograd Function per family, whose backward applies the same Function, gives derivatives of every order (the
# reference gets them by differentiating its einsums, e3nn/o3/_tensor_product/_codegen.py:148-187; a loss on forces
# needs the second).  Every member runs on a kernel that exists for the first-order pass: the forward kernel, the
# forward kernel on a transposed plan, or one of the weight / second-input gradient kernels.
_X1, _X2, _W, _OUT = 0, 1, 2, 3


def _tp_gradients(tp, x1, x2, w, g, need1, need2, needw):
    """``(d/dx1, d/dx2, d/dw)`` of ``<g, tp(x1, x2, w)>``, None where not needed: d/dx1 and (for ``uvw``) d/dx2 run the
    forward kernels on transposed plans; d/dw and d/dx2 of ``uvu`` have their own edge-parallel kernel, which writes
    both in one pass when both are wanted.  An argument that no wanted gradient depends on (``x1`` for d/dx1, ``x2``
    for d/dx2, ``w`` for d/dw) may be None."""
    g = g.contiguous()
    dt, Z = g.dtype, g.shape[0]
    g1 = g2 = gw = None
    mode = tp._live_mode()
    needw = needw and tp.weight_numel > 0
    if mode == "uvu":
        if need1:
            g1 = tp._grad_plan("x1", dt).forward(g, x2, w)
        if need2 or needw:
            if tp.shared_weights and needw and dt != torch.float32:
                # the sum over the batch is taken by fp32 atomics: the fp32 kernel on widened copies
                gw, g2 = tp._plan(torch.float32).backward_w_x2(
                    x1.float(), x2.float(), None if w is None else w.float(), g.float(), None, None, True, need2, Z
                )
                gw = gw.to(dt)
                g2 = None if g2 is None else g2.to(dt)
            else:
                gw, g2 = tp._plan(dt).backward_w_x2(x1, x2, w, g, None, None, needw, need2, Z)
    elif mode == "uvw":
        if needw:
            if dt != torch.float32:
                # the weight-gradient kernels read fp32 rows: widened copies of the operands, result in storage type
                gw = tp._plan(torch.float32).backward_w_uvw(x1.float(), x2.float(), g.float(), tp.shared_weights).to(dt)
            else:
                gw = tp._plan(dt).backward_w_uvw(x1, x2, g, tp.shared_weights)
        if need1:
            g1 = tp._grad_plan("x1", dt).forward(g, x2, _permuted_weights(tp, w, (2, 1, 0)))
        if need2:
            g2 = tp._grad_plan("x2", dt).forward(x1, g, _permuted_weights(tp, w, (0, 2, 1)))
    elif mode == "general":
        raise AssertionError("general connection modes are differentiated through TensorProduct._dense_equivalent")
    else:
        g1 = g.new_zeros(Z, tp._in1_dim) if need1 else None
        g2 = g.new_zeros(Z, tp._in2_dim) if need2 else None
    return g1, g2, gw


def _slot_backward(fn, slot, saved, cot, needs, *context):
    """Backward of one member of a closed family (see above): the gradient with respect to the argument that fills
    slot ``t`` is the member ``t`` evaluated with the cotangent in slot ``slot``.  Differentiable itself."""
    others = [t for t in range(4) if t != slot]
    full = {slot: cot, **dict(zip(others, saved))}
    grads = []
    for t, need in zip(others, needs):
        grads.append(fn.apply(t, *context, *[full[u] for u in range(4) if u != t]) if need else None)
    return grads


class _TpSlot(torch.autograd.Function):
    """Member ``slot`` of the family of the plain product: ``_OUT`` is ``tp(x1, x2, w)``, ``_X1`` / ``_X2`` / ``_W`` its
    gradients; the three tensor arguments are the other slots in the order (x1, x2, w, g)."""

    @staticmethod
    def forward(ctx, slot, tp, a, b, c):
        ctx.slot, ctx.tp = slot, tp
        ctx.save_for_backward(a, b, c)
        if slot == _OUT:
            return tp._plan(a.dtype).forward(a, b, c)
        x1, x2, w, g = [a, b, c][:slot] + [None] + [a, b, c][slot:]
        out = _tp_gradients(tp, x1, x2, w, g, slot == _X1, slot == _X2, slot == _W)[slot]
        if out is None:  # the gradient of weights that do not exist
            shape = (0,) if tp.shared_weights else (g.shape[0], 0)
            out = g.new_zeros(shape)
        return out

    @staticmethod
    def backward(ctx, cot):
        saved, needs = ctx.saved_tensors, ctx.needs_input_grad[2:5]
        if ctx.slot == _OUT and not torch.is_grad_enabled():
            # the first-order pass: kernels that write several gradients at once
            g1, g2, gw = _tp_gradients(ctx.tp, *saved, cot, *needs)
            if needs[2] and gw is None:
                gw = torch.zeros_like(saved[2])
            return None, None, g1, g2, gw
        return (None, None, *_slot_backward(_TpSlot, ctx.slot, saved, cot.contiguous(), needs, ctx.tp))


class _TensorProductFn:
    """``tp(x1, x2, w)`` under autograd (every order of differentiation)."""

    @staticmethod
    def apply(x1, x2, w, tp):
        return _TpSlot.apply(_OUT, tp, x1, x2, w)


def _message_gradients(tp, edges, node_x, edge_attr, w, g, need1, need2, needw):
    """``(d/dnode_x, d/dedge_attr, d/dw)`` of ``<g, scatter(tp(node_x[src], edge_attr, w), dst)>``; None where not needed.
    d/dnode_x is the fused kernel on the transposed plan with the roles of source and destination exchanged.  An
    argument that no wanted gradient depends on may be None."""
    g = g.contiguous()
    dt = g.dtype
    g1 = g2 = gw = None
    needw = needw and tp.weight_numel > 0
    if need1 and needw and dt == torch.float32:
        # every gradient from one pass over the weights and one gather of g per edge
        res = tp._grad_plan("x1", dt).gather_scatter_grad_w(
            g, edge_attr, w, node_x, edges.edge_dst, edges.transposed(), need2 and edge_attr.shape[1] > 0
        )
        if res is not None:
            return res[0], (res[2] if need2 else None), res[1]
    if need1:
        rev = edges.transposed()
        g1 = tp._grad_plan("x1", dt).gather_scatter(g, edge_attr, w, edges.edge_dst, rev, g.shape[0])
    if need2 or needw:
        gw, g2 = tp._plan(dt).backward_w_x2(node_x, edge_attr, w, g, edges.edge_src, edges.edge_dst, needw, need2, edges.num_edges)
    return g1, g2, gw


class _MessageSlot(torch.autograd.Function):
    """Member ``slot`` of the family of the message step ``scatter(tp(node_x[src], edge_attr, w), dst)``: slots
    (node_x [N_src, dim1], edge_attr [E, dim2], w [E, weight_numel], g [N, dim_out])."""

    @staticmethod
    def forward(ctx, slot, tp, edges, a, b, c):
        ctx.slot, ctx.tp, ctx.edges = slot, tp, edges
        ctx.save_for_backward(a, b, c)
        if slot == _OUT:
            return tp._plan(a.dtype).gather_scatter(a, b, c, edges.edge_src, edges, a.shape[0])
        x, attr, w, g = [a, b, c][:slot] + [None] + [a, b, c][slot:]
        out = _message_gradients(tp, edges, x, attr, w, g, slot == _X1, slot == _X2, slot == _W)[slot]
        return g.new_zeros(edges.num_edges, 0) if out is None else out  # (the gradient of weights that do not exist)

    @staticmethod
    def backward(ctx, cot):
        saved, needs = ctx.saved_tensors, ctx.needs_input_grad[3:6]
        if ctx.slot == _OUT and not torch.is_grad_enabled():
            g1, g2, gw = _message_gradients(ctx.tp, ctx.edges, *saved, cot, *needs)
            if needs[2] and gw is None:
                gw = torch.zeros_like(saved[2])
            return None, None, None, g1, g2, gw
        return (None, None, None, *_slot_backward(_MessageSlot, ctx.slot, saved, cot.contiguous(), needs, ctx.tp, ctx.edges))


class _GatherScatterFn:
    """``scatter(tp(node_x[src], edge_attr, w), dst)`` under autograd (every order of differentiation)."""

    @staticmethod
    def apply(node_x, edge_attr, w, tp, edges):
        return _MessageSlot.apply(_OUT, tp, edges, node_x, edge_attr, w)


class _GatherScatterShFn(torch.autograd.Function):
    """``_GatherScatterFn`` on ``edge_attr = spherical_harmonics(0 .. lmax, edge_vec)``, the harmonics formed inside the
    kernel.  The backward pass evaluates them once with the stand-alone kernel (they are 3 % of the per-edge bytes)
    and runs the message gradients on them; the gradient of the vectors goes through the harmonics' own backward.
    Under ``create_graph`` the backward pass is the differentiable composition of the two families."""

    @staticmethod
    def forward(ctx, node_x, edge_vec, w, tp, edges, normalize, normalization):
        from .spherical_harmonics import _NORMALIZATION

        out = tp._plan(node_x.dtype).gather_scatter_sh(
            node_x, edge_vec, w, edges.edge_src, edges, node_x.shape[0], normalize, _NORMALIZATION[normalization]
        )
        if out is None:
            raise NotImplementedError("forward_gather_scatter_sh needs irreps_in2 = 0e + 1o + ... up to l <= 3 (multiplicity 1)")
        ctx.tp, ctx.edges, ctx.sh = tp, edges, (normalize, normalization)
        ctx.save_for_backward(node_x, edge_vec, w)
        return out

    @staticmethod
    def backward(ctx, g):
        from .spherical_harmonics import _sh_backward, _sh_forward

        node_x, edge_vec, w = ctx.saved_tensors
        need1, need_vec, needw = ctx.needs_input_grad[:3]
        tp, edges = ctx.tp, ctx.edges
        ls = tuple(range(len(tp.irreps_in2)))
        if torch.is_grad_enabled():
            attr = _sh_forward(edge_vec, ls, *ctx.sh).to(node_x.dtype)  # differentiable in edge_vec
            g1, g2, gw = _slot_backward(_MessageSlot, _OUT, (node_x, attr, w), g.contiguous(), (need1, need_vec, needw), tp, edges)
            gvec = _sh_backward(edge_vec, g2.to(edge_vec.dtype), ls, *ctx.sh) if need_vec else None
            return g1, gvec, gw, None, None, None, None
        attr = _sh_forward(edge_vec, ls, *ctx.sh).to(node_x.dtype)
        g1, g2, gw = _message_gradients(tp, edges, node_x, attr, w, g, need1, need_vec, needw)
        gvec = _sh_backward(edge_vec, g2.to(edge_vec.dtype), ls, *ctx.sh) if need_vec else None
        return g1, gvec, gw, None, None, None, None


class _Constants(torch.nn.Module):
    """Holder of constant buffers under the names the reference's generated modules give them."""

    def __init__(self, tensors) -> None:
        super().__init__()
        for name, value in tensors.items():
            self.register_buffer(name, value)


class TensorProduct(torch.nn.Module):
    r"""Tensor product with parametrised paths (see the reference docstring, ``_tensor_product.py:25-194``).

    ``instructions`` is a list of ``(i_in1, i_in2, i_out, mode, has_weight[, path_weight])``.
    All-``uvu`` and all-``uvw`` instruction sets have dedicated kernels with a backward pass; every other
    connection mode (and mixtures) runs forward on the general vector-ALU kernel.
    """

    def __init__(
        self,
        irreps_in1,
        irreps_in2,
        irreps_out,
        instructions: List[tuple],
        in1_var=None,
        in2_var=None,
        out_var=None,
        irrep_normalization: str = None,
        path_normalization: str = None,
        internal_weights: Optional[bool] = None,
        shared_weights: Optional[bool] = None,
        compile_left_right: bool = True,
        compile_right: bool = False,
        normalization=None,  # for backward compatibility
        _specialized_code: Optional[bool] = None,
        _optimize_einsums: Optional[bool] = None,
    ) -> None:
        super().__init__()
        if normalization is not None:
            warnings.warn("`normalization` is deprecated. Use `irrep_normalization` instead.", DeprecationWarning)
            irrep_normalization = normalization
        irrep_normalization = "component" if irrep_normalization is None else irrep_normalization
        path_normalization = "element" if path_normalization is None else path_normalization
        assert irrep_normalization in ["component", "norm", "none"]
        assert path_normalization in ["element", "path", "none"]
        self._compile_right = compile_right  # right() runs on the forward kernel: nothing extra to build

        self.irreps_in1 = Irreps(irreps_in1)
        self.irreps_in2 = Irreps(irreps_in2)
        self.irreps_out = Irreps(irreps_out)
        i1, i2, io = self.irreps_in1, self.irreps_in2, self.irreps_out

        raw = [tuple(t) if len(t) == 6 else tuple(t) + (1.0,) for t in instructions]
        for a, b, c, mode, _, _ in raw:
            assert mode in _MODES
            assert i1[a].ir.p * i2[b].ir.p == io[c].ir.p
            assert abs(i1[a].ir.l - i2[b].ir.l) <= io[c].ir.l <= i1[a].ir.l + i2[b].ir.l

        def variances(var, irreps, name):
            if var is None:
                return [1.0] * len(irreps)
            var = [float(v) for v in var]
            assert len(var) == len(irreps), f"Len of {name} must be equal to len of the irreps"
            return var

        in1_var = variances(in1_var, i1, "in1_var")
        in2_var = variances(in2_var, i2, "in2_var")
        out_var = variances(out_var, io, "out_var")

        # path normalisation: alpha / (sum over the paths into the same output of the number of
        # summed elements), times the variances and the user path weight; stored as sqrt
        self.instructions = []
        for a, b, c, mode, has_weight, pw in raw:
            alpha = {"component": io[c].ir.dim, "norm": i1[a].ir.dim * i2[b].ir.dim, "none": 1}[irrep_normalization]
            if path_normalization == "element":
                x = sum(in1_var[a2] * in2_var[b2] * _num_elements(m, i1[a2].mul, i2[b2].mul) for a2, b2, c2, m, _, _ in raw if c2 == c)
            elif path_normalization == "path":
                x = in1_var[a] * in2_var[b] * _num_elements(mode, i1[a].mul, i2[b].mul)
                x *= len([t for t in raw if t[2] == c])
            else:
                x = 1
            if x > 0.0:
                alpha /= x
            alpha *= out_var[c]
            alpha *= pw
            self.instructions.append(
                Instruction(a, b, c, mode, has_weight, sqrt(alpha), _path_shape(mode, i1[a].mul, i2[b].mul, io[c].mul))
            )

        self._in1_dim, self._in2_dim = i1.dim, i2.dim

        if shared_weights is False and internal_weights is None:
            internal_weights = False
        if shared_weights is None:
            shared_weights = True
        if internal_weights is None:
            internal_weights = shared_weights and any(t.has_weight for t in self.instructions)
        assert shared_weights or not internal_weights
        self.internal_weights = internal_weights
        self.shared_weights = shared_weights

        opt = get_optimization_defaults()
        self._specialized_code = opt["specialized_code"] if _specialized_code is None else _specialized_code
        self._optimize_einsums = opt["optimize_einsums"] if _optimize_einsums is None else _optimize_einsums
        self._compile_left_right = compile_left_right

        for t in self.instructions:
            if t.connection_mode == "uvu":
                assert i1[t.i_in1].mul == io[t.i_out].mul
            if t.connection_mode in ("uvw", "u<vw"):
                assert t.has_weight

        self.weight_numel = sum(prod(t.path_shape) for t in self.instructions if t.has_weight)
        if internal_weights and self.weight_numel > 0:
            assert self.shared_weights, "Having internal weights impose shared weights"
            self.weight = torch.nn.Parameter(torch.randn(self.weight_numel))
        else:
            self.register_buffer("weight", torch.Tensor())

        if io.dim > 0:
            output_mask = torch.cat(
                [
                    torch.ones(mul * ir.dim)
                    if any(t.i_out == c and t.path_weight != 0 and 0 not in t.path_shape for t in self.instructions)
                    else torch.zeros(mul * ir.dim)
                    for c, (mul, ir) in enumerate(io)
                ]
            )
        else:
            output_mask = torch.ones(0)
        self.register_buffer("output_mask", output_mask)
        self._plans = {}
        # The reference keeps the Wigner tensors (and the index pairs of the triangular modes) as buffers of its
        # generated modules, so they are part of its state_dict.  The kernels here carry those constants as
        # immediates; the buffers exist so that checkpoints load in both directions with strict=True.
        self._compiled_main_left_right = _Constants(self._reference_constants(right=False))
        if compile_right:
            self._compiled_main_right = _Constants(self._reference_constants(right=True))

    def _reference_constants(self, right: bool):
        """Names and values of the buffers of the reference's generated module (``_codegen.py:143-144,289-325`` for
        ``forward``, ``:514-515,560-641`` for ``right``): a tensor ``_w3j_l1_l2_l3`` for every instruction whose
        contraction is not one of the specialised einsums, ``_triu_indices_n`` for the modes over pairs u < v."""
        from .wigner import wigner_3j

        spec = self._specialized_code
        out = {}
        for t in self.instructions:
            m1, m2, mo = self.irreps_in1[t.i_in1], self.irreps_in2[t.i_in2], self.irreps_out[t.i_out]
            if m1.dim == 0 or m2.dim == 0 or mo.dim == 0:
                continue
            l = (m1.ir.l, m2.ir.l, mo.ir.l)
            mode, special = t.connection_mode, spec and 0 in l
            if mode in ("uvu<v", "u<vw"):
                if right:
                    raise NotImplementedError  # as the reference (_codegen.py:620-623)
                uses = True
            elif mode == "uvuv" or (mode == "uuw" and (right or not t.has_weight)):
                uses = True
            elif mode in ("uvu", "uvv") and not t.has_weight and (right or mode == "uvu"):
                uses = True
            elif mode == "uuu":
                uses = not (special or (spec and l == (1, 1, 1) and not right))
            else:
                uses = not special
            if uses:
                out.setdefault(f"_w3j_{l[0]}_{l[1]}_{l[2]}", wigner_3j(*l))
            if mode in ("uvu<v", "u<vw"):
                out.setdefault(f"_triu_indices_{m1.mul}", torch.triu_indices(m1.mul, m1.mul, 1))
        return out

    # ------------------------------------------------------------------ plans
    def _kernel_instructions(self):
        return [(t.i_in1, t.i_in2, t.i_out, t.connection_mode, t.has_weight, t.path_weight) for t in self.instructions]

    def _live_mode(self):
        """"uvu" / "uvw" for the two families with backward kernels, "general" for anything else, None if empty."""
        live = {t.connection_mode for t in self.instructions if 0 not in t.path_shape}
        if not live:
            return None
        return next(iter(live)) if len(live) == 1 and live <= {"uvu", "uvw"} else "general"

    def _plan(self, dtype: torch.dtype) -> _Plan:
        if dtype not in _DTYPES:
            raise TypeError(f"TensorProduct kernels support float32 and bfloat16 storage, got {dtype}")
        plan = self._plans.get(dtype)
        if plan is None:
            plan = self._plans[dtype] = _Plan(
                self.irreps_in1, self.irreps_in2, self.irreps_out, self._kernel_instructions(), self.shared_weights, dtype
            )
            assert plan.weight_numel == self.weight_numel, (plan.weight_numel, self.weight_numel)
        return plan

    def _grad_plan(self, wrt: str, dtype: torch.dtype) -> _Plan:
        """Transposed plan whose forward pass is the gradient with respect to ``x1`` or (``uvw`` only) ``x2``.

        d out / d x1 contracts the same Wigner tensor over (j, k) instead of (i, j): a tensor product
        ``irreps_out x irreps_in2 -> irreps_in1`` with the index-swap sign folded into the path weight
        (``uvw`` also needs the weight blocks transposed, see ``_permuted_weights``)."""
        key = (wrt, dtype)
        plan = self._plans.get(key)
        if plan is None:
            ins = []
            for t in self.instructions:
                pw = t.path_weight * _w3j_swap_sign(self, t)
                if wrt == "x1":
                    ins.append((t.i_out, t.i_in2, t.i_in1, t.connection_mode, t.has_weight, pw))
                else:
                    ins.append((t.i_in1, t.i_out, t.i_in2, t.connection_mode, t.has_weight, pw))
            if wrt == "x1":
                plan = _Plan(self.irreps_out, self.irreps_in2, self.irreps_in1, ins, self.shared_weights, dtype)
            else:
                assert self._live_mode() in ("uvw", None)
                plan = _Plan(self.irreps_in1, self.irreps_out, self.irreps_in2, ins, self.shared_weights, dtype)
            self._plans[key] = plan
        return plan

    def compile(self, dtype: torch.dtype = torch.float32) -> "TensorProduct":
        """Builds (or finds in the kernel cache) the specialised kernels now; needs no GPU."""
        self._plan(dtype)
        return self

    def _dense_equivalent(self):
        """``(tp, expand)`` for instruction sets outside pure ``uvu`` / pure ``uvw``: the same bilinear map written as
        a pure ``uvw`` product whose weight blocks ``[U, V, W]`` are zero except where the connection mode couples
        the indices (``uvu``: ``D[u, v, u] = w[u, v]``, ``uuu``: ``D[u, u, u] = w[u]``, ``u<vw``: ``D[u, v, w] = w[p(u, v), w]``
        for ``u < v`` ...), with the path weights carried over unchanged.  ``expand(w)`` builds the dense weights
        from the structured ones by a differentiable ``index_copy``.  It costs U V W instead of U V products per path,
        but every gradient of the ``uvw`` family has a kernel; the forward pass without gradients keeps the
        mode-specific kernel."""
        cached = self._plans.get("dense")
        if cached is not None:
            return cached
        i1, i2, io = self.irreps_in1, self.irreps_in2, self.irreps_out
        ins, blocks = [], []  # blocks: (weighted, numel of the structured block, positions in the dense block, dense numel)
        for t in self.instructions:
            U, V, W = i1[t.i_in1].mul, i2[t.i_in2].mul, io[t.i_out].mul
            ins.append((t.i_in1, t.i_in2, t.i_out, "uvw", True, t.path_weight**2))
            u, v = torch.meshgrid(torch.arange(U), torch.arange(V), indexing="ij")
            u, v = u.reshape(-1), v.reshape(-1)
            m = t.connection_mode
            if m == "uvw":
                pos = torch.arange(U * V * W)
            elif m == "uvu":
                pos = (u * V + v) * W + u
            elif m == "uvv":
                pos = (u * V + v) * W + v
            elif m == "uuw":
                a = torch.arange(U)
                base = (a * V + a) * W
                pos = (base[:, None] + torch.arange(W)[None, :]).reshape(-1) if t.has_weight else base
            elif m == "uuu":
                a = torch.arange(U)
                pos = (a * V + a) * W + a
            elif m == "uvuv":
                pos = (u * V + v) * W + (u * V + v)
            else:
                pu, pv = torch.triu_indices(U, V, 1)
                pair = (pu * V + pv) * W
                if m == "uvu<v":
                    pos = pair + torch.arange(pair.numel())
                else:  # u<vw
                    pos = (pair[:, None] + torch.arange(W)[None, :]).reshape(-1)
            blocks.append((t.has_weight, prod(t.path_shape) if t.has_weight else pos.numel(), pos, U * V * W))
        shared = self.shared_weights or self.weight_numel == 0
        tp = TensorProduct(
            i1, i2, io, ins, irrep_normalization="none", path_normalization="none", internal_weights=False, shared_weights=shared
        )

        def expand(w, like):
            batch = () if shared else w.shape[:-1]
            out, off = [], 0
            for weighted, n, pos, dense in blocks:
                pos = pos.to(like.device)
                if weighted:
                    vals = w.narrow(-1, off, n)
                    off += n
                else:
                    vals = like.new_ones(batch + (n,))
                out.append(like.new_zeros(batch + (dense,)).index_copy(-1, pos, vals.to(like.dtype)))
            return torch.cat(out, dim=-1) if out else like.new_empty(batch + (0,))

        self._plans["dense"] = (tp, expand)
        return tp, expand

    def compile_backward(self, dtype: torch.dtype = torch.float32) -> "TensorProduct":
        """Also builds the transposed plans the backward pass uses."""
        self._plan(dtype)
        if self._live_mode() == "general":
            self._dense_equivalent()[0].compile_backward(dtype)
            return self
        self._grad_plan("x1", dtype)
        if self._live_mode() == "uvu":
            _lib.check(_lib.lib().e3x_tp_plan_prepare_backward_w(self._plan(dtype).handle))
            if dtype == torch.float32 and not self.shared_weights and self.weight_numel:
                # the message-step backward kernel on the transposed plan, where the instruction set fits it
                rc = _lib.lib().e3x_tp_plan_prepare_gather_scatter_grad_w(self._grad_plan("x1", dtype).handle)
                if rc != _lib.ERR_INVALID:
                    _lib.check(rc)
            if dtype != torch.float32 and self.shared_weights and self.weight_numel:  # summed over the batch in fp32
                _lib.check(_lib.lib().e3x_tp_plan_prepare_backward_w(self._plan(torch.float32).handle))
        if self._live_mode() == "uvw":
            self._grad_plan("x2", dtype)
            if self.weight_numel:  # the weight gradient always runs on the fp32 plan
                _lib.check(_lib.lib().e3x_tp_plan_prepare_backward_w(self._plan(torch.float32).handle))
        return self

    def __getstate__(self):
        state = self.__dict__.copy()
        state["_plans"] = {}
        return state

    def __deepcopy__(self, memo):
        import copy

        cls = self.__class__
        new = cls.__new__(cls)
        memo[id(self)] = new
        for k, v in self.__dict__.items():
            new.__dict__[k] = {} if k == "_plans" else copy.deepcopy(v, memo)
        return new

    def __repr__(self) -> str:
        npath = sum(prod(t.path_shape) for t in self.instructions)
        return (
            f"{self.__class__.__name__}"
            f"({self.irreps_in1.simplify()} x {self.irreps_in2.simplify()} "
            f"-> {self.irreps_out.simplify()} | {npath} paths | {self.weight_numel} weights)"
        )

    # ------------------------------------------------------------------ weights
    def _prep_weights(self, weight):
        if isinstance(weight, list):
            shapes = [t.path_shape for t in self.instructions if t.has_weight]
            if not self.shared_weights:
                weight = [w.reshape(-1, prod(s)) for w, s in zip(weight, shapes)]
            else:
                weight = [w.reshape(prod(s)) for w, s in zip(weight, shapes)]
            return torch.cat(weight, dim=-1)
        return weight

    def _get_weights(self, weight) -> torch.Tensor:
        weight = self._prep_weights(weight)
        if weight is None:
            if self.weight_numel > 0 and not self.internal_weights:
                raise RuntimeError("Weights must be provided when the TensorProduct does not have `internal_weights`")
            return self.weight
        if self.shared_weights:
            torch._assert(weight.shape == (self.weight_numel,), "Invalid weight shape")
        else:
            torch._assert(weight.shape[-1] == self.weight_numel, "Invalid weight shape")
            torch._assert(weight.ndim > 1, "When shared weights is false, weights must have batch dimension")
        return weight

    def weight_view_for_instruction(self, instruction: int, weight: Optional[torch.Tensor] = None) -> torch.Tensor:
        if not self.instructions[instruction].has_weight:
            raise ValueError(f"Instruction {instruction} has no weights.")
        offset = sum(prod(t.path_shape) for t in self.instructions[:instruction])
        t = self.instructions[instruction]
        weight = self._get_weights(weight)
        return weight.narrow(-1, offset, prod(t.path_shape)).view(weight.shape[:-1] + t.path_shape)

    def weight_views(self, weight: Optional[torch.Tensor] = None, yield_instruction: bool = False):
        weight = self._get_weights(weight)
        batchshape = weight.shape[:-1]
        offset = 0
        for i, t in enumerate(self.instructions):
            if t.has_weight:
                n = prod(t.path_shape)
                view = weight.narrow(-1, offset, n).view(batchshape + t.path_shape)
                offset += n
                yield (i, t, view) if yield_instruction else view

    # ------------------------------------------------------------------ evaluation
    def right(self, y, weight=None):
        r"""Partially evaluate :math:`w x \otimes y`: the matrices ``[..., irreps_in1.dim, irreps_out.dim]`` with
        ``forward(x, y, w) == x @ right(y, w)`` (reference ``_tensor_product.py:447-486``).  There is no kernel of its
        own: row ``a`` of the result is the tensor product of the ``a``-th basis vector with ``y``, so one forward
        launch on ``irreps_in1.dim`` rows per sample gives the whole matrix (and its gradients)."""
        torch._assert(self._compile_right, "`right` method is not compiled, set `compile_right` to True when creating the TensorProduct")
        torch._assert(y.shape[-1] == self._in2_dim, "Incorrect last dimension for y")
        w = self._get_weights(weight)
        self._check_device(y)
        if self.shared_weights or self.weight_numel == 0:
            batch = tuple(y.shape[:-1])
        else:
            batch = tuple(torch.broadcast_shapes(y.shape[:-1], w.shape[:-1]))
        d1 = self._in1_dim
        eye = torch.eye(d1, dtype=y.dtype, device=y.device).expand(batch + (d1, d1))
        yb = y.expand(batch + (-1,)).unsqueeze(-2).expand(batch + (d1, self._in2_dim))
        if not (self.shared_weights or self.weight_numel == 0):
            w = w.expand(batch + (-1,)).unsqueeze(-2).expand(batch + (d1, self.weight_numel))
        return self.forward(eye, yb, w if self.weight_numel else None)

    def _check_device(self, *tensors):
        for t in tensors:
            if not t.is_cuda:
                raise RuntimeError("e3nn_amd.o3.TensorProduct runs on the GPU only; got a CPU tensor")

    def forward(self, x, y, weight: Optional[Union[torch.Tensor, List[torch.Tensor]]] = None):
        r"""Evaluate :math:`w x \otimes y`: ``x[..., irreps_in1.dim]``, ``y[..., irreps_in2.dim]``,
        ``weight[weight_numel]`` (shared) or ``weight[..., weight_numel]`` -> ``[..., irreps_out.dim]``."""
        torch._assert(x.shape[-1] == self._in1_dim, "Incorrect last dimension for x")
        torch._assert(y.shape[-1] == self._in2_dim, "Incorrect last dimension for y")
        torch._assert(self._compile_left_right, "`left_right` method is not compiled, set `compile_left_right` to True when creating the TensorProduct")
        w = self._get_weights(weight)
        self._check_device(x, y)
        if w.numel() and w.device != x.device:
            raise RuntimeError("weights and inputs must be on the same device")
        # broadcast all batch dimensions (everything but the last)
        if self.shared_weights or self.weight_numel == 0:
            batch = torch.broadcast_shapes(x.shape[:-1], y.shape[:-1])
        else:
            batch = torch.broadcast_shapes(x.shape[:-1], y.shape[:-1], w.shape[:-1])
        x1 = x.expand(batch + (-1,)).reshape(-1, self._in1_dim).contiguous()
        x2 = y.expand(batch + (-1,)).reshape(-1, self._in2_dim).to(x1.dtype).contiguous()
        if self.weight_numel == 0:
            wf = x1.new_empty(0)
        elif self.shared_weights:
            wf = w.to(x1.dtype).contiguous()
        else:
            wf = w.expand(batch + (-1,)).reshape(-1, self.weight_numel).to(x1.dtype).contiguous()
        if self._live_mode() == "general" and torch.is_grad_enabled() and (x1.requires_grad or x2.requires_grad or wf.requires_grad):
            dense_tp, expand = self._dense_equivalent()
            out = _TensorProductFn.apply(x1, x2, expand(wf, x1), dense_tp)
        else:
            out = _TensorProductFn.apply(x1, x2, wf, self)
        return out.reshape(batch + (self.irreps_out.dim,))

    def forward_gather_scatter(
        self,
        node_x: torch.Tensor,
        edge_attr: torch.Tensor,
        weight: torch.Tensor,
        edge_src: Optional[torch.Tensor] = None,
        edge_dst: Optional[torch.Tensor] = None,
        num_nodes: Optional[int] = None,
        edges=None,
    ) -> torch.Tensor:
        """``scatter(self(node_x[edge_src], edge_attr, weight), edge_dst, num_nodes)`` in one kernel.

        ``node_x[N_src, irreps_in1.dim]``, ``edge_attr[E, irreps_in2.dim]``, ``weight[E, weight_numel]``
        (per-edge weights, ``shared_weights=False``); result ``[num_nodes, irreps_out.dim]``.
        Pass a prebuilt ``DstSortedEdges`` as ``edges`` to amortise the index preprocessing
        over several calls on the same graph.
        """
        if any(t.connection_mode != "uvu" for t in self.instructions):
            raise NotImplementedError("forward_gather_scatter needs an all-uvu TensorProduct")
        torch._assert(node_x.ndim == 2 and node_x.shape[-1] == self._in1_dim, "Incorrect shape for node_x")
        torch._assert(edge_attr.ndim == 2 and edge_attr.shape[-1] == self._in2_dim, "Incorrect shape for edge_attr")
        self._check_device(node_x, edge_attr)
        if edges is None:
            from ..nn.edges import DstSortedEdges  # here: e3nn_amd.nn imports this module

            edges = DstSortedEdges(edge_src, edge_dst, node_x.shape[0] if num_nodes is None else num_nodes, node_x.shape[0])
        torch._assert(edge_attr.shape[0] == edges.num_edges, "edge_attr must have one row per edge")
        torch._assert(edges.num_src_nodes == node_x.shape[0], "edge list was built for another node count")
        if self.weight_numel:
            torch._assert(not self.shared_weights, "forward_gather_scatter needs per-edge weights (shared_weights=False)")
            w = self._get_weights(weight)
            torch._assert(w.shape == (edges.num_edges, self.weight_numel), "Invalid weight shape")
            w = w.to(node_x.dtype).contiguous()
        else:
            w = node_x.new_empty(0)
        return _GatherScatterFn.apply(node_x.contiguous(), edge_attr.to(node_x.dtype).contiguous(), w, self, edges)


    def forward_gather_scatter_sh(self, node_x, edge_vec, weight, edges, normalize: bool = True, normalization: str = "component"):
        """``forward_gather_scatter(node_x, spherical_harmonics(range(lmax + 1), edge_vec, normalize, normalization),
        weight, edges=edges)`` with the harmonics formed inside the kernel: ``edge_vec[E, 3]`` (float32) is read in
        place of the stored ``[E, (lmax + 1)^2]`` attributes.  Needs ``irreps_in2 = 0e + 1o + ...`` up to ``lmax <= 3``
        with multiplicity 1 (what the reference's convolutions feed the product, e3nn/nn/models/gate_points_2101.py:329)."""
        if any(t.connection_mode != "uvu" for t in self.instructions):
            raise NotImplementedError("forward_gather_scatter_sh needs an all-uvu TensorProduct")
        assert normalization in ["integral", "component", "norm"]
        torch._assert(node_x.ndim == 2 and node_x.shape[-1] == self._in1_dim, "Incorrect shape for node_x")
        torch._assert(edge_vec.shape == (edges.num_edges, 3), "edge_vec must be [num_edges, 3]")
        self._check_device(node_x, edge_vec)
        if edge_vec.dtype != torch.float32:
            raise TypeError(f"edge vectors are read as float32, got {edge_vec.dtype}")
        torch._assert(edges.num_src_nodes == node_x.shape[0], "edge list was built for another node count")
        if self.weight_numel:
            torch._assert(not self.shared_weights, "forward_gather_scatter_sh needs per-edge weights (shared_weights=False)")
            w = self._get_weights(weight)
            torch._assert(w.shape == (edges.num_edges, self.weight_numel), "Invalid weight shape")
            w = w.to(node_x.dtype).contiguous()
        else:
            w = node_x.new_empty(0)
        return _GatherScatterShFn.apply(node_x.contiguous(), edge_vec.contiguous(), w, self, edges, bool(normalize), normalization)

    def _radial_description(self, net):
        """Arguments of the library's fused radial-network kernel for ``net``; None when ``net`` is not a two-layer
        ``nn.FullyConnectedNet`` ending in this product's per-edge weights."""
        from ..nn.activation import _KINDS, second_moment_constant

        layers = list(net)
        if len(layers) != 2 or layers[1].act is not None or net.hs[-1] != self.weight_numel or self.shared_weights:
            return None
        if not self.instructions or any(t.connection_mode != "uvu" for t in self.instructions):
            return None
        name = layers[0]._act_name or "identity"
        cst = second_moment_constant(name) if layers[0].act is not None else 1.0
        return net.hs[0], net.hs[1], _KINDS[name], cst, float(layers[0].var_in), float(layers[1].var_out)

    def prepare_gather_scatter_radial(self, net) -> bool:
        """Builds the kernel of ``forward_gather_scatter_radial`` for ``net`` ahead of the first call (no GPU needed);
        False when the instruction set or the network is outside what the kernel takes."""
        desc = self._radial_description(net)
        if desc is None:
            return False
        rc = _lib.lib().e3x_tp_plan_prepare_radial(self._plan(torch.float32).handle, *desc)
        if rc == _lib.ERR_INVALID:
            return False
        _lib.check(rc)
        return True

    def forward_gather_scatter_radial(self, node_x, edge_attr, edge_scalars, net, edges):
        """``forward_gather_scatter(node_x, edge_attr, net(edge_scalars), edges=edges)`` in one kernel, without the
        ``[E, weight_numel]`` weights ever being stored: ``net`` is a two-layer ``nn.FullyConnectedNet``
        ``[n_in, n_hidden, weight_numel]``.  Inference only (no autograd graph is recorded); returns None when the
        instruction set, the network or the tensors are outside what the kernel takes, so that the caller can run the
        two steps separately."""
        desc = self._radial_description(net)
        if desc is None:
            return None
        layers = list(net)
        tensors = (node_x, edge_attr, edge_scalars, layers[0].weight, layers[1].weight)
        if not all(t.is_cuda and t.dtype == torch.float32 for t in tensors):
            return None
        if node_x.ndim != 2 or node_x.shape[-1] != self._in1_dim or edge_attr.shape != (edges.num_edges, self._in2_dim):
            return None
        if edge_scalars.shape != (edges.num_edges, net.hs[0]) or edges.num_src_nodes != node_x.shape[0]:
            return None
        with torch.no_grad():
            return self._plan(torch.float32).gather_scatter_radial(
                node_x.contiguous(), edge_attr.contiguous(), edge_scalars.contiguous(), layers[0].weight.detach().contiguous(),
                layers[1].weight.detach().contiguous(), desc[2], desc[3], desc[4], desc[5], edges.edge_src, edges, node_x.shape[0],
            )  # fmt: skip


class FullyConnectedTensorProduct(TensorProduct):
    r"""All paths allowed by :math:`|l_1 - l_2| \leq l_{out} \leq l_1 + l_2`, mode ``uvw``, weighted
    (reference ``_sub.py:46-68``)."""

    def __init__(self, irreps_in1, irreps_in2, irreps_out, irrep_normalization: str = None, path_normalization: str = None, **kwargs) -> None:
        irreps_in1, irreps_in2, irreps_out = Irreps(irreps_in1), Irreps(irreps_in2), Irreps(irreps_out)
        instr = [
            (i_1, i_2, i_out, "uvw", True, 1.0)
            for i_1, (_, ir_1) in enumerate(irreps_in1)
            for i_2, (_, ir_2) in enumerate(irreps_in2)
            for i_out, (_, ir_out) in enumerate(irreps_out)
            if ir_out in ir_1 * ir_2
        ]
        super().__init__(
            irreps_in1, irreps_in2, irreps_out, instr,
            irrep_normalization=irrep_normalization, path_normalization=path_normalization, **kwargs,
        )  # fmt: skip
