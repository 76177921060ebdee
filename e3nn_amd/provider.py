"""The binding an e3nn maintainer would add: a code-generation provider that serves ``TensorProduct`` from libe3x.

e3nn asks every entry of ``e3nn.o3._tensor_product._tensor_product._CODEGEN_PROVIDERS_LEFT_RIGHT``
(e3nn/o3/_tensor_product/_tensor_product.py:17-21) for an ``fx.GraphModule`` that is later called as
``mod(x1, x2, w)`` (:348-361, :554).  ``hip_provider`` answers for every instruction set the library has a kernel
for and returns ``None`` otherwise, which defers to the next provider (e3nn's own einsum code generator).

Nothing here imports e3nn: the functions take e3nn's objects by their attributes (``Irreps`` iterate as
``(mul, ir)`` with ``ir.l`` / ``ir.p``; ``Instruction`` has ``i_in1, i_in2, i_out, connection_mode, has_weight,
path_weight``), which this package's own classes share, so the binding is exercised by this repository's tests.

    import e3nn.o3._tensor_product._tensor_product as m
    from e3nn_amd.provider import register
    register(m._CODEGEN_PROVIDERS_LEFT_RIGHT)      # from then on o3.TensorProduct(...) runs on the HIP kernels
"""
import ctypes

import torch
from torch import fx

from . import _lib

_MODES = {"uvw": 0, "uvu": 1, "uvv": 2, "uuw": 3, "uuu": 4, "uvuv": 5, "uvu<v": 6, "u<vw": 7}  # E3X_MODE_*
_DTYPES = {torch.float32: _lib.F32, torch.bfloat16: _lib.BF16}


def make_desc(irreps_in1, irreps_in2, irreps_out, instructions, shared_weights, dtype=torch.float32):
    """``e3x_tp_desc`` (include/e3x.h) from e3nn's constructor data.  ``path_weight`` is taken as e3nn has already
    normalised it (_tensor_product.py:289-324).  Returns ``(desc, keepalive)``: the arrays the descriptor points to."""

    def irreps_array(irreps):
        rows = [_lib.Irrep(int(mul), int(ir.l), int(ir.p)) for mul, ir in irreps]
        return (_lib.Irrep * max(1, len(rows)))(*rows), len(rows)

    (in1, n1), (in2, n2), (out, no) = irreps_array(irreps_in1), irreps_array(irreps_in2), irreps_array(irreps_out)
    rows = [
        _lib.Instruction(int(t.i_in1), int(t.i_in2), int(t.i_out), _MODES[t.connection_mode], int(bool(t.has_weight)), float(t.path_weight))
        for t in instructions
    ]  # fmt: skip
    ins = (_lib.Instruction * max(1, len(rows)))(*rows)
    desc = _lib.TpDesc(n1, n2, no, len(rows), in1, in2, out, ins, int(bool(shared_weights)), _DTYPES[dtype])
    return desc, (in1, in2, out, ins)


class HipTensorProduct(torch.nn.Module):
    """``forward(x1 [Z, dim1], x2 [Z, dim2], w)`` on one ``e3x_plan``: the module the fx graph calls."""

    def __init__(self, irreps_in1, irreps_in2, irreps_out, instructions, shared_weights, dtype=torch.float32):
        super().__init__()
        desc, keep = make_desc(irreps_in1, irreps_in2, irreps_out, instructions, shared_weights, dtype)
        self._plan = _lib.c_void_p()
        _lib.check(_lib.lib().e3x_tp_plan_create(ctypes.byref(desc), ctypes.byref(self._plan)))
        del keep  # the plan copies what it needs
        wn, d1, d2, do = (ctypes.c_int64() for _ in range(4))
        _lib.check(_lib.lib().e3x_tp_plan_info(self._plan, ctypes.byref(wn), ctypes.byref(d1), ctypes.byref(d2), ctypes.byref(do), None, None))
        self.weight_numel, self.in1_dim, self.in2_dim, self.out_dim = wn.value, d1.value, d2.value, do.value
        self.shared_weights = bool(shared_weights)

    def __del__(self):
        plan, self._plan = getattr(self, "_plan", None), None
        if plan:
            _lib.lib().e3x_tp_plan_destroy(plan)

    def forward(self, x1, x2, w):
        """Leading dimensions broadcast as in e3nn's generated code (_codegen.py:43-76); ``w`` is ``[weight_numel]``
        for shared weights, ``[..., weight_numel]`` otherwise (an empty tensor when there are no weights, :410)."""
        L = _lib.lib()
        per_sample = (not self.shared_weights) and self.weight_numel > 0
        batch = torch.broadcast_shapes(x1.shape[:-1], x2.shape[:-1], w.shape[:-1] if per_sample else ())
        x1 = x1.expand(batch + (self.in1_dim,)).reshape(-1, self.in1_dim).contiguous()
        x2 = x2.expand(batch + (self.in2_dim,)).reshape(-1, self.in2_dim).contiguous()
        w = w.expand(batch + (self.weight_numel,)).reshape(-1, self.weight_numel).contiguous() if per_sample else w.contiguous()
        out = x1.new_empty(x1.shape[0], self.out_dim)
        with torch.cuda.device(x1.device):
            nbytes = L.e3x_tp_forward_workspace_bytes(self._plan)
            ws = torch.empty(nbytes, dtype=torch.uint8, device=x1.device) if nbytes else None
            _lib.check(L.e3x_tp_forward_ws(self._plan, _lib.ptr(x1), _lib.ptr(x2), _lib.ptr(w), _lib.ptr(out), x1.shape[0],
                                           _lib.ptr(ws), nbytes, _lib.stream_ptr(x1.device)))  # fmt: skip
        return out.reshape(batch + (self.out_dim,))


def hip_provider(irreps_in1, irreps_in2, irreps_out, instructions, shared_weights, specialized_code, optimize_einsums):
    """Provider for ``_CODEGEN_PROVIDERS_LEFT_RIGHT``; ``None`` when the library has no kernel for the instruction set
    (the plan is refused) or nothing to compute."""
    live = [t for t in instructions if 0 not in t.path_shape]
    if not live:
        return None
    try:
        mod = HipTensorProduct(irreps_in1, irreps_in2, irreps_out, live, shared_weights)
    except _lib.E3xError:
        return None
    graph = fx.Graph()  # the hook requires an fx.GraphModule (e3nn/util/codegen/_mixin.py:40)
    x1, x2, w = (graph.placeholder(name) for name in ("x1", "x2", "w"))
    graph.output(graph.call_module("hip", (x1, x2, w)))
    root = torch.nn.Module()
    root.hip = mod
    return fx.GraphModule(root, graph, "tp_forward")


def register(providers: list) -> None:
    """Puts ``hip_provider`` in front of e3nn's own code generator."""
    if hip_provider not in providers:
        providers.insert(0, hip_provider)
