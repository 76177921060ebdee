"""Activation functions of scalar irreps and the gate non-linearity, on one HIP kernel (csrc/gate.hip).

Reference: ``e3nn/nn/_activation.py:9-104`` (``Activation``), ``e3nn/nn/_gate.py:8-154`` (``Gate``) and the
second-moment normalisation ``e3nn/math/_normalize_activation.py:9-57``.
"""
import ctypes
from typing import List

import torch
from torch.autograd.function import once_differentiable

from .. import _lib
from ..o3.irreps import Irrep, Irreps

_KINDS = {"identity": 0, "silu": 1, "tanh": 2, "sigmoid": 3, "abs": 4, "relu": 5}
_TORCH_NAMES = {
    torch.nn.functional.silu: "silu", torch.tanh: "tanh", torch.nn.functional.tanh: "tanh", torch.sigmoid: "sigmoid",
    torch.nn.functional.sigmoid: "sigmoid", torch.abs: "abs", torch.relu: "relu", torch.nn.functional.relu: "relu",
}  # fmt: skip
_TORCH_FUNCS = {"silu": torch.nn.functional.silu, "tanh": torch.tanh, "sigmoid": torch.sigmoid, "abs": torch.abs,
                "relu": torch.relu, "identity": lambda x: x}  # fmt: skip


class _ActBlock(ctypes.Structure):
    _fields_ = [("offset_in", ctypes.c_int32), ("offset_out", ctypes.c_int32), ("count", ctypes.c_int32),
                ("act", ctypes.c_int32), ("cst", ctypes.c_float)]  # fmt: skip


class _GateBlock(ctypes.Structure):
    _fields_ = [("gate_offset_in", ctypes.c_int32), ("gated_offset_in", ctypes.c_int32), ("offset_out", ctypes.c_int32),
                ("mul", ctypes.c_int32), ("dim", ctypes.c_int32), ("act", ctypes.c_int32), ("cst", ctypes.c_float)]  # fmt: skip


def activation_name(act) -> str:
    """Name of a supported activation given as a string, a torch function or ``None`` (identity)."""
    if act is None:
        return "identity"
    if isinstance(act, str):
        if act not in _KINDS:
            raise ValueError(f"unknown activation {act!r}; the gate kernel implements {sorted(_KINDS)}")
        return act
    if act in _TORCH_NAMES:
        return _TORCH_NAMES[act]
    if isinstance(act, torch.nn.SiLU):
        return "silu"
    if isinstance(act, torch.nn.Tanh):
        return "tanh"
    if isinstance(act, torch.nn.Sigmoid):
        return "sigmoid"
    if isinstance(act, torch.nn.ReLU):
        return "relu"
    raise NotImplementedError(f"activation {act!r} has no kernel; the gate kernel implements {sorted(_KINDS)}")


_CST_CACHE = {}


def second_moment_constant(name: str) -> float:
    """``<f(z)^2>^(-1/2)`` over one million seeded normal samples, snapped to 1 within 1e-4: the reference's
    ``normalize2mom`` (``_normalize_activation.py:9-19,42-48``), so that the constants agree to the last bit."""
    if name == "identity":
        return 1.0
    if name not in _CST_CACHE:
        gen = torch.Generator(device="cpu").manual_seed(0)
        z = torch.randn(1_000_000, generator=gen, dtype=torch.float64)
        cst = _TORCH_FUNCS[name](z).pow(2).mean().pow(-0.5).item()
        _CST_CACHE[name] = 1.0 if abs(cst - 1) < 1e-4 else cst
    return _CST_CACHE[name]


def _parity(name: str) -> int:
    return {"identity": -1, "silu": 0, "tanh": -1, "sigmoid": 0, "abs": 1, "relu": 0}[name]


def _act_irreps_out(irreps_in: Irreps, names: List[str], given: List[bool]) -> Irreps:
    """Output irreps of ``Activation`` (``_activation.py:40-66``): odd scalars take the parity of the activation."""
    out = []
    for (mul, ir), name, has in zip(irreps_in, names, given):
        if not has:
            out.append((mul, ir))
            continue
        if ir.l != 0:
            raise ValueError("Activation: cannot apply an activation function to a non-scalar input.")
        p_out = _parity(name) if ir.p == -1 else ir.p
        if p_out == 0:
            raise ValueError(
                "Activation: the parity is violated! The input scalar is odd but the activation is neither even nor odd."
            )
        out.append((mul, Irrep(0, p_out)))
    return Irreps(out)


class _GateFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, mod):
        ctx.mod = mod
        ctx.save_for_backward(x)
        return mod._launch(x, None)

    @staticmethod
    def backward(ctx, g):
        (x,) = ctx.saved_tensors
        return _GateBackwardFn.apply(x, g.contiguous(), ctx.mod), None


class _GateBackwardFn(torch.autograd.Function):
    """``(x, g) -> d<g, gate(x)>/dx``, itself differentiable once more (``e3x_gate_backward2``: second derivatives of the
    activations), which is what a loss on forces differentiates.  Third derivatives are not provided."""

    @staticmethod
    def forward(ctx, x, g, mod):
        ctx.mod = mod
        ctx.save_for_backward(x, g)
        return mod._launch(x, g)

    @staticmethod
    @once_differentiable
    def backward(ctx, cot):
        x, g = ctx.saved_tensors
        return ctx.mod._launch_second(x, g, cot.contiguous()) + (None,)


def _storage(x):
    return _lib.BF16 if x.dtype == torch.bfloat16 else _lib.F32


class _BlockModule(torch.nn.Module):
    """Rows ``[..., in_dim] -> [..., out_dim]`` through tables of scalar and gated blocks."""

    def _set_tables(self, acts, gates, in_dim, out_dim):
        if len(acts) > 16 or len(gates) > 16:
            raise NotImplementedError("the gate kernel takes at most 16 scalar blocks and 16 gated blocks")
        self._acts = (_ActBlock * max(1, len(acts)))(*[_ActBlock(*a) for a in acts])
        self._gates = (_GateBlock * max(1, len(gates)))(*[_GateBlock(*g) for g in gates])
        self._n = (len(acts), len(gates))
        self._dims = (in_dim, out_dim)

    def _launch(self, x, grad_out):
        in_dim, out_dim = self._dims
        Z = x.shape[0]
        res = torch.empty(Z, in_dim if grad_out is not None else out_dim, dtype=x.dtype, device=x.device)
        L = _lib.lib()
        with torch.cuda.device(x.device):
            if grad_out is None:
                rc = L.e3x_gate_forward(self._acts, self._n[0], self._gates, self._n[1], _lib.ptr(x), _lib.ptr(res), Z, in_dim,
                                        out_dim, _storage(x), _lib.stream_ptr(x.device))  # fmt: skip
            else:
                rc = L.e3x_gate_backward(self._acts, self._n[0], self._gates, self._n[1], _lib.ptr(x), _lib.ptr(grad_out),
                                         _lib.ptr(res), Z, in_dim, out_dim, _storage(x), _lib.stream_ptr(x.device))  # fmt: skip
        _lib.check(rc)
        return res

    def _launch_second(self, x, grad_out, cot):
        """``(d/dx, d/dgrad_out)`` of ``<cot, backward(x, grad_out)>``."""
        in_dim, out_dim = self._dims
        Z = x.shape[0]
        gx, gg = torch.empty_like(x), torch.empty_like(grad_out)
        with torch.cuda.device(x.device):
            rc = _lib.lib().e3x_gate_backward2(self._acts, self._n[0], self._gates, self._n[1], _lib.ptr(x), _lib.ptr(grad_out),
                                               _lib.ptr(cot), _lib.ptr(gg), _lib.ptr(gx), Z, in_dim, out_dim, _storage(x), _lib.stream_ptr(x.device))  # fmt: skip
        _lib.check(rc)
        return gx, gg

    def forward(self, features):
        in_dim, out_dim = self._dims
        torch._assert(features.shape[-1] == in_dim, "Incorrect last dimension for features")
        if not features.is_cuda:
            raise RuntimeError("e3nn_amd runs on the GPU only: move the features to a HIP device")
        if features.dtype not in (torch.float32, torch.bfloat16):
            raise NotImplementedError("the gate kernel stores rows as fp32 or bf16")
        x = features.reshape(-1, in_dim).contiguous()
        return _GateFn.apply(x, self).reshape(features.shape[:-1] + (out_dim,))


class Activation(_BlockModule):
    """Scalar activation function (``e3nn/nn/_activation.py``): ``acts[i]`` acts on the i-th irrep (``None``: identity,
    required for non-scalars).  Activations: silu, tanh, sigmoid, abs, relu (torch functions or names)."""

    def __init__(self, irreps_in, acts) -> None:
        super().__init__()
        irreps_in = Irreps(irreps_in)
        if len(irreps_in) != len(acts):
            raise ValueError(f"Irreps in and number of activation functions does not match: {len(acts), (irreps_in, acts)}")
        names = [activation_name(a) for a in acts]
        given = [a is not None for a in acts]
        self.irreps_in = irreps_in
        self.irreps_out = _act_irreps_out(irreps_in, names, given)
        blocks = []
        for (mul, ir), sl, name in zip(irreps_in, irreps_in.slices(), names):
            blocks.append((sl.start, sl.start, mul * ir.dim, _KINDS[name], second_moment_constant(name)))
        self._set_tables(blocks, [], irreps_in.dim, irreps_in.dim)
        self._repr = "".join("x" if g else " " for g in given)

    def __repr__(self) -> str:
        return f"{self.__class__.__name__} [{self._repr}] ({self.irreps_in} -> {self.irreps_out})"


class Gate(_BlockModule):
    """Gate activation function (``e3nn/nn/_gate.py:35-154``): input rows hold ``irreps_scalars + irreps_gates +
    irreps_gated`` sorted by ``(l, p)`` and simplified, output rows ``act(scalars) + act(gates) * gated``."""

    def __init__(self, irreps_scalars, act_scalars, irreps_gates, act_gates, irreps_gated) -> None:
        super().__init__()
        irreps_scalars, irreps_gates, irreps_gated = Irreps(irreps_scalars), Irreps(irreps_gates), Irreps(irreps_gated)
        if len(irreps_gates) > 0 and irreps_gates.lmax > 0:
            raise ValueError(f"Gate scalars must be scalars, instead got irreps_gates = {irreps_gates}")
        if len(irreps_scalars) > 0 and irreps_scalars.lmax > 0:
            raise ValueError(f"Scalars must be scalars, instead got irreps_scalars = {irreps_scalars}")
        if irreps_gates.num_irreps != irreps_gated.num_irreps:
            raise ValueError(
                f"There are {irreps_gated.num_irreps} irreps in irreps_gated, but a different number "
                f"({irreps_gates.num_irreps}) of gate scalars in irreps_gates"
            )
        if len(irreps_scalars) != len(act_scalars) or len(irreps_gates) != len(act_gates):
            raise ValueError("one activation function per irrep of irreps_scalars and of irreps_gates")
        # the reference applies the activations to the irreps as given and sorts the *simplified* groups
        # (_gate.py:10-24,103-116)
        names_s, names_g = [activation_name(a) for a in act_scalars], [activation_name(a) for a in act_gates]
        groups = [irreps_scalars, irreps_gates, irreps_gated]
        # the reference multiplies gates and gated irreps with an ElementwiseTensorProduct submodule `mul`, whose
        # (empty) weight and output mask are in its state_dict
        self.mul = torch.nn.Module()
        self.mul.register_buffer("weight", torch.Tensor())
        self.mul.register_buffer("output_mask", torch.ones(Irreps(irreps_gated).dim))
        simplified = [g.simplify() for g in groups]
        self.irreps_scalars, self.irreps_gates, self.irreps_gated = simplified
        cat = sum(simplified, Irreps([]))
        sorted_in, p, _ = cat.sort()
        in_slices = sorted_in.slices()
        self._irreps_in = sorted_in.simplify()
        pos = 0
        starts = []  # column of every entry of the simplified (scalars, gates, gated) in the sorted input rows
        for g in simplified:
            starts.append([in_slices[p[pos + i]].start for i in range(len(g))])
            pos += len(g)

        def columns_as_given(group, simple, simple_starts):
            # simplify() joins neighbouring entries of one irrep and keeps the order of the columns, so an entry as given
            # sits inside one simplified entry, behind the entries joined before it
            cols, si, used = [], 0, 0
            for mul, ir in group:
                if mul == 0:
                    cols.append(0)
                    continue
                cols.append(simple_starts[si] + used * ir.dim)
                used += mul
                if used == simple[si].mul:
                    si, used = si + 1, 0
            return cols

        # the activations act on the irreps as given: neighbouring entries of one irrep may carry different functions
        out_scalars = _act_irreps_out(irreps_scalars, names_s, [a is not None for a in act_scalars])
        out_gates = _act_irreps_out(irreps_gates, names_g, [a is not None for a in act_gates])
        acts, col = [], 0
        for (mul, ir), start, name in zip(irreps_scalars, columns_as_given(irreps_scalars, simplified[0], starts[0]), names_s):
            if mul:
                acts.append((start, col, mul, _KINDS[name], second_moment_constant(name)))
            col += mul
        # one record per gate scalar: its column, activation and the parity of the activated scalar
        gate_copies = []
        for (mul, ir), (_, ir_out), start, name in zip(irreps_gates, out_gates, columns_as_given(irreps_gates, simplified[1], starts[1]), names_g):
            gate_copies += [(start + u, _KINDS[name], second_moment_constant(name), ir_out.p) for u in range(mul)]
        # kernel blocks: gates and gated irreps are paired copy by copy; a block is a run of copies of one gated entry
        # whose gate scalars are neighbours and share an activation
        gate_blocks, u = [], 0
        for (mul_y, ir_y), start_y in zip(simplified[2], starts[2]):
            k = 0
            while k < mul_y:
                g_col, kind, cst, _ = gate_copies[u + k]
                n = 1
                while k + n < mul_y and gate_copies[u + k + n][:3] == (g_col + n, kind, cst):
                    n += 1
                gate_blocks.append((g_col, start_y + k * ir_y.dim, col + k * ir_y.dim, n, ir_y.dim, kind, cst))
                k += n
            col += mul_y * ir_y.dim
            u += mul_y
        # output irreps of the gated part: the reference's ElementwiseTensorProduct of the simplified gated irreps and the
        # simplified activated gates, runs split where their multiplicities differ (e3nn/o3/_tensor_product/_sub.py:103-142)
        left_y = [[mul, ir] for mul, ir in simplified[2]]
        left_g = [[mul, ir] for mul, ir in out_gates.simplify()]
        out_gated, gi = [], 0
        for mul_y, ir_y in left_y:
            while mul_y > 0:
                n = min(mul_y, left_g[gi][0])
                out_gated.append((n, Irrep(ir_y.l, ir_y.p * left_g[gi][1].p)))
                mul_y -= n
                left_g[gi][0] -= n
                if left_g[gi][0] == 0:
                    gi += 1
        self._irreps_out = out_scalars + Irreps(out_gated)
        assert col == self._irreps_out.dim
        self._set_tables(acts, gate_blocks, self._irreps_in.dim, col)

    def __repr__(self) -> str:
        return f"{self.__class__.__name__} ({self.irreps_in} -> {self.irreps_out})"

    @property
    def irreps_in(self):
        return self._irreps_in

    @property
    def irreps_out(self):
        return self._irreps_out
