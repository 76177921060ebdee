"""The binding an e3nn maintainer would add: code-generation providers that serve ``TensorProduct`` from libe3x.

e3nn asks every entry of ``e3nn.o3._tensor_product._tensor_product._CODEGEN_PROVIDERS_LEFT_RIGHT``
(e3nn/o3/_tensor_product/_tensor_product.py:17-21) for an ``fx.GraphModule`` that is later called as
``mod(x1, x2, w)`` (:348-361, :554), and every entry of ``_CODEGEN_PROVIDERS_RIGHT`` for one called as
``mod(x2, w)`` (:376-389, :527).  ``hip_provider`` / ``hip_provider_right`` answer for every instruction set the
library has a kernel for and return ``None`` otherwise, which defers to the next provider (e3nn's own einsum code
generator).

The module a provider returns honours what e3nn does with its generated modules:

* it is differentiable -- the call goes through the same ``torch.autograd.Function`` as this package's own
  ``TensorProduct`` (gradients of all three arguments), so a model built on e3nn trains;
* it pickles and deep-copies -- ``CodeGenMixin.__getstate__`` (e3nn/util/codegen/_mixin.py:55-99) runs
  ``pickle.dumps`` on every generated submodule; what is stored here is the constructor data (irreps, instructions,
  ``shared_weights``), and the kernels' plan handles are rebuilt on first use after loading;
* it refuses what the kernels do not take (CPU tensors, float64, mixed dtypes) with a ``RuntimeError`` instead of
  handing a foreign pointer to the GPU.

Nothing here imports e3nn: the functions take e3nn's objects by their attributes (``Irreps`` iterate as
``(mul, ir)`` with ``ir.l`` / ``ir.p``; ``Instruction`` has ``i_in1, i_in2, i_out, connection_mode, has_weight,
path_weight, path_shape``), which this package's own classes share, so the binding is exercised by this repository's
tests.

    import e3nn.o3._tensor_product._tensor_product as m
    from e3nn_amd.provider import register
    register(m._CODEGEN_PROVIDERS_LEFT_RIGHT, m._CODEGEN_PROVIDERS_RIGHT)   # o3.TensorProduct(...) now runs on the HIP kernels
"""
import torch
from torch import fx

from . import _lib

_DTYPES = {torch.float32: _lib.F32, torch.bfloat16: _lib.BF16}


class HipTensorProduct(torch.nn.Module):
    """The module the fx graph calls: ``forward(x1 [..., dim1], x2 [..., dim2], w)`` for the left-right provider,
    ``forward(x2, w)`` (the matrices ``[..., dim1, dim_out]``) for the right provider.

    Holds nothing but plain Python data (three irreps lists, the instruction table with e3nn's final path weights,
    two flags).  The kernels are reached through an engine -- this package's ``TensorProduct`` built from that data
    with every normalisation switched off -- which is created on first use, lives outside ``state_dict`` and
    ``_modules``, and is left out of pickles and copies."""

    def __init__(self, irreps_in1, irreps_in2, irreps_out, instructions, shared_weights, right=False):
        super().__init__()
        flat = lambda irreps: tuple((int(mul), int(ir.l), int(ir.p)) for mul, ir in irreps)  # noqa: E731
        self.irreps = (flat(irreps_in1), flat(irreps_in2), flat(irreps_out))
        self.instructions = tuple(
            (int(t.i_in1), int(t.i_in2), int(t.i_out), str(t.connection_mode), bool(t.has_weight), float(t.path_weight))
            for t in instructions
        )
        self.shared_weights = bool(shared_weights)
        self.is_right = bool(right)
        self._engine = []  # [TensorProduct] once built; a list so that torch.nn.Module does not register it
        tp = self.engine()
        self.weight_numel, self.in1_dim, self.in2_dim, self.out_dim = tp.weight_numel, tp.irreps_in1.dim, tp.irreps_in2.dim, tp.irreps_out.dim

    def engine(self):
        if not self._engine:
            from .o3 import Irreps, TensorProduct

            in1, in2, out = (Irreps([(mul, (l, p)) for mul, l, p in rows]) for rows in self.irreps)
            # sqrt(pw * pw) == pw in binary floating point: the engine's normalisation returns e3nn's path weights
            ins = [(a, b, c, mode, hw, pw * pw) for a, b, c, mode, hw, pw in self.instructions]
            tp = TensorProduct(
                in1, in2, out, ins, irrep_normalization="none", path_normalization="none", internal_weights=False,
                shared_weights=self.shared_weights, compile_right=self.is_right,  # right() runs on the forward kernel
            )  # fmt: skip
            assert all(abs(t.path_weight - row[5]) <= 1e-15 * abs(row[5]) for t, row in zip(tp.instructions, self.instructions))
            tp.compile(torch.float32)  # refusals of the library surface here, as E3xError
            self._engine.append(tp)
        return self._engine[0]

    def __getstate__(self):
        state = self.__dict__.copy()
        state["_engine"] = []
        return state

    def extra_repr(self):
        return f"{len(self.instructions)} instructions, shared_weights={self.shared_weights}, right={self.is_right}"

    def _check(self, x, w):
        tensors = [t for t in (*x, w) if t.numel() > 0]
        for t in tensors:
            if not t.is_cuda:
                raise RuntimeError("the HIP tensor product runs on GPU tensors only; got a tensor on " + str(t.device))
            if t.dtype not in _DTYPES:
                raise RuntimeError(f"the HIP tensor product takes float32 or bfloat16 storage, got {t.dtype}")
        if len({t.dtype for t in tensors}) > 1 or len({t.device for t in tensors}) > 1:
            raise RuntimeError("inputs and weights of the HIP tensor product must share one dtype and one device")

    def forward(self, *args):
        """Leading dimensions broadcast as in e3nn's generated code (_codegen.py:43-76); ``w`` is ``[weight_numel]``
        for shared weights, ``[..., weight_numel]`` otherwise (an empty tensor when there are no weights, :410)."""
        *x, w = args
        self._check(x, w)
        tp = self.engine()
        w = w if self.weight_numel else None
        return tp.right(x[0], w) if self.is_right else tp(x[0], x[1], w)


def _graph_module(mod, names):
    graph = fx.Graph()  # the hook requires an fx.GraphModule (e3nn/util/codegen/_mixin.py:40)
    args = tuple(graph.placeholder(name) for name in names)
    graph.output(graph.call_module("hip", args))
    root = torch.nn.Module()
    root.hip = mod
    return fx.GraphModule(root, graph, "tp_forward")


def _provide(irreps_in1, irreps_in2, irreps_out, instructions, shared_weights, right):
    live = [t for t in instructions if 0 not in t.path_shape]  # dropped by e3nn too (_codegen.py:51)
    if not live:
        return None
    try:
        mod = HipTensorProduct(irreps_in1, irreps_in2, irreps_out, live, shared_weights, right=right)
    except (_lib.E3xError, NotImplementedError):
        return None  # no kernel for this instruction set: the next provider answers
    return _graph_module(mod, ("x2", "w") if right else ("x1", "x2", "w"))


def hip_provider(irreps_in1, irreps_in2, irreps_out, instructions, shared_weights, specialized_code, optimize_einsums):
    """Provider for ``_CODEGEN_PROVIDERS_LEFT_RIGHT``; ``None`` when the library has no kernel for the instruction set
    (the plan is refused) or nothing to compute."""
    return _provide(irreps_in1, irreps_in2, irreps_out, instructions, shared_weights, right=False)


def hip_provider_right(irreps_in1, irreps_in2, irreps_out, instructions, shared_weights, specialized_code, optimize_einsums):
    """Provider for ``_CODEGEN_PROVIDERS_RIGHT``: ``mod(x2, w) -> [..., irreps_in1.dim, irreps_out.dim]``
    (_tensor_product.py:447-527; code generator _codegen.py:398-717)."""
    return _provide(irreps_in1, irreps_in2, irreps_out, instructions, shared_weights, right=True)


def register(providers_left_right: list, providers_right: list = None) -> None:
    """Puts the HIP providers in front of e3nn's own code generators."""
    if hip_provider not in providers_left_right:
        providers_left_right.insert(0, hip_provider)
    if providers_right is not None and hip_provider_right not in providers_right:
        providers_right.insert(0, hip_provider_right)
