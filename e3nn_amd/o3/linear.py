"""``o3.Linear``: the equivariant linear map of the reference (``e3nn/o3/_linear.py:27-260``), run as a ``uvw`` tensor
product with a constant ``0e`` second input.

For a path ``i_in -> i_out`` the reference computes ``alpha^(-1/2) * einsum("uw,zui->zwi", W, x)`` with ``alpha`` the
fan-in (``_linear.py:152-165``).  The tensor product ``x (x) 1`` with instruction ``(i_in, 0, i_out, "uvw")`` has the
Clebsch-Gordan tensor ``delta / sqrt(2l+1)`` and, under component normalisation, the path weight
``sqrt((2l+1) / fan_in)``: the same map, with the same ``[mul_in, mul_out]`` weight blocks in the same order.  So the
matrix-core ``uvw`` kernels (forward, input gradient, weight gradient) serve linear layers unchanged.
"""
from typing import List, NamedTuple, Optional, Tuple, Union

import torch

from .irreps import Irreps
from .tensor_product import TensorProduct


class Instruction(NamedTuple):
    i_in: int
    i_out: int
    path_shape: tuple
    path_weight: float


class Linear(torch.nn.Module):
    r"""Linear operation equivariant to :math:`O(3)`; same arguments as the reference's ``o3.Linear`` except ``f_in`` /
    ``f_out`` (not implemented)."""

    def __init__(
        self,
        irreps_in,
        irreps_out,
        *,
        f_in: Optional[int] = None,
        f_out: Optional[int] = None,
        internal_weights: Optional[bool] = None,
        shared_weights: Optional[bool] = None,
        instructions: Optional[List[Tuple[int, int]]] = None,
        biases: Union[bool, List[bool]] = False,
        path_normalization: str = "element",
        _optimize_einsums: Optional[bool] = None,
    ) -> None:
        super().__init__()
        assert path_normalization in ["element", "path"]
        if (f_in is None) != (f_out is None):
            raise ValueError("Linear: f_in and f_out come together")
        self.f_in, self.f_out = f_in, f_out
        irreps_in, irreps_out = Irreps(irreps_in), Irreps(irreps_out)
        if instructions is None:  # every pair of blocks that carry the same irrep
            instructions = [(a, b) for a, x in enumerate(irreps_in) for b, y in enumerate(irreps_out) if x.ir == y.ir]
        for a, b in instructions:
            for index, irreps, name in ((a, irreps_in, "irreps_in"), (b, irreps_out, "irreps_out")):
                if index >= len(irreps):
                    raise IndexError(f"{index} is not a valid index for {name}")
            if irreps_in[a].ir != irreps_out[b].ir:
                raise ValueError(f"{a} and {b} do not have the same irrep")

        def alpha(i_in, i_out) -> float:
            x = sum(irreps_in[a if path_normalization == "element" else i_in].mul for a, b in instructions if b == i_out)
            x *= 1 if f_in is None else f_in  # every input channel feeds every output channel (_linear.py:158-159)
            return 1.0 if x == 0 else x

        self.instructions = [
            Instruction(i_in, i_out, (irreps_in[i_in].mul, irreps_out[i_out].mul), alpha(i_in, i_out) ** (-0.5))
            for i_in, i_out in instructions
        ]
        if biases is None or isinstance(biases, bool):  # one flag: a bias on every scalar output block
            biases = [bool(biases) and ir.is_scalar() for _, ir in irreps_out]
        assert len(biases) == len(irreps_out)
        assert all(ir.is_scalar() for flag, (_, ir) in zip(biases, irreps_out) if flag), "only scalars take a bias"
        self._bias_slices = [sl for b, sl in zip(biases, irreps_out.slices()) if b]
        self.instructions += [
            Instruction(-1, i_out, (mul_ir.dim,), 1.0) for i_out, (b, mul_ir) in enumerate(zip(biases, irreps_out)) if b
        ]

        # weights are shared over the batch unless the caller says otherwise, and the module owns them exactly when
        # they are shared (unless the caller says otherwise); per-sample weights cannot be parameters
        shared_weights = True if shared_weights is None else bool(shared_weights)
        internal_weights = shared_weights if internal_weights is None else bool(internal_weights)
        assert shared_weights or not internal_weights
        self.internal_weights, self.shared_weights = internal_weights, shared_weights
        self.irreps_in, self.irreps_out = irreps_in, irreps_out

        # the same map as a tensor product with "0e": the reference's own normalisation formula for TensorProduct
        # (component / element or path) reproduces alpha^(-1/2) once the delta / sqrt(2l+1) of the 3j tensor is counted
        # (kept out of the module tree: the reference's Linear has no such submodule in its state_dict)
        # With f_in / f_out the features are [..., f_in, irreps_in.dim] -> [..., f_out, irreps_out.dim] and the weights
        # [f_in, f_out, weight_numel] (_linear.py:226, :445-448): the same product on f_in * mul copies of every input
        # irrep and f_out * mul copies of every output irrep, once the columns are regrouped irrep by irrep.
        fi, fo = (1, 1) if f_in is None else (f_in, f_out)
        wide_in = Irreps([(fi * mul, ir) for mul, ir in irreps_in])
        wide_out = Irreps([(fo * mul, ir) for mul, ir in irreps_out])
        object.__setattr__(self, "_tp", TensorProduct(
            wide_in, "0e", wide_out, [(i, 0, o, "uvw", True) for i, o in instructions],
            path_normalization=path_normalization, internal_weights=False, shared_weights=shared_weights,
        ))  # fmt: skip
        if f_in is not None:
            def regroup(irreps, f):  # position in the wide row -> position in the flattened [f, irreps.dim] features
                cols = [c * irreps.dim + sl.start + j for sl in irreps.slices() for c in range(f) for j in range(sl.stop - sl.start)]
                return torch.tensor(cols, dtype=torch.long)

            self.register_buffer("_cols_in", regroup(irreps_in, f_in), persistent=False)
            cols_out = regroup(irreps_out, f_out)
            self.register_buffer("_cols_out", torch.argsort(cols_out), persistent=False)
        self.weight_numel = self._tp.weight_numel // (fi * fo)
        self.bias_numel = sum(sl.stop - sl.start for sl in self._bias_slices)
        if internal_weights and self.weight_numel > 0:
            self.weight = torch.nn.Parameter(torch.randn(*(() if f_in is None else (f_in, f_out)), self.weight_numel))
        else:
            self.register_buffer("weight", torch.Tensor())
        if internal_weights and self.bias_numel > 0:
            self.bias = torch.nn.Parameter(torch.zeros(*(() if f_out is None else (f_out,)), self.bias_numel))
        else:
            self.register_buffer("bias", torch.Tensor())
        mask = self._tp.output_mask.clone()
        if f_in is not None:  # the reference's mask is that of one output channel
            mask = torch.cat([mask[f_out * sl.start : f_out * sl.start + (sl.stop - sl.start)] for sl in irreps_out.slices()]) if len(irreps_out) else mask[:0]
        self.register_buffer("output_mask", mask)

    def __repr__(self) -> str:
        return f"{self.__class__.__name__}({self.irreps_in} -> {self.irreps_out} | {self.weight_numel} weights)"

    def forward(self, features, weight: Optional[torch.Tensor] = None, bias: Optional[torch.Tensor] = None):
        if weight is None:
            if self.weight_numel > 0 and not self.internal_weights:
                raise RuntimeError("Weights must be provided when internal_weights = False")
            weight = self.weight
        if bias is None:
            if self.bias_numel > 0 and not self.internal_weights:
                raise RuntimeError("Biases must be provided when internal_weights = False")
            bias = self.bias
        if self.f_in is not None:
            return self._forward_channels(features, weight, bias)
        ones = features.new_ones(features.shape[:-1] + (1,))
        out = self._tp(features, ones, weight)
        if self.bias_numel > 0:
            off = 0
            out = out.clone()
            for sl in self._bias_slices:
                n = sl.stop - sl.start
                out[..., sl] += bias[..., off : off + n]
                off += n
        return out

    def _forward_channels(self, features, weight, bias):
        f_in, f_out = self.f_in, self.f_out
        lead = features.shape[:-2]
        x = features.reshape(*lead, f_in * self.irreps_in.dim)[..., self._cols_in]
        # weights [..., f_in, f_out, numel] -> per instruction [f_in * U, f_out * W], row-major, instruction after instruction
        blocks, off = [], 0
        for ins in self.instructions:
            if ins.i_in == -1:
                continue
            U, W = ins.path_shape
            blk = weight[..., off : off + U * W].reshape(*weight.shape[:-3], f_in, f_out, U, W)
            blocks.append(blk.transpose(-3, -2).reshape(*weight.shape[:-3], f_in * U * f_out * W))
            off += U * W
        wide_w = torch.cat(blocks, dim=-1) if blocks else weight.new_zeros(*weight.shape[:-3], 0)
        out = self._tp(x, x.new_ones(*lead, 1), wide_w)[..., self._cols_out].reshape(*lead, f_out, self.irreps_out.dim)
        if self.bias_numel > 0:
            off = 0
            out = out.clone()
            for sl in self._bias_slices:
                n = sl.stop - sl.start
                out[..., sl] += bias[..., off : off + n]
                off += n
        return out

    def weight_view_for_instruction(self, instruction: int, weight: Optional[torch.Tensor] = None) -> torch.Tensor:
        weight = self.weight if weight is None else weight
        ins = self.instructions[instruction]
        if ins.i_in == -1:
            raise ValueError(f"Instruction {instruction} is a bias")
        off = sum(i.path_shape[0] * i.path_shape[1] for i in self.instructions[:instruction] if i.i_in != -1)
        n = ins.path_shape[0] * ins.path_shape[1]
        return weight.narrow(-1, off, n).view(weight.shape[:-1] + ins.path_shape)

    def weight_views(self, weight: Optional[torch.Tensor] = None, yield_instruction: bool = False):
        for i, ins in enumerate(self.instructions):
            if ins.i_in != -1:
                v = self.weight_view_for_instruction(i, weight)
                yield (i, ins, v) if yield_instruction else v
