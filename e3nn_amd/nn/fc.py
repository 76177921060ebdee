"""``nn.FullyConnectedNet`` (``e3nn/nn/_fc.py:9-88``): dense layers ``x @ W / sqrt(h_in)`` with a second-moment
normalised activation.  A dense layer of scalars is the ``uvw`` tensor product ``h_in x0e (x) 0e -> h_out x0e``, so each
layer runs on the tensor-product kernels (matrix cores when h_in and h_out are multiples of 32) and the activation on
the gate kernel; parameter names and shapes (``layer{i}.weight [h_in, h_out]``) are the reference's.
"""
import torch

from ..o3.tensor_product import TensorProduct
from .activation import Activation, activation_name


class _Layer(torch.nn.Module):
    def __init__(self, h_in, h_out, act, var_in, var_out) -> None:
        super().__init__()
        self.weight = torch.nn.Parameter(torch.randn(h_in, h_out))
        self.h_in, self.h_out, self.var_in, self.var_out = h_in, h_out, var_in, var_out
        self._act_name = None if act is None else activation_name(act)
        # path weight of the tensor product: 1 / sqrt(h_in); the variance factors of _fc.py:41-48 ride on top
        self._tp = TensorProduct(
            f"{h_in}x0e", "0e", f"{h_out}x0e", [(0, 0, 0, "uvw", True)], internal_weights=False, shared_weights=True
        )
        self.act = None if act is None else Activation(f"{h_out}x0e", [self._act_name])

    def __repr__(self) -> str:
        return f"Layer({self.h_in}->{self.h_out}, act={self._act_name})"

    def forward(self, x: torch.Tensor):
        ones = x.new_ones(x.shape[:-1] + (1,))
        if self.act is not None:
            x = self._tp(x, ones, self.weight.reshape(-1))
            if self.var_in != 1:
                x = x / self.var_in**0.5
            x = self.act(x)
            if self.var_out != 1:
                x = x * self.var_out**0.5
        else:
            x = self._tp(x, ones, self.weight.reshape(-1))
            if self.var_in != self.var_out:
                x = x * (self.var_out / self.var_in) ** 0.5
        return x


class FullyConnectedNet(torch.nn.Sequential):
    r"""Fully-connected network ``hs[0] -> hs[1] -> ... -> hs[-1]``; ``act`` is normalised to unit second moment."""

    def __init__(self, hs, act=None, variance_in: int = 1, variance_out: int = 1, out_act: bool = False) -> None:
        super().__init__()
        self.hs = list(hs)
        var_in = variance_in
        for i, (h1, h2) in enumerate(zip(self.hs, self.hs[1:])):
            if i == len(self.hs) - 2:
                var_out = variance_out
                a = act if out_act else None
            else:
                var_out = 1
                a = act
            setattr(self, f"layer{i}", _Layer(h1, h2, a, var_in, var_out))
            var_in = var_out

    def __repr__(self) -> str:
        return f"{self.__class__.__name__}{self.hs}"
