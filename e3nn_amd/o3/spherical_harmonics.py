"""Spherical harmonics as polynomials of x, y, z, evaluated by a HIP kernel.

API of the reference's ``e3nn.o3.SphericalHarmonics`` / ``e3nn.o3.spherical_harmonics``
(e3nn/o3/_spherical_harmonics.py:14-112, :115-190).
"""
import ctypes
from typing import Any, List, Union

import torch
from torch.autograd.function import once_differentiable

from .. import _lib
from .irreps import Irreps

_NORMALIZATION = {"integral": _lib.NORM_INTEGRAL, "component": _lib.NORM_COMPONENT, "norm": _lib.NORM_NORM}


def _launch(entry, ls, normalize, normalization, n, device, *tensors):
    arr = (ctypes.c_int32 * len(ls))(*ls)
    with torch.cuda.device(device):
        _lib.check(
            getattr(_lib.lib(), entry)(
                arr, len(ls), int(bool(normalize)), _NORMALIZATION[normalization], *[_lib.ptr(t) for t in tensors], n,
                _lib.F32, _lib.stream_ptr(device),
            )  # fmt: skip
        )


class _SphericalHarmonicsFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, ls, normalize, normalization):
        if not x.is_cuda:
            raise RuntimeError("e3nn_amd.o3.spherical_harmonics runs on the GPU only; got a CPU tensor")
        if x.dtype != torch.float32:
            raise TypeError(f"spherical_harmonics kernel supports float32 input, got {x.dtype}")
        batch = x.shape[:-1]
        xyz = x.reshape(-1, 3).contiguous()
        n = xyz.shape[0]
        n_out = sum(2 * l + 1 for l in ls)
        out = torch.empty(n, n_out, dtype=x.dtype, device=x.device)
        _launch("e3x_sh_forward", ls, normalize, normalization, n, x.device, xyz, out)
        ctx.save_for_backward(x)
        ctx.cfg = (ls, normalize, normalization)
        return out.reshape(batch + (n_out,))

    @staticmethod
    def backward(ctx, g):
        (x,) = ctx.saved_tensors
        return _ShBackwardFn.apply(x, g, *ctx.cfg), None, None, None


class _ShBackwardFn(torch.autograd.Function):
    """``(x, g) -> grad_x <g, Y(x)>``, itself differentiable once more (``e3x_sh_backward2``): what a loss on forces
    differentiates.  Third derivatives are not provided."""

    @staticmethod
    def forward(ctx, x, g, ls, normalize, normalization):
        batch = x.shape[:-1]
        xyz = x.reshape(-1, 3).contiguous()
        n = xyz.shape[0]
        g2 = g.reshape(n, sum(2 * l + 1 for l in ls)).contiguous()  # the width spelled out: -1 is ambiguous for n = 0
        gx = torch.empty_like(xyz)
        _launch("e3x_sh_backward", ls, normalize, normalization, n, x.device, xyz, g2, gx)
        ctx.save_for_backward(xyz, g2)
        ctx.cfg = (ls, normalize, normalization, batch, g.shape)
        return gx.reshape(batch + (3,))

    @staticmethod
    @once_differentiable
    def backward(ctx, cot):
        xyz, g = ctx.saved_tensors
        ls, normalize, normalization, batch, g_shape = ctx.cfg
        if tuple(ls) != tuple(range(len(ls))) or len(ls) > 4:
            raise NotImplementedError("second derivatives of the spherical harmonics are implemented for l = 0 .. lmax <= 3")
        n = xyz.shape[0]
        cot = cot.reshape(n, 3).contiguous()
        gg, gx = torch.empty_like(g), torch.empty_like(xyz)
        _launch("e3x_sh_backward2", ls, normalize, normalization, n, xyz.device, xyz, g, cot, gg, gx)
        return gx.reshape(batch + (3,)), gg.reshape(g_shape), None, None, None


def _sh_forward(x, ls, normalize, normalization):
    return _SphericalHarmonicsFn.apply(x, tuple(ls), normalize, normalization)


def _sh_backward(x, g, ls, normalize, normalization):
    return _ShBackwardFn.apply(x, g, tuple(ls), normalize, normalization)


class SphericalHarmonics(torch.nn.Module):
    """Module version of :func:`spherical_harmonics`; parameters as in the reference (:28-34)."""

    def __init__(
        self,
        irreps_out: Union[int, List[int], str, Irreps],
        normalize: bool,
        normalization: str = "integral",
        irreps_in: Any = None,
    ) -> None:
        super().__init__()
        self.normalize = normalize
        self.normalization = normalization
        assert normalization in ["integral", "component", "norm"]

        if isinstance(irreps_out, str):
            irreps_out = Irreps(irreps_out)
        if isinstance(irreps_out, Irreps) and irreps_in is None:
            # an odd-l even-parity output can only come from a pseudovector input
            if any(l % 2 == 1 and p == 1 for _, (l, p) in irreps_out):
                irreps_in = Irreps("1e")
        if irreps_in is None:
            irreps_in = Irreps("1o")
        irreps_in = Irreps(irreps_in)
        if irreps_in not in (Irreps("1x1o"), Irreps("1x1e")):
            raise ValueError(
                f"irreps_in for SphericalHarmonics must be either a vector (`1x1o`) or a pseudovector (`1x1e`), "
                f"not `{irreps_in}`"
            )
        self.irreps_in = irreps_in
        input_p = irreps_in[0].ir.p

        if isinstance(irreps_out, Irreps):
            ls = []
            for mul, (l, p) in irreps_out:
                if p != input_p**l:
                    raise ValueError(
                        f"irreps_out `{irreps_out}` passed to SphericalHarmonics asked for an output of l = {l} with "
                        f"parity p = {p}, which is inconsistent with the input parity {input_p} — the output parity "
                        f"should have been p = {input_p**l}"
                    )
                ls.extend([l] * mul)
        elif isinstance(irreps_out, int):
            ls = [irreps_out]
        else:
            ls = list(irreps_out)

        self.irreps_out = Irreps([(1, (l, input_p**l)) for l in ls]).simplify()
        self._ls_list = ls
        self._lmax = max(ls)
        if self._lmax > 12:
            raise NotImplementedError("spherical_harmonics maximum l implemented is 12, send us an email to ask for more")

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return _SphericalHarmonicsFn.apply(x, tuple(self._ls_list), self.normalize, self.normalization)


def spherical_harmonics(
    l: Union[int, List[int], str, Irreps], x: torch.Tensor, normalize: bool, normalization: str = "integral"
) -> torch.Tensor:
    r"""Spherical harmonics :math:`Y^l(x)` of the vectors ``x[..., 3]``; output ``[..., sum(2l+1)]``.

    ``normalize`` projects ``x`` onto the unit sphere first (the zero vector gives the
    l = 0 constant and zeros elsewhere); ``normalization`` is ``'integral'``,
    ``'component'`` (:math:`\|Y^l\|^2 = 2l+1` on the sphere) or ``'norm'``.
    """
    return SphericalHarmonics(l, normalize, normalization)(x)
