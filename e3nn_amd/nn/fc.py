"""``nn.FullyConnectedNet`` (``e3nn/nn/_fc.py:9-88``): dense layers ``x @ W / sqrt(h_in)`` with a second-moment
normalised activation; parameter names and shapes (``layer{i}.weight [h_in, h_out]``) are the reference's.

Two device paths, both HIP kernels of this package:

* no gradient wanted (inference, or nothing upstream requires one): the whole network runs as ONE kernel that
  keeps the hidden activations in registers (``e3x_fc_forward``);
* otherwise the network runs layer by layer and keeps what the backward pass needs.  A dense layer is the same
  kernel specialised to one layer, forward (``x @ W``) and for the input gradient (``g @ W^T``); the weight gradient
  is that of the ``uvw`` tensor product ``h_in x0e (x) 0e -> h_out x0e``; the activation is the gate kernel.
  Layers outside the one-kernel limits run on the tensor-product kernels throughout.
"""
import ctypes

import torch

from .. import _lib
from ..o3.tensor_product import TensorProduct
from .activation import _KINDS, Activation, activation_name, second_moment_constant


_X, _WT, _G = 0, 1, 2


def _dense_member(layer, slot, a, b):
    """One of the three maps of the bilinear form ``F(x, W, g) = <g, x @ W * s>`` of a layer (``s`` is folded in by the
    plans): ``_G``: ``x @ W * s``; ``_X``: ``g @ W^T * s``; ``_WT``: ``x^T @ g * s``; ``a, b`` are the other two slots in
    the order (x, W, g)."""
    if slot == _G:
        return layer._fwd.forward(a, [b.contiguous()])
    if slot == _X:  # g @ W^T * s through the plan [h_out -> h_in], whose own factor is 1 / sqrt(h_out)
        w, g = a, b.contiguous()
        g = g.clone() if g.data_ptr() % 16 else g
        return layer._bwd.forward(g, [(w.t() * (layer._scale * layer.h_out**0.5)).contiguous()])
    x, g = a.contiguous(), b.contiguous()
    x, g = (t.clone() if t.data_ptr() % 16 else t for t in (x, g))
    if layer._fwd.has_backward_w:
        return layer._fwd.backward_w(x, g)
    # wider than the dense weight-gradient kernel takes: the uvw weight gradient of the same layer
    ones = x.new_ones(x.shape[0], 1)
    gw = layer._tp._plan(torch.float32).backward_w_uvw(x, ones, g, True).reshape(layer.h_in, layer.h_out)
    return gw * (layer._scale * layer.h_in**0.5)  # the tensor product's path weight is 1 / sqrt(h_in)


class _DenseSlot(torch.autograd.Function):
    """Member ``slot`` of the closed family of one dense layer (see ``_dense_member``): the derivative of a member with
    respect to one of its arguments is another member, so derivatives of every order run on the same three kernels."""

    @staticmethod
    def forward(ctx, slot, layer, a, b):
        ctx.slot, ctx.layer = slot, layer
        ctx.save_for_backward(a, b)
        return _dense_member(layer, slot, a, b)

    @staticmethod
    def backward(ctx, cot):
        others = [t for t in range(3) if t != ctx.slot]
        full = {ctx.slot: cot.contiguous(), **dict(zip(others, ctx.saved_tensors))}
        grads = []
        for t, need in zip(others, ctx.needs_input_grad[2:4]):
            grads.append(_DenseSlot.apply(t, ctx.layer, *[full[u] for u in range(3) if u != t]) if need else None)
        return (None, None, *grads)


class _DenseFn:
    """``x @ W * s`` of one layer on the one-layer specialisations of the fused kernel, under autograd."""

    @staticmethod
    def apply(x, w, layer):
        return _DenseSlot.apply(_G, layer, x, w)


class _ActDenseFn(torch.autograd.Function):
    """``dense(act(z))`` of two consecutive layers without the activated tensor: the dense kernel applies the
    activation to its input rows as it loads them (forward and weight gradient), and the backward pass takes the input
    gradient through the activation in the epilogue of the input-gradient kernel, ``(g @ W^T * s) * cst * act'(z)``.
    Under ``create_graph`` the backward pass is the differentiable composition of the activation's and the dense
    layer's own gradients instead (the activated tensor is then formed)."""

    @staticmethod
    def forward(ctx, z, w, layer, prev):
        ctx.plans = layer.act_dense_plans(prev)
        ctx.scale = layer._scale * layer.h_out**0.5
        ctx.layer, ctx.prev = layer, prev
        ctx.save_for_backward(z, w)
        return ctx.plans[0].forward(z, [w.contiguous()])

    @staticmethod
    def backward(ctx, g):
        z, w = ctx.saved_tensors
        fwd, bwd = ctx.plans
        g = g.contiguous()
        if g.data_ptr() % 16:
            g = g.clone()
        if torch.is_grad_enabled():
            from .activation import _GateBackwardFn

            h = ctx.prev.act(z)  # differentiable in z
            gz = gw = None
            if ctx.needs_input_grad[0]:
                gz = _GateBackwardFn.apply(z, _DenseSlot.apply(_X, ctx.layer, w, g), ctx.prev.act)
            if ctx.needs_input_grad[1]:
                gw = _DenseSlot.apply(_WT, ctx.layer, h, g)
            return gz, gw, None, None
        gz = gw = None
        if ctx.needs_input_grad[0]:
            gz = bwd.forward(g, [(w.t() * ctx.scale).contiguous()], z)
        if ctx.needs_input_grad[1]:
            gw = fwd.backward_w(z, g)
        return gz, gw, None, None


class _Layer(torch.nn.Module):
    def __init__(self, h_in, h_out, act, var_in, var_out) -> None:
        super().__init__()
        self.weight = torch.nn.Parameter(torch.randn(h_in, h_out))
        self.h_in, self.h_out, self.var_in, self.var_out = h_in, h_out, var_in, var_out
        self._act_name = None if act is None else activation_name(act)
        # path weight of the tensor product: 1 / sqrt(h_in); the variance factors of _fc.py:41-48 ride on top
        # (kept out of the module tree: the reference's layer has `weight` only in its state_dict)
        object.__setattr__(self, "_tp", TensorProduct(
            f"{h_in}x0e", "0e", f"{h_out}x0e", [(0, 0, 0, "uvw", True)], internal_weights=False, shared_weights=True
        ))  # fmt: skip
        self.act = None if act is None else Activation(f"{h_out}x0e", [self._act_name])
        # _fc.py:41-48: x @ W / sqrt(h_in var_in) before an activation, x @ W / sqrt(h_in var_in / var_out) without
        self._scale = (h_in * var_in) ** -0.5 if act is not None else (h_in * var_in / var_out) ** -0.5
        self._fwd = self._bwd = None
        self._bwd_act = {}

    def act_dense_plans(self, prev):
        """Plans of this layer fused with the activation of ``prev`` (the layer in front): ``act(z) @ W`` with its weight
        gradient, and ``g @ W^T`` times the derivative of the activation; None when a kernel involved is outside its
        limits."""
        name = prev._act_name
        if name not in self._bwd_act:
            pair = None
            if self.dense_plans()[0] and self._fwd.has_backward_w and prev.var_out == 1:
                var_ratio = self.var_in if self.act is not None else self.var_in / self.var_out
                fwd = _FusedPlan([self.h_in, self.h_out], "identity", False, var_ratio, 1, input_act=name)
                bwd = _FusedPlan([self.h_out, self.h_in], "identity", False, 1, 1, epilogue=name)
                if fwd.handle is not None and bwd.handle is not None:
                    fwd.prepare_backward_w()
                    pair = (fwd, bwd) if fwd.has_backward_w else None
            self._bwd_act[name] = pair
        return self._bwd_act[name]

    def __repr__(self) -> str:
        return f"Layer({self.h_in}->{self.h_out}, act={self._act_name})"

    def dense_plans(self):
        """One-layer plans of the fused kernel for ``x @ W`` and ``g @ W^T`` (built on first use); False outside its limits."""
        if self._fwd is None:
            var_ratio = self.var_in if self.act is not None else self.var_in / self.var_out
            fwd = _FusedPlan([self.h_in, self.h_out], "identity", False, var_ratio, 1)
            bwd = _FusedPlan([self.h_out, self.h_in], "identity", False, 1, 1)
            if fwd.handle is None or bwd.handle is None:
                self._fwd = self._bwd = False
            else:
                fwd.prepare_backward_w()
                self._fwd, self._bwd = fwd, bwd
        return self._fwd, self._bwd

    def forward(self, x: torch.Tensor):
        if x.is_cuda and x.dtype == torch.float32 and self.weight.dtype == torch.float32 and self.dense_plans()[0]:
            lead = x.shape[:-1]
            x2 = x.reshape(-1, self.h_in).contiguous()
            if x2.data_ptr() % 16:
                x2 = x2.clone()
            y = _DenseFn.apply(x2, self.weight, self).reshape(lead + (self.h_out,))
            if self.act is not None:
                y = self.act(y)
                if self.var_out != 1:
                    y = y * self.var_out**0.5
            return y
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


class _FusedPlan:
    """Handle of a fused-network plan of the library; ``None`` handle when the network is outside its limits."""

    def __init__(self, hs, act_name, out_act, variance_in, variance_out, epilogue=None, input_act=None) -> None:
        """``epilogue``: name of an activation; the outputs are then multiplied by ``cst * act'(z)`` of a tensor ``z``
        given to ``forward`` (the input gradient of a layer taken through the activation in front of it).
        ``input_act``: the rows given are pre-activations, the network starts from ``cst * act(x)``."""
        self.handle = None
        self.key = None
        self.reason = None
        self._args = (list(hs), act_name, out_act, variance_in, variance_out, epilogue, input_act)
        L = _lib.lib()
        arr = (ctypes.c_int32 * len(hs))(*hs)
        h = ctypes.c_void_p()
        rc = L.e3x_fc_plan_create_fused(
            arr, len(hs), _KINDS[act_name], second_moment_constant(act_name), int(bool(out_act)), float(variance_in),
            float(variance_out), 0, _KINDS[input_act or "identity"], second_moment_constant(input_act) if input_act else 1.0,
            _KINDS[epilogue or "identity"], second_moment_constant(epilogue) if epilogue else 1.0, ctypes.byref(h),
        )  # fmt: skip
        if rc == _lib.ERR_INVALID:
            self.reason = L.e3x_last_error().decode()  # outside the fused kernel's limits: layer by layer instead
            return
        _lib.check(rc)
        self.handle = h
        self.key = L.e3x_fc_plan_key(h).decode()
        self.workspace_bytes = L.e3x_fc_workspace_bytes(h)

    def __reduce__(self):  # copies and pickles rebuild the plan from its arguments
        return (_FusedPlan, self._args)

    def __del__(self):
        if getattr(self, "handle", None) is not None:
            try:
                _lib.lib().e3x_fc_plan_destroy(self.handle)
            except Exception:
                pass

    has_backward_w = False

    def prepare_backward_w(self):
        """Builds the weight-gradient kernel of a one-layer plan; ``has_backward_w`` stays False outside its limits."""
        rc = _lib.lib().e3x_fc_plan_prepare_backward_w(self.handle)
        if rc != _lib.ERR_INVALID:
            _lib.check(rc)
            self.has_backward_w = True

    def backward_w(self, x, g):
        hs = self._args[0]
        gw = torch.empty(hs[0], hs[1], device=x.device, dtype=torch.float32)
        with torch.cuda.device(x.device):
            _lib.check(
                _lib.lib().e3x_fc_backward_w(self.handle, _lib.ptr(x), _lib.ptr(g), _lib.ptr(gw), x.shape[0], _lib.stream_ptr(x.device))
            )
        return gw

    def forward(self, x, weights, z=None):
        L = _lib.lib()
        Z = x.shape[0]
        out = torch.empty((Z, weights[-1].shape[1]), device=x.device, dtype=torch.float32)
        ws = torch.empty(self.workspace_bytes, device=x.device, dtype=torch.uint8)
        ptrs = (ctypes.c_void_p * len(weights))(*[w.data_ptr() for w in weights])
        assert z is None or (z.shape == out.shape and z.is_contiguous() and z.dtype == torch.float32)
        with torch.cuda.device(x.device):
            _lib.check(
                L.e3x_fc_forward_epilogue(self.handle, _lib.ptr(x), ptrs, _lib.ptr(z) if z is not None else None, _lib.ptr(out),
                                          Z, _lib.ptr(ws), self.workspace_bytes, _lib.stream_ptr(x.device))
            )  # fmt: skip
        return out


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
        self._fused_args = (self.hs, activation_name(act), out_act, variance_in, variance_out)
        self._fused = None

    def __repr__(self) -> str:
        return f"{self.__class__.__name__}{self.hs}"

    def fused_plan(self):
        """The one-kernel plan of this network (built on first use); its ``handle`` is None outside the kernel's limits."""
        if self._fused is None:
            self._fused = _FusedPlan(*self._fused_args) if len(self.hs) >= 2 else False
        return self._fused

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        layers = list(self)
        wants_grad = torch.is_grad_enabled() and (x.requires_grad or any(l.weight.requires_grad for l in layers))
        if layers and not wants_grad and x.is_cuda and x.dtype == torch.float32 and x.shape[-1] == self.hs[0]:
            plan = self.fused_plan()
            if plan and plan.handle is not None:
                lead = x.shape[:-1]
                x2 = x.reshape(-1, self.hs[0]).contiguous()
                if x2.data_ptr() % 16:
                    x2 = x2.clone()
                ws = [l.weight.detach().contiguous() for l in layers]
                if all(w.is_cuda and w.dtype == torch.float32 for w in ws):
                    return plan.forward(x2, ws).reshape(lead + (self.hs[-1],))
        if wants_grad and len(layers) > 1 and x.is_cuda and x.dtype == torch.float32 and x.shape[-1] == self.hs[0]:
            out = self._forward_chained(x, layers)
            if out is not None:
                return out
        for layer in layers:
            x = layer(x)
        return x

    def _forward_chained(self, x, layers):
        """Layer by layer with every hidden activation attached to the dense layer behind it (``_ActDenseFn``); None
        when a layer is outside the limits of the kernels involved."""
        for prev, layer in zip(layers, layers[1:]):
            if prev.act is None or prev.weight.dtype != torch.float32 or layer.act_dense_plans(prev) is None:
                return None
        if not layers[0].dense_plans()[0] or layers[-1].weight.dtype != torch.float32:
            return None
        lead = x.shape[:-1]
        x2 = x.reshape(-1, self.hs[0]).contiguous()
        if x2.data_ptr() % 16:
            x2 = x2.clone()
        z = _DenseFn.apply(x2, layers[0].weight, layers[0])
        for prev, layer in zip(layers, layers[1:]):
            z = _ActDenseFn.apply(z, layer.weight, layer, prev)
        last = layers[-1]
        if last.act is not None:
            z = last.act(z)
            if last.var_out != 1:
                z = z * last.var_out**0.5
        return z.reshape(lead + (self.hs[-1],))
