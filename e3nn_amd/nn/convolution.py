"""Equivariant point convolution of the reference's ``v2106`` model family
(``e3nn/nn/models/v2106/points_convolution.py:19-113``), every step on the HIP kernels of this package:

    self-connection, lin1, lin2, alpha   FullyConnectedTensorProduct(features, node_attr)   uvw kernels
    radial network                        FullyConnectedNet(edge_scalars)                     uvw + gate kernels
    message                               scatter(tp(x[src], edge_attr, w), dst)              fused uvu kernel

``node_features[edge_src]`` and the per-edge messages are never materialised.
"""
import torch

from ..o3.irreps import Irrep, Irreps
from ..o3.tensor_product import _OUT, FullyConnectedTensorProduct, TensorProduct, _permuted_weights, _slot_backward, _TpSlot
from .edges import DstSortedEdges
from .fc import FullyConnectedNet
from .message import message_instructions


class _Mix(torch.autograd.Function):
    """``sc + (c0 + alpha * c1) * conv`` with ``c0 = (1 - m) / sqrt(n)``, ``c1 = m / n`` (reference
    points_convolution.py:110-113 with the division by sqrt(num_neighbors) moved behind lin2 and alpha): two elementwise
    kernels forward and three backward, where autograd through the separate operations launches a dozen over the
    [N, channels] arrays.  The backward pass is written in differentiable elementwise operations, so it can itself be
    differentiated (``create_graph``)."""

    @staticmethod
    def forward(ctx, sc, alpha, conv, c0, c1):
        coeff = torch.addcmul(c0, alpha, c1)  # [N, channels]
        ctx.save_for_backward(coeff, conv, c1, alpha, c0)
        return torch.addcmul(sc, coeff, conv)

    @staticmethod
    def backward(ctx, g):
        coeff, conv, c1, alpha, c0 = ctx.saved_tensors
        if torch.is_grad_enabled():
            coeff = torch.addcmul(c0, alpha, c1)  # as a function of alpha
        need_sc, need_alpha, need_conv = ctx.needs_input_grad[:3]
        g_alpha = (g * conv * c1).sum(-1, keepdim=True) if need_alpha else None
        return (g if need_sc else None), g_alpha, (g * coeff if need_conv else None), None, None


class _Lin2Alpha(torch.autograd.Function):
    """``lin2(features, attr)`` and ``alpha(features, attr)`` as one node of the autograd graph.  ``alpha`` reads only
    the leading scalars of the features (``head`` is ``alpha`` restricted to them, same weights), so its input gradient
    is added into the leading columns of lin2's instead of being written as a second zero-padded [N, features] array
    that autograd then adds to the first: three passes over an array as wide as the messages saved."""

    @staticmethod
    def forward(ctx, features, attr, w_lin2, w_alpha, lin2, head):
        ctx.lin2, ctx.head = lin2, head
        scalars = features[:, : head.irreps_in1.dim].contiguous()
        ctx.save_for_backward(features, attr, w_lin2, w_alpha, scalars)
        dt = features.dtype
        return lin2._plan(dt).forward(features, attr, w_lin2), head._plan(dt).forward(scalars, attr, w_alpha)

    @staticmethod
    def backward(ctx, g_conv, g_alpha):
        lin2, head = ctx.lin2, ctx.head
        features, attr, w_lin2, w_alpha, scalars = ctx.saved_tensors
        g_conv, g_alpha = g_conv.contiguous(), g_alpha.contiguous()
        if torch.is_grad_enabled():
            # under create_graph: the two products' own differentiable gradients
            need = ctx.needs_input_grad
            k = head.irreps_in1.dim
            gf, _, gw_lin2 = _slot_backward(_TpSlot, _OUT, (features, attr, w_lin2), g_conv, (need[0], False, need[2]), lin2)
            gs, _, gw_alpha = _slot_backward(_TpSlot, _OUT, (features[:, :k].contiguous(), attr, w_alpha), g_alpha, (need[0], False, need[3]), head)
            if need[0]:
                gf = gf + torch.nn.functional.pad(gs, (0, features.shape[1] - k))
            return gf, None, gw_lin2, gw_alpha, None, None
        dt = features.dtype
        g_features = gw_lin2 = gw_alpha = None
        if ctx.needs_input_grad[2]:
            gw_lin2 = lin2._plan(dt).backward_w_uvw(features, attr, g_conv, True)
        if ctx.needs_input_grad[3]:
            gw_alpha = head._plan(dt).backward_w_uvw(scalars, attr, g_alpha, True)
        if ctx.needs_input_grad[0]:
            g_features = lin2._grad_plan("x1", dt).forward(g_conv, attr, _permuted_weights(lin2, w_lin2, (2, 1, 0)))
            g_scalars = head._grad_plan("x1", dt).forward(g_alpha, attr, _permuted_weights(head, w_alpha, (2, 1, 0)))
            g_features[:, : scalars.shape[1]] += g_scalars
        return g_features, None, gw_lin2, gw_alpha, None, None


class Convolution(torch.nn.Module):
    r"""Same constructor and ``forward`` arguments as the reference; ``forward`` also accepts a prebuilt
    ``edges=DstSortedEdges(...)`` so that the destination sort is paid once per graph instead of once per layer."""

    def __init__(
        self, irreps_node_input, irreps_node_attr, irreps_edge_attr, irreps_node_output, fc_neurons, num_neighbors
    ) -> None:
        super().__init__()
        self.irreps_node_input, self.irreps_node_attr = Irreps(irreps_node_input), Irreps(irreps_node_attr)
        self.irreps_edge_attr, self.irreps_node_output = Irreps(irreps_edge_attr), Irreps(irreps_node_output)
        self.num_neighbors = num_neighbors

        def node_wise(features, out):  # features (x) node attributes -> out, shared weights
            return FullyConnectedTensorProduct(features, self.irreps_node_attr, out)

        # messages carry every irrep the output asks for, plus scalars for the per-node mixing coefficient `alpha`
        wanted = {ir for _, ir in self.irreps_node_output} | {Irrep(0, 1)}
        irreps_mid, instructions = message_instructions(self.irreps_node_input, self.irreps_edge_attr, wanted)
        if irreps_mid.dim == 0:
            raise AssertionError(
                f"no product of an input irrep ({self.irreps_node_input}) with an edge irrep ({self.irreps_edge_attr}) "
                f"lies in the output irreps ({self.irreps_node_output}): there is no message to send"
            )
        # submodules in the reference's registration order (state_dict keys and the random stream of the initial weights)
        self.sc = node_wise(self.irreps_node_input, self.irreps_node_output)
        self.lin1 = node_wise(self.irreps_node_input, self.irreps_node_input)
        message = TensorProduct(
            self.irreps_node_input, self.irreps_edge_attr, irreps_mid, instructions, internal_weights=False, shared_weights=False
        )
        self.fc = FullyConnectedNet([*fc_neurons, message.weight_numel], torch.nn.functional.silu)
        self.tp = message
        self.lin2 = node_wise(irreps_mid, self.irreps_node_output)
        self.alpha = node_wise(irreps_mid, "0e")
        torch.nn.init.zeros_(self.alpha.weight)  # the block starts as its self-connection
        if self.alpha.output_mask[0] != 1.0:
            raise AssertionError(f"the messages ({irreps_mid}) and the node attributes ({self.irreps_node_attr}) cannot produce a scalar for alpha")
        # alpha restricted to the leading irreps of the messages when those are all it reads (scalar node attributes and
        # sorted messages: always): same instructions, weights and normalisation; kept out of the module tree, it has
        # no parameters and must not add keys to the state_dict
        self.__dict__["_alpha_head"] = None
        n_head = 1 + max(ins.i_in1 for ins in self.alpha.instructions)
        if irreps_mid[:n_head].dim % 4 == 0 and n_head < len(irreps_mid):
            head = FullyConnectedTensorProduct(irreps_mid[:n_head], self.irreps_node_attr, "0e", internal_weights=False, shared_weights=True)
            key = lambda tp: [(i.i_in1, i.i_in2, i.i_out, i.path_shape, i.path_weight) for i in tp.instructions]  # noqa: E731
            if key(head) == key(self.alpha) and head.weight_numel == self.alpha.weight_numel:
                self.__dict__["_alpha_head"] = head

    def forward(self, node_input, node_attr, edge_src, edge_dst, edge_attr, edge_scalars, edges=None) -> torch.Tensor:
        node_self_connection = self.sc(node_input, node_attr)
        node_features = self.lin1(node_input, node_attr)
        if edges is None:
            edges = DstSortedEdges(edge_src, edge_dst, node_input.shape[0])
        messages = None
        wants_grad = torch.is_grad_enabled() and (
            any(t.requires_grad for t in (node_features, edge_attr, edge_scalars)) or any(p.requires_grad for p in self.fc.parameters())
        )
        if not wants_grad:
            # the radial network inside the message kernel: the [E, weight_numel] weights are never stored
            messages = self.tp.forward_gather_scatter_radial(node_features, edge_attr, edge_scalars, self.fc, edges)
        if messages is None:
            weight = self.fc(edge_scalars)
            messages = self.tp.forward_gather_scatter(node_features, edge_attr, weight, edges=edges)
        node_features = messages
        # lin2 and alpha are linear in the features, so the division by sqrt(num_neighbors) that the reference applies
        # to the summed messages (points_convolution.py:108) is applied to their outputs instead, which are four to a
        # thousand times narrower than the messages
        inv = 1.0 / self.num_neighbors**0.5
        if (
            self._alpha_head is not None
            and torch.is_grad_enabled()
            and node_features.requires_grad
            and not node_attr.requires_grad
            and node_features.dim() == 2
            and node_attr.shape[:-1] == node_features.shape[:-1]
            and node_features.dtype == torch.float32
        ):
            node_conv_out, alpha = _Lin2Alpha.apply(
                node_features.contiguous(), node_attr.to(node_features.dtype).contiguous(), self.lin2.weight, self.alpha.weight,
                self.lin2, self._alpha_head,
            )  # fmt: skip
        else:
            node_conv_out = self.lin2(node_features, node_attr)
            alpha = self.alpha(node_features, node_attr)
        m = self.sc.output_mask
        key = (m.device, m.dtype, m._version, inv)
        if self.__dict__.get("_mix_key") != key:  # the two constant rows of the mixing, once per device
            self.__dict__["_mix_key"], self.__dict__["_mix_rows"] = key, ((1 - m) * inv, m * (inv * inv))
        c0, c1 = self.__dict__["_mix_rows"]
        return _Mix.apply(node_self_connection, alpha, node_conv_out, c0, c1)
