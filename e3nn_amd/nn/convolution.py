"""Equivariant point convolution of the reference's ``v2106`` model family
(``e3nn/nn/models/v2106/points_convolution.py:19-113``), every step on the HIP kernels of this package:

    self-connection, lin1, lin2, alpha   FullyConnectedTensorProduct(features, node_attr)   uvw kernels
    radial network                        FullyConnectedNet(edge_scalars)                     uvw + gate kernels
    message                               scatter(tp(x[src], edge_attr, w), dst)              fused uvu kernel

``node_features[edge_src]`` and the per-edge messages are never materialised.
"""
import torch
from torch.autograd.function import once_differentiable

from ..o3.irreps import Irrep, Irreps
from ..o3.tensor_product import FullyConnectedTensorProduct, TensorProduct
from .edges import DstSortedEdges
from .fc import FullyConnectedNet
from .message import message_instructions


class _Mix(torch.autograd.Function):
    """``sc + ((1 - m) + alpha * m * inv) * conv * inv`` (reference points_convolution.py:110-113 with the division by
    sqrt(num_neighbors) moved behind lin2 and alpha): two elementwise kernels forward and three backward, where autograd
    through the separate operations launches a dozen over the [N, channels] arrays."""

    @staticmethod
    def forward(ctx, sc, alpha, conv, m, inv):
        coeff = torch.addcmul((1 - m) * inv, alpha, m * (inv * inv))  # [N, channels]
        ctx.save_for_backward(coeff, conv, m)
        ctx.inv = inv
        return torch.addcmul(sc, coeff, conv)

    @staticmethod
    @once_differentiable
    def backward(ctx, g):
        coeff, conv, m = ctx.saved_tensors
        need_sc, need_alpha, need_conv = ctx.needs_input_grad[:3]
        g_alpha = ((g * conv) @ (m * (ctx.inv * ctx.inv))).unsqueeze(-1) if need_alpha else None
        return (g if need_sc else None), g_alpha, (g * coeff if need_conv else None), None, None


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
        node_conv_out = self.lin2(node_features, node_attr)
        alpha = self.alpha(node_features, node_attr)
        return _Mix.apply(node_self_connection, alpha, node_conv_out, self.sc.output_mask, inv)
