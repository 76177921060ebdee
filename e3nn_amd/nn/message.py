"""Instruction lists of the per-edge-weight (``uvu``) message tensor product.

``message_instructions`` is the builder the reference's convolution uses at its call site
(e3nn/nn/models/v2106/points_convolution.py:60-76): one ``uvu`` path per
(node irrep, edge irrep, allowed output irrep), each path writing its own output block,
blocks sorted by irrep.  ``merged_instructions`` instead sums all paths with the same
output irrep into one block of a given ``irreps_out``.
"""
import itertools

from ..o3.irreps import Irrep, Irreps
from ..o3.tensor_product import TensorProduct


def message_instructions(irreps_node_input, irreps_edge_attr, keep):
    """Returns ``(irreps_mid, instructions)``; ``keep`` is an Irreps, a collection of irreps or a predicate on an irrep."""
    nodes, edges = Irreps(irreps_node_input), Irreps(irreps_edge_attr)
    if callable(keep):
        wanted = keep
    else:
        kept = {Irrep(ir) for ir in (Irreps(keep) if isinstance(keep, str) else keep)}
        wanted = kept.__contains__
    # one path per (node irrep, edge irrep, allowed product irrep), in that nesting; path n writes output block n
    paths = [(i, j, mul, ir) for (i, (mul, a)), (j, (_, b)) in itertools.product(enumerate(nodes), enumerate(edges)) for ir in a * b if wanted(ir)]
    blocks, position, _ = Irreps([(mul, ir) for _, _, mul, ir in paths]).sort()  # ... then the blocks are sorted by irrep
    return blocks, [(i, j, position[n], "uvu", True) for n, (i, j, _, _) in enumerate(paths)]


def merged_instructions(irreps_node_input, irreps_edge_attr, irreps_out):
    irreps_node_input, irreps_edge_attr, irreps_out = Irreps(irreps_node_input), Irreps(irreps_edge_attr), Irreps(irreps_out)
    return [
        (i, j, k, "uvu", True)
        for i, (_, a) in enumerate(irreps_node_input)
        for j, (_, b) in enumerate(irreps_edge_attr)
        for k, (_, c) in enumerate(irreps_out)
        if c in a * b
    ]


def message_tensor_product(irreps_node_input, irreps_edge_attr, keep=None, irreps_out=None) -> TensorProduct:
    """``uvu`` TensorProduct with per-edge external weights, as built inside the reference's convolution.

    Give ``keep`` for per-path sorted output blocks, or ``irreps_out`` for merged outputs.
    """
    if (keep is None) == (irreps_out is None):
        raise ValueError("give exactly one of keep and irreps_out")
    if keep is not None:
        irreps_out, ins = message_instructions(irreps_node_input, irreps_edge_attr, keep)
    else:
        ins = merged_instructions(irreps_node_input, irreps_edge_attr, irreps_out)
    return TensorProduct(irreps_node_input, irreps_edge_attr, irreps_out, ins, internal_weights=False, shared_weights=False)
