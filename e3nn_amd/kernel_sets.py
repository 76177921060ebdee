"""The benchmark's instruction sets and the ahead-of-time build of their kernels.

``cfg1`` ... ``cfg5`` are the five benchmark configurations; the other makers are the shapes each kernel family is
exercised on (tile edges, ragged channel counts, every connection mode).  ``prebuild`` compiles all of their kernels
into the in-tree cache, so that nothing has to be compiled on a GPU box; callers may hand it further products and
modules to build beside these (the test suite adds the instruction sets of its fixtures).
"""
import os

import torch

from . import o3
from .nn.message import message_tensor_product

SH2 = str(o3.Irreps.spherical_harmonics(2))
SH3 = str(o3.Irreps.spherical_harmonics(3))

# backward pass in bf16 storage as well (callers of prebuild may add names): a matrix-core uvw set, per-edge uvu weights
BACKWARD_BF16_CASES = ["mfma_small", "cfg3_merged", "wide_k_l3"]


def cfg1():
    return o3.FullyConnectedTensorProduct("16x0e+16x1o", "0e+1o+2e", "16x0e+16x1o+16x2e")


def cfg3(merged=True):
    f = "32x0e+32x1o+32x2e"
    return message_tensor_product(f, SH2, irreps_out=f) if merged else message_tensor_product(f, SH2, keep="0e+1o+2e")


def cfg4(variant="A"):
    f = "128x0e+128x1o+128x2e+128x3o"
    keep = "0e+1o+2e+3o" if variant == "A" else "0e+0o+1e+1o+2e+2o+3e+3o"
    return message_tensor_product(f, SH3, keep=keep)


def cfg5():
    f = "128x0e+128x1o+128x2e"
    return o3.FullyConnectedTensorProduct(f, f, f)


def mfma_small():
    # smallest shapes the matrix-core uvw kernel takes: multiplicities 32 / 64, three output irreps
    return o3.FullyConnectedTensorProduct("64x0e+32x1o", "32x0e+32x1o+32x2e", "64x0e+64x1o+64x1e+64x2e")


def mfma_full_tiles():
    # every multiplicity a multiple of 64: the uvw weight gradient takes its split-operand path (both contraction
    # orders: paths onto 0e with l > 0 inputs synthesise the A operand, the others the B operand)
    return o3.FullyConnectedTensorProduct("64x0e+64x1o", "64x0e+64x1o+64x2e", "64x0e+128x1o+64x1e+64x2e")


def mfma_half_tiles():
    # output multiplicities 32 and 96: the matrix-core kernels end an irrep with a tile of 32 channels (bf16 storage:
    # half of the 64-channel workgroup tile computes on copies and stores nothing)
    return o3.FullyConnectedTensorProduct("64x0e+32x1o", "32x0e+32x1o", "32x0e+96x1o+32x2e")


def mfma_l3_out():
    # an l = 3 output (seven accumulator tiles per wave) beside a vector output, 32 and 64 channels
    return o3.FullyConnectedTensorProduct("64x1o+64x2e", "64x1o+64x2e", "32x3o+64x1o")


def wide_k_l3():
    # 256 and 96 copies of l = 2, 3 against 32 vectors: the input gradients contract over 256 indices with an R operand
    # of 5 and 7 components, the largest LDS footprint of the bf16 matrix-core kernel
    return o3.FullyConnectedTensorProduct("256x2e+96x3o", "32x1o", "128x1o+64x3o")


def node_fctp():
    # node-wise step of a convolution: features x a few scalar node attributes (one-hot species), the GEMM K index is
    # the feature multiplicity and the attribute index is a short outer loop (reference
    # e3nn/nn/models/v2106/points_convolution.py:56-58)
    return o3.FullyConnectedTensorProduct("128x0e+64x1o+32x2e", "4x0e", "128x0e+64x1o+96x2e")


def node_many_species():
    # six species at 128 channels: 96 weight blocks per target, more than half of the LDS (one workgroup per CU)
    return o3.FullyConnectedTensorProduct("128x0e+64x1o", "6x0e", "64x0e+32x1o")


def node_block():
    # a node-wise layer of an interaction block at NequIP-like width: 32 channels out, 4 species (the weight-gradient
    # kernel puts two species side by side in the 64 columns of a tile)
    return o3.FullyConnectedTensorProduct("96x0e+128x1o+32x2e", "4x0e", "32x0e+32x1o+32x2e")


def node_wide_out():
    # scalar second input with several 32-channel output tiles per irrep, l = 3 and a pseudoscalar attribute: the
    # shape of an input gradient of a node-wise layer (few channels in, many out)
    return o3.FullyConnectedTensorProduct("32x0e+32x1o+32x3o", "3x0e+2x0o", "96x0e+64x1o+64x1e+32x3o+32x3e")


def node_narrow():
    # scalar second input, channel counts that are not multiples of 4 (weight rows read float by float, a partly
    # filled 32-channel tile) and multiplicities 8 / 24 / 40: the shape of the per-node mixing coefficient of a
    # convolution (reference e3nn/nn/models/v2106/points_convolution.py:92-97) with two more irreps
    return o3.FullyConnectedTensorProduct("96x0e+40x1o+8x2e", "4x0e", "1x0e+23x1o+9x2e")


def node_partial_tile():
    # channel counts that are multiples of 4 but not of 32: 16-byte weight pieces inside and outside the last tile
    return o3.FullyConnectedTensorProduct("64x0e+16x1o", "3x0e", "48x0e+20x1o")


def outer_split():
    # 32-channel output tiles with several outer indices and a second input that is not scalar: the matrix-core
    # kernel gives its second wave column every other outer index
    return o3.FullyConnectedTensorProduct("64x0e+32x1o", "4x0e+2x1o", "32x1o+32x1e+32x2e")


def wide_k():
    # GEMM K extents above 128 (256 and 160): the K operand is resident in LDS in blocks of 128, restaged per outer index
    return o3.FullyConnectedTensorProduct("256x0e+160x1o", "32x0e+32x1o", "64x0e+64x1o")


def wide_k_full_tiles():
    # as wide_k with every multiplicity a multiple of 64: the split-operand matrix steps on restaged K blocks
    return o3.FullyConnectedTensorProduct("256x0e+192x1o", "64x0e+64x1o", "64x0e+128x1o")


def unaligned_mfma():
    # matrix-core forward, but an irrep no output reaches (3x2e) makes the input row 175 floats long: the matrix-core
    # weight-gradient kernel needs 16-byte aligned operands within a row, so the gradient runs on the vector-ALU kernel
    return o3.FullyConnectedTensorProduct("64x0e+32x1o+3x2e", "0e", "64x0e+32x1o")


def unaligned_offsets():
    # a 5-float irrep in front of the tiled one: operand offset 5
    return o3.FullyConnectedTensorProduct("1x2e+32x0e", "0e", "32x0e")


def radial_layer():
    # one dense layer of a radial network written as a tensor product of scalars: 64 -> 352 (= 5.5 tiles of 64
    # channels: the last tile is half full), second input "0e"
    return o3.FullyConnectedTensorProduct("64x0e", "0e", "352x0e")


def mixed_modes(**extra):
    # uvu and uvw paths into the same output irrep plus an elementwise and an unweighted path: the general kernel
    ins = [(0, 0, 0, "uvu", True), (1, 1, 0, "uvw", True), (1, 0, 1, "uvu", False), (1, 1, 2, "uvv", True),
           (0, 0, 3, "uuu", True), (1, 2, 4, "uuw", False)]  # fmt: skip
    return o3.TensorProduct("4x0e+4x1o", "4x0e+3x1o+4x1e", "4x0e+4x1o+3x1e+4x0e+1x0o", ins, shared_weights=False, **extra)


def right_small():
    # a small fully connected product with right() compiled: the matrices [irreps_in1.dim, irreps_out.dim] per sample
    return o3.FullyConnectedTensorProduct("4x0e+4x1o", "0e+1o", "4x0e+4x1o+2x2e", compile_right=True)


def scalar_exact():
    # 1x1 Clebsch-Gordan, path weight 1: products and sums of small integers are exact in fp32
    return message_tensor_product("32x0e", "0e", irreps_out="32x0e")


def odd_mul():
    # multiplicities that are no multiple of the lane-group width, several chunks
    return message_tensor_product("80x0e+24x1o+5x2e", SH2, keep="0e+1o+2e")


def narrow_message():
    # 16 channels per irrep: fewer multiplicity indices per lane than the wider sets, so that a lane group stays busy
    f = "16x0e+16x1o+16x2e"
    return message_tensor_product(f, SH2, irreps_out=f)


def all_tensor_products():
    """(name, TensorProduct, dtypes) for everything that must be in the kernel cache."""
    out = [
        ("cfg1", cfg1(), (torch.float32,)),
        ("cfg3_merged", cfg3(True), (torch.float32, torch.bfloat16)),
        ("cfg3_builder", cfg3(False), (torch.float32,)),
        ("cfg4_A", cfg4("A"), (torch.float32, torch.bfloat16)),
        ("cfg4_B", cfg4("B"), (torch.float32, torch.bfloat16)),
        ("cfg5", cfg5(), (torch.float32, torch.bfloat16)),
        ("mfma_small", mfma_small(), (torch.float32,)),
        ("mfma_full_tiles", mfma_full_tiles(), (torch.float32,)),
        ("mfma_half_tiles", mfma_half_tiles(), (torch.float32, torch.bfloat16)),
        ("wide_k_l3", wide_k_l3(), (torch.float32, torch.bfloat16)),
        ("mfma_l3_out", mfma_l3_out(), (torch.float32,)),
        ("node_fctp", node_fctp(), (torch.float32, torch.bfloat16)),
        ("radial_layer", radial_layer(), (torch.float32,)),
        ("wide_k", wide_k(), (torch.float32,)),
        ("wide_k_full_tiles", wide_k_full_tiles(), (torch.float32,)),
        ("outer_split", outer_split(), (torch.float32,)),
        ("node_block", node_block(), (torch.float32,)),
        ("node_many_species", node_many_species(), (torch.float32, torch.bfloat16)),
        ("node_wide_out", node_wide_out(), (torch.float32, torch.bfloat16)),
        ("node_narrow", node_narrow(), (torch.float32, torch.bfloat16)),
        ("node_partial_tile", node_partial_tile(), (torch.float32, torch.bfloat16)),
        ("unaligned_mfma", unaligned_mfma(), (torch.float32,)),
        ("unaligned_offsets", unaligned_offsets(), (torch.float32,)),
        ("mixed_modes", mixed_modes(), (torch.float32,)),
        ("scalar_exact", scalar_exact(), (torch.float32,)),
        ("right_small", right_small(), (torch.float32,)),
        ("odd_mul", odd_mul(), (torch.float32,)),
        ("narrow_message", narrow_message(), (torch.float32, torch.bfloat16)),
    ]
    return out


# instruction sets whose backward pass the GPU tests run (transposed plans are separate kernels)
BACKWARD_CASES = ["cfg1", "cfg3_merged", "cfg3_builder", "cfg4_A", "cfg5", "mfma_small", "mfma_full_tiles", "outer_split", "node_fctp", "node_block",
                  "node_wide_out", "node_narrow", "node_partial_tile", "radial_layer", "odd_mul", "unaligned_mfma", "unaligned_offsets",
                  "mixed_modes", "scalar_exact", "narrow_message"]  # fmt: skip


def linear_channels(norm="element"):
    return o3.Linear("4x0e+3x1o+2x0e", "5x0e+2x1o", f_in=3, f_out=2, biases=True, path_normalization=norm)


def nn_modules():
    """(name, module) for the node-wise blocks the GPU tests run; every TensorProduct inside needs its kernels."""
    from e3nn_amd import nn

    out = [("linear_wide", o3.Linear("128x0e+128x1o+64x2e", "128x0e+64x1o+32x1o"))]
    for norm in ("element", "path"):  # input and output channels: the product on f_in / f_out copies of every irrep
        out.append((f"linear_channels_{norm}", linear_channels(norm)))
    out.append(("fc_radial", nn.FullyConnectedNet([8, 64, 352], torch.nn.functional.silu)))
    # a hidden layer too wide for the one-kernel path and its one-layer specialisations: tensor-product kernels throughout
    out.append(("fc_wide_hidden", nn.FullyConnectedNet([8, 512, 16], torch.nn.functional.silu)))
    out.append(("conv_wide", conv_wide()))
    return out


# (hs, act, out_act, variance_in, variance_out) of the networks the one-kernel path is tested on: the radial network of
# the benchmark block; three layers with a 96-wide output; widths that are multiples of nothing (scalar input loads,
# zero-padded hidden layer, a partial last column tile); one layer with an output activation and variances; no activation
FUSED_FC_CASES = [
    ([8, 64, 352], "silu", False, 1, 1),
    ([8, 64, 64, 96], "tanh", False, 1, 1),
    ([5, 100, 50], "silu", False, 1, 1),
    ([16, 40], "sigmoid", True, 2, 3),
    ([12, 32, 32], None, False, 1, 2),
    ([128, 128, 128, 8], "relu", True, 1, 1),
]


def fused_fc_nets():
    from e3nn_amd import nn

    torch.manual_seed(20240611)  # the weights are drawn at construction
    return [nn.FullyConnectedNet(hs, act, variance_in=vi, variance_out=vo, out_act=oa) for hs, act, oa, vi, vo in FUSED_FC_CASES]


def radial_message_cases():
    """(name, all-uvu TensorProduct, two-layer radial network) for the message kernel with the network inside."""
    from e3nn_amd import nn

    torch.manual_seed(20240612)  # the weights are drawn at construction
    tp = cfg3(merged=True)
    small = o3.TensorProduct("32x0e+32x1o", "0e+1o", "32x0e+32x1o+32x1e", [(0, 0, 0, "uvu", True), (0, 1, 1, "uvu", True), (1, 0, 1, "uvu", True),
                             (1, 1, 0, "uvu", True), (1, 1, 2, "uvu", True)], shared_weights=False, internal_weights=False)  # fmt: skip
    return [
        ("nequip_silu", tp, nn.FullyConnectedNet([8, 64, tp.weight_numel], torch.nn.functional.silu)),
        ("small_tanh", small, nn.FullyConnectedNet([5, 32, small.weight_numel], torch.tanh, variance_in=2, variance_out=3)),
        ("small_linear", small, nn.FullyConnectedNet([12, 16, small.weight_numel], None)),
    ]


def conv_wide():
    # one interaction block at NequIP-like width: 32 channels per irrep, 4 species, 8 radial basis functions
    from e3nn_amd import nn

    f = "32x0e+32x1o+32x2e"
    return nn.Convolution(f, "4x0e", SH2, f, [8, 64], 37.5)


# (set, normalize, normalization) of the message kernels that form the spherical harmonics of the edge vectors themselves
SH_MESSAGE_CASES = [("cfg3_merged", True, "component"), ("cfg3_merged", False, "integral"), ("cfg3_builder", True, "norm"),
                    ("cfg4_A", True, "component"), ("odd_mul", True, "integral"), ("narrow_message", True, "component")]  # fmt: skip


# node-wise blocks that the GPU tests also run in bf16 storage (forward and backward)
BF16_MODULES = ("fc_radial", "conv_wide", "linear_wide")


def prebuild(verbose=True, workers=6, extra_tensor_products=(), extra_modules=(), backward_cases=(), backward_bf16_cases=()):
    """Builds every kernel of this module's lists, plus ``extra_tensor_products`` (``(name, TensorProduct, dtypes)``;
    those named in ``backward_cases`` with their backward kernels) and ``extra_modules`` (``(name, module)``).  Plan creation spends its time in the HIP compiler (a child
    process, the calling thread waits with the GIL released), so a few threads build several kernels at once."""
    from concurrent.futures import ThreadPoolExecutor

    from e3nn_amd import nn

    from . import _lib

    jobs = []
    modules = nn_modules() + list(extra_modules)
    products = all_tensor_products() + list(extra_tensor_products)
    backward = set(BACKWARD_CASES) | set(backward_cases)
    for name, mod in modules + [(f"fused_fc{i}", net) for i, net in enumerate(fused_fc_nets())]:
        for sub in mod.modules():
            # Linear and the dense layers keep theirs out of the module tree, the convolution its alpha on the scalars
            for tp in (sub, sub.__dict__.get("_tp"), sub.__dict__.get("_alpha_head")):
                if isinstance(tp, o3.TensorProduct):
                    dtypes = (torch.float32, torch.bfloat16) if name in BF16_MODULES else (torch.float32,)
                    jobs.append((f"module {name}", tp, dtypes, True))
            if isinstance(sub, nn.FullyConnectedNet):
                jobs.append((f"module {name} (one kernel)", sub, None, False))
    for name, tp, dtypes in products:
        jobs.append((f"kernel {name}", tp, dtypes, name in backward))
    by_name = {name: tp for name, tp, _ in products}
    for name, normalize, normalization in SH_MESSAGE_CASES:
        jobs.append((f"harmonics {name}", by_name[name], (normalize, normalization), False))
    for name, tp, net in radial_message_cases():
        jobs.append((f"radial {name}", tp, net, False))
    for name, mod in modules:
        if isinstance(mod, nn.Convolution):  # the block runs its radial network inside the message kernel when it can
            jobs.append((f"radial {name}", mod.tp, mod.fc, False))

    def build(job):
        name, tp, dtypes, backward = job
        if name.startswith("harmonics "):
            from .o3.spherical_harmonics import _NORMALIZATION

            rc = _lib.lib().e3x_tp_plan_prepare_gather_scatter_sh(tp._plan(torch.float32).handle, int(dtypes[0]), _NORMALIZATION[dtypes[1]])
            _lib.check(rc)
            return name, [f"normalize={dtypes[0]} {dtypes[1]}"]
        if name.startswith("radial "):
            plan = dtypes.fused_plan()  # the network on its own, which the tests run beside the fused kernel
            return name, ["built" if tp.prepare_gather_scatter_radial(dtypes) else "(separate kernels)", plan.key or ""]
        if dtypes is None:
            plan = tp.fused_plan()
            keys = [plan.key or "(layer by layer: " + plan.reason + ")"]
            for layer in tp:
                fwd, bwd = layer.dense_plans()
                keys += [fwd.key, bwd.key] if fwd else ["(tensor-product kernels)"]
            layers = list(tp)
            for prev, layer in zip(layers, layers[1:]):  # input gradient through the activation in one kernel
                pair = layer.act_dense_plans(prev) if prev.act is not None else None
                keys += [pair[0].key, pair[1].key] if pair is not None else []
            return name, keys
        keys = [tp._plan(dt).key for dt in dtypes]
        if backward:
            tp.compile_backward(torch.float32)
        if name.replace("kernel ", "") in set(BACKWARD_BF16_CASES) | set(backward_bf16_cases) or (backward and torch.bfloat16 in dtypes):
            tp.compile_backward(torch.bfloat16)
        return name, keys

    with ThreadPoolExecutor(max_workers=workers) as pool:
        for name, keys in pool.map(build, jobs):
            if verbose:
                print(f"{name:40s} {' '.join(keys)}", flush=True)
    # the benchmark times config 5 on the fp32 matrix instruction beside the split-operand default; the generator reads
    # its switches from the environment at plan creation, so these two are built here, after the threads are done
    saved = {k: os.environ.get(k) for k in ("E3X_UVW_SPLIT", "E3X_DW_SPLIT")}
    os.environ.update({k: "0" for k in saved})
    try:
        plan = cfg5()._plan(torch.float32)
        _lib.check(_lib.lib().e3x_tp_plan_prepare_backward_w(plan.handle))
        if verbose:
            print(f"{'kernel cfg5 (fp32 matrix instruction)':40s} {plan.key} / {plan.arithmetic} / {plan.arithmetic_weight_gradient}", flush=True)
    finally:
        for k, v in saved.items():
            os.environ.pop(k) if v is None else os.environ.__setitem__(k, v)
