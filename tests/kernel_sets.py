"""The package's instruction-set list (e3nn_amd.kernel_sets) plus the cases of tests/golden: instruction tables and
constructor arguments written from the reference (tp_cases.json, nn_cases.json and their .npz arrays)."""
import json
import os

import torch

from e3nn_amd import kernel_sets as _ks
from e3nn_amd import nn, o3
from e3nn_amd.kernel_sets import *  # noqa: F401,F403
from e3nn_amd.kernel_sets import FUSED_FC_CASES, SH2, SH3  # noqa: F401

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")

GOLDEN_GPU_CASES = [
    "fctp_cfg1", "fctp_small_cfg5_like", "fctp_per_sample_weights", "fctp_norm_path",
    "uvu_merged_cfg3_like_mul4", "uvu_builder_cfg3_like_mul4", "uvu_builderA_cfg4_like_mul2",
    "uvu_builderB_cfg4_like_mul2", "uvu_shared_v2", "uvu_mixed_weightless", "empty_path_and_missing_output",
    "modes_uuu_uvuv_uuw_uvv", "modes_triangular", "conv_small",
]  # fmt: skip

# instruction sets whose backward pass the GPU tests run (transposed plans are separate kernels)
BACKWARD_CASES = _ks.BACKWARD_CASES + ["uvu_merged_cfg3_like_mul4", "uvu_builderA_cfg4_like_mul2", "uvu_shared_v2", "fctp_small_cfg5_like",
                                       "fctp_per_sample_weights", "modes_uuu_uvuv_uuw_uvv", "modes_triangular"]  # fmt: skip
BACKWARD_BF16_CASES = _ks.BACKWARD_BF16_CASES + ["uvu_shared_v2"]


def golden_meta():
    with open(os.path.join(GOLDEN, "tp_cases.json")) as f:
        return json.load(f)


def tp_from_meta(m, **extra):
    upw = m.get("user_path_weights", [1.0] * len(m["instructions"]))
    ins = [tuple(t[:5]) + (pw,) for t, pw in zip(m["instructions"], upw)]
    kw = {}
    if m.get("irrep_normalization"):
        kw = dict(irrep_normalization=m["irrep_normalization"], path_normalization=m["path_normalization"])
    return o3.TensorProduct(
        m["irreps_in1"], m["irreps_in2"], m["irreps_out"], ins,
        internal_weights=m["internal_weights"], shared_weights=m["shared_weights"], **kw, **extra,
    )  # fmt: skip


def golden_tp(name, meta=None, **extra):
    m = dict((meta or golden_meta())[name])
    if name == "fctp_norm_path":
        m.update(irrep_normalization="norm", path_normalization="path")
    return tp_from_meta(m, **extra)


def nn_golden():
    import numpy as np

    with open(os.path.join(GOLDEN, "nn_cases.json")) as f:
        meta = json.load(f)
    return np.load(os.path.join(GOLDEN, "nn_cases.npz")), meta


def golden_tensor_products():
    meta = golden_meta()
    return [(n, golden_tp(n, meta), (torch.float32,)) for n in GOLDEN_GPU_CASES]


def golden_modules():
    _, meta = nn_golden()
    out = []
    for name in ("linear_mixed", "linear_path_norm", "linear_bias"):
        m = meta[name]
        out.append((name, o3.Linear(m["irreps_in"], m["irreps_out"], **m["kwargs"])))
    out.append(("fc_golden", nn.FullyConnectedNet(meta["fc"]["hs"], torch.nn.functional.silu)))
    a = meta["conv"]["args"]
    out.append(("conv_golden", nn.Convolution(a[0], a[1], a[2], a[3], a[4], a[5])))
    return out


def prebuild(verbose=True):
    """Every kernel the tests and the benchmark use: the package's list plus the fixtures' instruction sets."""
    _ks.prebuild(verbose=verbose, extra_tensor_products=golden_tensor_products(), extra_modules=golden_modules(),
                 backward_cases=BACKWARD_CASES, backward_bf16_cases=BACKWARD_BF16_CASES)  # fmt: skip
