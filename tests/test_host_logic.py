"""CPU-only tests: the C-ABI library loads and exports what include/e3x.h declares, host-side
functions (Wigner 3j, plan creation) and the Python mirror of the reference API."""
import copy
import ctypes
import io
import os
import pickle
import re

import numpy as np
import pytest
import torch

from e3nn_amd import _lib, get_optimization_defaults, o3, set_optimization_defaults
from e3nn_amd.nn.message import message_instructions, message_tensor_product
from oracle import tensor_product as otp
from oracle.wigner import wigner_3j as oracle_w3j
from tests import kernel_sets as ks

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "e3x.h")).read()
    declared = set(re.findall(r"\b(e3x_[a-z0-9_]+)\s*\(", header))
    assert len(declared) >= 12
    handle = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared:
        assert hasattr(handle, name), f"{name} declared in e3x.h but not exported"
    assert declared == set(_lib._SIGNATURES), "ctypes signatures out of sync with e3x.h"
    # ... and nothing else: internal C++ symbols stay inside the library
    import subprocess

    syms = subprocess.run(["nm", "-D", "--defined-only", _lib.LIB_PATH], capture_output=True, text=True, check=True).stdout
    exported = {line.split()[-1] for line in syms.splitlines() if line.strip()}
    assert exported == declared, sorted(exported ^ declared)
    assert _lib.lib().e3x_version() >= 100


def test_wigner_3j_matches_oracle_and_golden(golden_w3j):
    for key, ref in golden_w3j.items():
        l1, l2, l3 = map(int, key.split("_"))
        got = o3.wigner_3j(l1, l2, l3, dtype=torch.float64).numpy()
        np.testing.assert_allclose(got, ref, atol=1e-13)
    for l1, l2, l3 in ((6, 5, 3), (8, 8, 8), (10, 9, 4), (12, 1, 11)):
        np.testing.assert_allclose(o3.wigner_3j(l1, l2, l3, dtype=torch.float64).numpy(), oracle_w3j(l1, l2, l3), atol=1e-13)
    assert o3.wigner_3j(1, 1, 1).dtype == torch.get_default_dtype()
    with pytest.raises(AssertionError):
        o3.wigner_3j(1, 1, 3)
    buf = (ctypes.c_double * 27)()
    assert _lib.lib().e3x_wigner_3j(1, 1, 3, buf) != 0
    assert b"l1" in _lib.lib().e3x_last_error()


def test_irreps_api():
    assert repr(o3.Irrep("1y")) == "1o" and o3.Irrep("2o").dim == 5
    assert o3.Irrep("2e") in list(o3.Irrep("1o") * o3.Irrep("1o"))
    assert repr(o3.Irrep("1o") + o3.Irrep("2o")) == "1x1o+1x2o"
    it = o3.Irrep.iterator()
    assert [repr(next(it)) for _ in range(4)] == ["0e", "0o", "1o", "1e"]
    irreps = o3.Irreps("2x0e + 1e")
    assert irreps.slices() == [slice(0, 2), slice(2, 5)] and irreps.dim == 5 and irreps.num_irreps == 3
    assert repr(o3.Irreps.spherical_harmonics(3)) == "1x0e+1x1o+1x2e+1x3o"
    assert repr(o3.Irreps.spherical_harmonics(4, p=1)) == "1x0e+1x1e+1x2e+1x3e+1x4e"
    assert repr(o3.Irreps("1e + 1e + 0e").simplify()) == "2x1e+1x0e"
    assert repr(o3.Irreps("1e + 1e + 0e + 1e").simplify()) == "2x1e+1x0e+1x1e"
    assert repr(o3.Irreps("4x0e + 0x1o + 2x3e").remove_zero_multiplicities()) == "4x0e+2x3e"
    assert repr(o3.Irreps("1e + 0e + 1e + 0x2e").regroup()) == "1x0e+2x1e"
    assert repr(o3.Irreps("1e + 2e + 0e").filter(keep=["0e", "1e"])) == "1x1e+1x0e"
    assert repr(o3.Irreps("1e + 2e + 0e").filter(drop="2e + 2x1e")) == "1x0e"
    assert repr(o3.Irreps("1e + 2e + 0e").filter(lmax=1)) == "1x1e+1x0e"
    assert repr(2 * o3.Irreps("0e + 1e")) == "1x0e+1x1e+1x0e+1x1e" and repr(3 * o3.Irrep("1e")) == "3x1e"
    assert o3.Irreps("5x0e + 10x1o").randn(5, -1, 5, normalization="norm").shape == (5, 35, 5)
    assert o3.Irreps("3x1o + 2x1o").count("1o") == 5 and "2e" not in o3.Irreps("1o")
    for bad in ("1x", "-1e", "2x1z"):
        with pytest.raises(ValueError):
            o3.Irreps(bad)
    with pytest.raises(NotImplementedError):
        o3.Irreps("1o") * o3.Irreps("1o")


def test_sort_matches_reference_golden(golden_tp):
    for s, ref in golden_tp[0]["sort"].items():
        r = o3.Irreps(s).sort()
        assert str(r.irreps) == ref["irreps"] and list(r.p) == ref["p"] and list(r.inv) == ref["inv"]


def test_constructor_tables_match_reference_golden(golden_tp):
    meta = golden_tp[0]
    n = 0
    for name, m in meta.items():
        if "instructions" not in m or any(t[3] not in ("uvu", "uvw") for t in m["instructions"]):
            continue
        tp = ks.golden_tp(name, meta)
        assert tp.weight_numel == m["weight_numel"] and tp.shared_weights == m["shared_weights"]
        assert tp.internal_weights == m["internal_weights"]
        for t, ref in zip(tp.instructions, m["instructions"]):
            assert abs(t.path_weight - ref[5]) <= 1e-15 * max(1.0, abs(ref[5])) and list(t.path_shape) == ref[6]
        for sl, flag in zip(tp.irreps_out.slices(), m["output_mask_blocks"]):
            if flag >= 0:
                assert (tp.output_mask[sl] == flag).all()
        n += 1
    assert n >= 15


def test_builders_match_reference_golden(golden_tp):
    meta = golden_tp[0]
    for name, tp in (("fctp_cfg1", ks.cfg1()), ("fctp_cfg5_structure", ks.cfg5()), ("uvu_merged_cfg3_structure", ks.cfg3(True)),
                     ("uvu_builder_cfg3_structure", ks.cfg3(False)), ("uvu_builderA_cfg4_structure", ks.cfg4("A")),
                     ("uvu_builderB_cfg4_structure", ks.cfg4("B"))):  # fmt: skip
        m = meta[name]
        assert str(tp.irreps_out) == m["irreps_out"], name
        assert [[t.i_in1, t.i_in2, t.i_out, t.connection_mode] for t in tp.instructions] == [t[:4] for t in m["instructions"]]
        assert tp.weight_numel == m["weight_numel"]
        for t, ref in zip(tp.instructions, m["instructions"]):
            assert abs(t.path_weight - ref[5]) < 1e-15
    mid, ins = message_instructions("4x0e+4x1o", "0e+1o", "0e+1o")
    omid, oins = otp.convolution_instructions("4x0e+4x1o", "0e+1o", lambda l, p: (l, p) in {(0, 1), (1, -1)})
    assert [tuple(t) for t in ins] == [tuple(t) for t in oins] and str(mid) == "4x0e+4x0e+4x1o+4x1o"


def test_module_state_and_api_details():
    tp = ks.cfg1()
    # weight, mask and the Wigner buffers of the reference's generated module (see the state_dict test below)
    assert set(tp.state_dict()) == {"weight", "output_mask", "_compiled_main_left_right._w3j_1_1_2", "_compiled_main_left_right._w3j_1_2_1"}
    assert repr(tp).startswith("FullyConnectedTensorProduct(16x0e+16x1o x 1x0e+1x1o+1x2e -> 16x0e+16x1o+16x2e | 1792 paths | 1792 weights")
    views = list(tp.weight_views())
    assert [tuple(v.shape) for v in views] == [(16, 1, 16)] * 7
    assert tp.weight_view_for_instruction(2).shape == (16, 1, 16)
    assert tp.weight_view_for_instruction(2).data_ptr() == views[2].data_ptr()
    tp2 = copy.deepcopy(tp)
    assert torch.equal(tp2.weight, tp.weight) and tp2.instructions == tp.instructions
    ext = ks.cfg3(True)
    assert ext.weight.numel() == 0 and not ext.internal_weights and not ext.shared_weights
    with pytest.raises(RuntimeError):
        ext._get_weights(None)
    with pytest.raises(AssertionError):
        o3.TensorProduct("1o", "1o", "1o", [(0, 0, 0, "uvu", True)])  # parity violates the selection rule
    with pytest.raises(AssertionError):
        o3.TensorProduct("1o", "1o", "3e", [(0, 0, 0, "uvu", True)])
    with pytest.raises(AssertionError):
        o3.TensorProduct("1o", "1o", "1e", [(0, 0, 0, "uvu", True)], internal_weights=True, shared_weights=False)
    # every connection mode of the reference builds a plan (the general vector-ALU kernel family)
    tp = o3.TensorProduct("2x1o", "2x1o", "2x1e", [(0, 0, 0, "uuu", True)])
    assert tp.weight_numel == 2 and tp._plan(torch.float32).family == "uvw_small"
    assert o3.TensorProduct("2x1o", "2x1o", "2x1e", [(0, 0, 0, "uuu", True)], compile_right=True)._compile_right
    set_optimization_defaults(specialized_code=False)
    assert get_optimization_defaults()["specialized_code"] is False
    set_optimization_defaults(specialized_code=True)
    with pytest.raises(ValueError):
        set_optimization_defaults(nonsense=1)


def test_plan_creation_needs_no_gpu_and_reports_family():
    tp = message_tensor_product("4x0e+4x1o+4x2e", ks.SH2, keep="0e+1o+2e")
    plan = tp.compile()._plans[torch.float32]
    assert plan.family == "uvu" and plan.key.startswith("uvu_")
    assert ks.cfg1().compile()._plans[torch.float32].family == "uvw_small"
    L = _lib.lib()
    bad = _lib.TpDesc(1, 1, 1, 1, (_lib.Irrep * 1)(_lib.Irrep(2, 1, -1)), (_lib.Irrep * 1)(_lib.Irrep(1, 1, -1)),
                      (_lib.Irrep * 1)(_lib.Irrep(2, 1, -1)), (_lib.Instruction * 1)(_lib.Instruction(0, 0, 0, 1, 1, 1.0)), 0, 0)  # fmt: skip
    h = _lib.c_void_p()
    assert L.e3x_tp_plan_create(ctypes.byref(bad), ctypes.byref(h)) == -1  # 1o x 1o -> 1o violates parity
    assert b"selection" in L.e3x_last_error()
    assert L.e3x_csr_workspace_bytes(1000, 10) > 3 * 4000


@pytest.mark.parametrize("name", ["mixed_modes", "modes_uuu_uvuv_uuw_uvv", "modes_triangular"])
def test_dense_uvw_equivalent_of_general_modes(name):
    """Gradients of connection modes outside pure uvu / pure uvw go through a pure-uvw product with structured weights:
    on the oracle, that product with the expanded weights is the same map as the original instruction set."""
    from oracle import tensor_product as otp
    from tests import kernel_sets as ks
    from tests.helpers import oracle_spec, seeded

    tp = ks.mixed_modes() if name == "mixed_modes" else ks.golden_tp(name)
    dense_tp, expand = tp._dense_equivalent()
    assert all(t.connection_mode == "uvw" for t in dense_tp.instructions)
    Z = 6
    wshape = (tp.weight_numel,) if tp.shared_weights else (Z, tp.weight_numel)
    x1, x2, w = seeded(Z, tp.irreps_in1.dim, seed=1), seeded(Z, tp.irreps_in2.dim, seed=2), seeded(*wshape, seed=3)
    want = otp.tp_forward(oracle_spec(tp), x1.numpy(), x2.numpy(), w.numpy() if tp.weight_numel else None)
    wd = expand(w, x1)
    assert wd.shape[-1] == dense_tp.weight_numel
    got = otp.tp_forward(oracle_spec(dense_tp, irrep_normalization="none", path_normalization="none",
                                     user_path_weights=[t.path_weight**2 for t in tp.instructions]), x1.numpy(), x2.numpy(), wd.numpy())
    np.testing.assert_allclose(got, want, rtol=1e-10, atol=1e-12)


def test_fully_connected_plans_need_no_gpu_and_reject_what_the_kernel_cannot_hold():
    """Plans of the fused network kernel are built (or found in the cache) without a GPU; widths beyond the register
    and LDS budgets, unknown activations and empty layer lists are E3X_ERR_INVALID, which the module answers by
    running layer by layer."""
    import ctypes

    from e3nn_amd import nn
    from e3nn_amd.nn.fc import _FusedPlan

    L = _lib.lib()
    plan = _FusedPlan([8, 64, 352], "silu", False, 1, 1)
    assert plan.handle is not None and plan.key.startswith("fc_mfma_")
    # packed weights, widths already multiples of 8 / 32: layer 0 in fp32, the 64 -> 352 layer as three bf16 planes
    assert plan.workspace_bytes == 8 * 64 * 4 + 64 * 352 * 6
    # zero padded; the last layer (128 -> 64, a wide input onto at most 64 outputs) as three bf16 planes
    assert _FusedPlan([5, 100, 50], "tanh", False, 1, 1).workspace_bytes == 8 * 128 * 4 + 128 * 64 * 6
    for hs in ([8, 512, 16], [128, 256, 8], [600, 8]):
        bad = _FusedPlan(hs, "silu", False, 1, 1)
        assert bad.handle is None and "e3x_fc_plan_create" in bad.reason
    h = ctypes.c_void_p()
    arr = (ctypes.c_int32 * 2)(4, 4)
    assert L.e3x_fc_plan_create(arr, 2, 99, 1.0, 0, 1.0, 1.0, 0, ctypes.byref(h)) == _lib.ERR_INVALID  # activation
    assert L.e3x_fc_plan_create(arr, 1, 1, 1.0, 0, 1.0, 1.0, 0, ctypes.byref(h)) == _lib.ERR_INVALID  # no layer
    assert L.e3x_fc_plan_create(arr, 2, 1, 1.0, 0, -1.0, 1.0, 0, ctypes.byref(h)) == _lib.ERR_INVALID  # variance
    assert L.e3x_fc_plan_create(arr, 2, 1, 1.0, 0, 1.0, 1.0, 1, ctypes.byref(h)) == _lib.ERR_INVALID  # bf16 storage
    # the weight gradient exists for one-layer plans only
    assert L.e3x_fc_plan_prepare_backward_w(plan.handle) == _lib.ERR_INVALID
    one = _FusedPlan([64, 352], "identity", False, 1, 1)
    one.prepare_backward_w()
    assert one.has_backward_w
    net = nn.FullyConnectedNet([8, 512, 16], torch.nn.functional.silu)
    assert net.fused_plan().handle is None and not net.layer0.dense_plans()[0]
    assert [tuple(p.shape) for p in net.parameters()] == [(8, 512), (512, 16)]  # the reference's parameters
    assert list(dict(net.named_parameters())) == ["layer0.weight", "layer1.weight"]


def test_row_order_entry_point_validates_its_arguments():
    import ctypes

    L = _lib.lib()
    assert L.e3x_row_order_workspace_bytes(-1) == 0
    small, large = L.e3x_row_order_workspace_bytes(10), L.e3x_row_order_workspace_bytes(1_000_000)
    assert 0 < small < large and large >= 4 * 4 * 1_000_000
    pairs = ctypes.c_int32(7)
    null = ctypes.c_void_p(0)
    assert L.e3x_row_order_build(null, 16, null, null, 0, 4, 4, null, ctypes.byref(pairs), null, 0, null) == _lib.ERR_INVALID
    assert L.e3x_row_order_build(null, 32, null, null, 0, 0, 0, null, ctypes.byref(pairs), null, 0, null) == 0 and pairs.value == 0
    assert L.e3x_row_order_build(null, 32, null, null, 0, 4, 4, null, None, null, 0, null) == _lib.ERR_INVALID  # null pointers


def test_state_dict_keys_match_the_reference():
    """Names and shapes of every state_dict entry as the reference has them (fixture written from the reference's
    modules): weights, output masks, the Wigner / index buffers of its generated modules, the `mul` submodule of the
    gate -- so that checkpoints load with strict=True in both directions."""
    import json

    from e3nn_amd import nn

    with open(os.path.join(ROOT, "tests", "golden", "state_dict_keys.json")) as f:
        ref = json.load(f)
    silu, sigmoid, tanh = torch.nn.functional.silu, torch.sigmoid, torch.tanh
    modules = {
        "module_linear": lambda: o3.Linear("2x0e+2x1o", "3x0e+1x1o", biases=True),
        "module_linear_l2": lambda: o3.Linear("2x0e+2x1o+2x2e", "3x0e+1x1o+2x2e"),
        "module_fc": lambda: nn.FullyConnectedNet([4, 8, 2], silu),
        "module_gate": lambda: nn.Gate("4x0e+2x0o", [silu, tanh], "3x0e", [sigmoid], "2x1o+1x2e"),
        "module_activation": lambda: nn.Activation("4x0e+2x0o", [silu, tanh]),
        "module_convolution_l1": lambda: nn.Convolution("4x0e+4x1o", "2x0e", "0e+1o", "4x0e+4x1o", [3, 8], 3.0),
        "module_convolution_l2": lambda: nn.Convolution("4x0e+4x1o+4x2e", "2x0e", "0e+1o+2e", "4x0e+4x1o+4x2e", [3, 8], 3.0),
    }
    assert set(modules) == {k for k in ref if k.startswith("module_")}
    for name, entry in ref.items():
        if name in modules:
            m = modules[name]()
        else:
            i1, i2, io, ins, kw = entry["args"]
            m = o3.FullyConnectedTensorProduct(i1, i2, io, **kw) if ins is None else o3.TensorProduct(i1, i2, io, [tuple(t) for t in ins], **kw)
        mine = {k: list(v.shape) for k, v in m.state_dict().items()}
        assert mine == entry["state_dict"], name
        # a state_dict with the reference's keys loads strictly, and the constants are the Wigner tensors
        fake = {k: torch.zeros(shape, dtype=m.state_dict()[k].dtype) for k, shape in entry["state_dict"].items()}
        m.load_state_dict(fake, strict=True)
    tp = o3.FullyConnectedTensorProduct("2x0e+2x1o+2x2e", "0e+1o+2e", "2x0e+2x1o+2x2e")
    assert torch.equal(tp._compiled_main_left_right._w3j_1_2_1, o3.wigner_3j(1, 2, 1))
    with pytest.raises(NotImplementedError):  # the reference's right() has no triangular modes
        o3.TensorProduct("4x1o", "4x1o", "6x1e", [(0, 0, 0, "uvu<v", True)], compile_right=True)


def test_kernel_family_selection_for_scalar_second_inputs():
    """Shared-weight uvw products whose second input holds scalars only take the node-wise matrix-core kernel when the
    input multiplicities are multiples of 8; a handful of (u, v) pairs stays on the vector-ALU kernel with its weights
    in registers; anything with a non-scalar second input or per-sample weights takes the other kernels.  The choice is
    the same in fp32 and bf16 storage."""
    fam = lambda tp, dt=torch.float32: tp._plan(dt).family  # noqa: E731
    assert fam(ks.node_fctp()) == fam(ks.node_narrow()) == fam(ks.node_partial_tile()) == fam(ks.node_wide_out()) == "uvw_node"
    assert fam(ks.outer_split()) == fam(ks.mfma_small()) == "uvw_mfma"  # second input with l > 0
    assert fam(o3.FullyConnectedTensorProduct("8x0e+8x1o", "2x0e", "8x0e+8x1o")) == "uvw_small"  # 32 pairs: cached weights
    assert fam(o3.FullyConnectedTensorProduct("12x0e", "4x0e", "32x0e")) == "uvw_small"  # multiplicity not a multiple of 8
    assert fam(o3.FullyConnectedTensorProduct("64x0e", "4x0e", "64x0e", shared_weights=False, internal_weights=False)) == "uvw_small"
    assert fam(ks.cfg5(), torch.bfloat16) == "uvw_mfma"
    for tp in (ks.node_fctp(), ks.node_narrow(), ks.node_partial_tile(), ks.node_wide_out()):
        assert fam(tp, torch.bfloat16) == "uvw_node"
    # the layers of a radial network 8 -> 64 -> 352 as products with the constant "0e": same family in both storages
    for h_in, h_out, want in ((8, 64, "uvw_small"), (64, 352, "uvw_node")):
        layer = o3.TensorProduct(f"{h_in}x0e", "0e", f"{h_out}x0e", [(0, 0, 0, "uvw", True)], internal_weights=False, shared_weights=True)
        assert fam(layer) == fam(layer, torch.bfloat16) == want


def test_radial_message_kernel_is_offered_only_for_what_it_takes():
    """forward_gather_scatter_radial: two-layer network ending in the product's per-edge weights, all-uvu instructions
    with multiplicity 32; everything else is declined (None / False) so that callers run the two kernels."""
    from e3nn_amd import nn

    tp = ks.cfg3(merged=True)
    good = nn.FullyConnectedNet([8, 64, tp.weight_numel], torch.nn.functional.silu)
    assert tp._radial_description(good) == (8, 64, 1, pytest.approx(1.679, abs=2e-3), 1.0, 1.0)
    assert tp.prepare_gather_scatter_radial(good)  # builds (or finds) the kernel without a GPU
    assert tp._radial_description(nn.FullyConnectedNet([8, 64, 64, tp.weight_numel], torch.tanh)) is None  # three layers
    assert tp._radial_description(nn.FullyConnectedNet([8, 64, tp.weight_numel], torch.tanh, out_act=True)) is None
    assert tp._radial_description(nn.FullyConnectedNet([8, 64, tp.weight_numel + 32], torch.tanh)) is None  # other width
    assert not tp.prepare_gather_scatter_radial(nn.FullyConnectedNet([8, 24, tp.weight_numel], torch.tanh))  # hidden % 16
    assert not tp.prepare_gather_scatter_radial(nn.FullyConnectedNet([100, 64, tp.weight_numel], torch.tanh))  # inputs > 64
    other = ks.cfg4("A")  # multiplicities other than 32
    assert not other.prepare_gather_scatter_radial(nn.FullyConnectedNet([8, 16, other.weight_numel], torch.tanh))
    shared = ks.golden_tp("uvu_shared_v2")  # shared weights: nothing per edge to compute
    assert shared._radial_description(nn.FullyConnectedNet([8, 16, shared.weight_numel], torch.tanh)) is None


def test_weight_gradient_of_matrix_core_plans_with_unaligned_rows_builds():
    # legal reference configurations whose rows are not multiples of 4 floats (an irrep no output reaches, an odd
    # total dimension): forward on the matrix cores, weight gradient on the vector-ALU kernel, decided at plan level
    for tp in (ks.unaligned_mfma(), ks.unaligned_offsets(), o3.FullyConnectedTensorProduct("32x0e+1x1o", "0e", "32x0e")):
        plan = tp._plan(torch.float32)
        assert plan.family in ("uvw_mfma", "uvw_node")
        tp.compile_backward()
        assert _lib.lib().e3x_tp_plan_prepare_backward_w(plan.handle) == 0
    lin = o3.Linear("1x2e+32x0e", "32x0e")
    lin._tp.compile_backward()


def test_weight_gradient_entry_point_rejects_other_connection_modes():
    tp = ks.mixed_modes()
    plan = tp._plan(torch.float32)
    assert plan.family == "uvw_small"
    L = _lib.lib()
    assert L.e3x_tp_plan_prepare_backward_w(plan.handle) == _lib.ERR_INVALID
    one = ctypes.c_void_p(16)  # never dereferenced: the mode check comes first
    assert L.e3x_tp_backward_w_uvw(plan.handle, one, one, one, one, 4, None) == _lib.ERR_INVALID
    assert b"all-uvw" in L.e3x_last_error()


def test_provider_binding_builds_plans_from_constructor_data():
    # the code-generation provider a reference maintainer would register: plans built from Irreps + Instruction data
    from e3nn_amd import provider

    for tp in (ks.cfg1(), ks.cfg3(True), ks.mixed_modes()):
        gm = provider.hip_provider(tp.irreps_in1, tp.irreps_in2, tp.irreps_out, tp.instructions, tp.shared_weights, True, True)
        assert isinstance(gm, torch.fx.GraphModule)
        assert (gm.hip.weight_numel, gm.hip.in1_dim, gm.hip.out_dim) == (tp.weight_numel, tp.irreps_in1.dim, tp.irreps_out.dim)
        # the engine evaluates e3nn's already normalised path weights, not a second normalisation of them
        engine = gm.hip.engine()
        assert [t.path_weight for t in engine.instructions] == [t.path_weight for t in tp.instructions if 0 not in t.path_shape]
        assert engine._plan(torch.float32).key == tp._plan(torch.float32).key  # same specialised kernel
        assert list(gm.state_dict()) == []  # nothing of the engine leaks into the host module's state_dict
    empty = o3.TensorProduct("0x0e", "0e", "0e", [(0, 0, 0, "uvw", True)])
    assert provider.hip_provider(empty.irreps_in1, empty.irreps_in2, empty.irreps_out, empty.instructions, True, True, True) is None
    left, right = ["einsum code generator"], ["einsum code generator (right)"]
    provider.register(left, right)
    provider.register(left, right)
    assert left == [provider.hip_provider, "einsum code generator"]
    assert right == [provider.hip_provider_right, "einsum code generator (right)"]


class _Host(torch.nn.Module):
    """What the reference's ``CodeGenMixin`` does with a generated module (e3nn/util/codegen/_mixin.py:55-133): the
    submodule leaves the pickled state as ``pickle.dumps(submodule)`` bytes and comes back through ``pickle.loads``."""

    def __init__(self, gm):
        super().__init__()
        self.gm = gm

    def __getstate__(self):
        state = self.__dict__.copy()
        state["_modules"] = state["_modules"].copy()
        state["__codegen__"] = pickle.dumps(state["_modules"].pop("gm"))
        return state

    def __setstate__(self, state):
        state = state.copy()
        blob = state.pop("__codegen__")
        self.__dict__.update(state)
        self.gm = pickle.loads(blob)


def test_provider_module_pickles_and_deepcopies():
    # reference tests/o3/tensor_product_test.py:429-439 (deepcopy) and the torch.save / pickle life-cycle of a module
    # that owns a generated submodule; plan creation needs no GPU
    from e3nn_amd import provider

    for tp, right in ((ks.cfg1(), False), (ks.cfg3(True), False), (ks.mixed_modes(), False), (ks.cfg1(), True)):
        make = provider.hip_provider_right if right else provider.hip_provider
        gm = make(tp.irreps_in1, tp.irreps_in2, tp.irreps_out, tp.instructions, tp.shared_weights, True, True)
        key = gm.hip.engine()._plan(torch.float32).key
        buf = io.BytesIO()
        torch.save(gm, buf)
        buf.seek(0)
        copies = [pickle.loads(pickle.dumps(gm)), copy.deepcopy(gm), torch.load(buf, weights_only=False),
                  copy.deepcopy(_Host(gm)).gm, pickle.loads(pickle.dumps(_Host(gm))).gm]  # fmt: skip
        for c in copies:
            assert isinstance(c, torch.fx.GraphModule) and c is not gm and c.hip is not gm.hip
            assert c.hip._engine == []  # no handle travelled; the plan is rebuilt on first use
            assert (c.hip.irreps, c.hip.instructions, c.hip.shared_weights, c.hip.is_right) == (
                gm.hip.irreps, gm.hip.instructions, gm.hip.shared_weights, right)  # fmt: skip
            assert c.hip.engine()._plan(torch.float32).key == key
            assert c.code == gm.code


def test_provider_module_refuses_what_the_kernels_do_not_take():
    from e3nn_amd import provider

    tp = ks.cfg1()
    gm = provider.hip_provider(tp.irreps_in1, tp.irreps_in2, tp.irreps_out, tp.instructions, True, True, True)
    x1, x2, w = torch.zeros(2, tp.irreps_in1.dim), torch.zeros(2, tp.irreps_in2.dim), torch.zeros(tp.weight_numel)
    with pytest.raises(RuntimeError, match="GPU tensors only"):
        gm(x1, x2, w)
    with pytest.raises(RuntimeError, match="GPU tensors only"):
        gm(x1.requires_grad_(), x2, w)  # never a silent result without a grad_fn
    meta = lambda t, dt: torch.empty(t.shape, dtype=dt, device="meta")  # noqa: E731  (is_cuda False: refused before any launch)
    with pytest.raises(RuntimeError):
        gm(meta(x1, torch.float64), meta(x2, torch.float64), meta(w, torch.float64))
    # triangular modes have no right() in the reference either (_codegen.py:620-623): the provider defers
    tri = o3.TensorProduct("4x1o", "4x1o", "6x0e", [(0, 0, 0, "uvu<v", True)])
    assert provider.hip_provider_right(tri.irreps_in1, tri.irreps_in2, tri.irreps_out, tri.instructions, True, True, True) is None


def test_code_object_cache_remembers_rejected_sources_and_honours_no_jit(tmp_path, monkeypatch):
    # a cache directory of its own: nothing in it, so every plan below has to be compiled (or refused)
    monkeypatch.setenv("E3X_KERNEL_CACHE", str(tmp_path))
    tp = o3.FullyConnectedTensorProduct("64x0e", "64x0e", "64x0e")
    monkeypatch.setenv("E3X_NO_JIT", "1")
    with pytest.raises(_lib.E3xError, match="is not in the cache"):
        tp._plan(torch.bfloat16)
    monkeypatch.delenv("E3X_NO_JIT")
    # two weight buffers cannot hold a stage that is fetched three stages ahead: the template's static_assert rejects it
    monkeypatch.setenv("E3X_UVW16_NBUF", "2")
    with pytest.raises(_lib.E3xError, match="failed:"):
        tp._plan(torch.bfloat16)
    marks = sorted(p.name for p in tmp_path.iterdir() if p.name.endswith(".failed"))
    assert len(marks) == 2, marks  # the template as it is and its always-building form, both rejected for the same reason
    assert "static assertion failed" in (tmp_path / marks[0]).read_text()
    with pytest.raises(_lib.E3xError, match="failed before"):  # no compiler run this time
        tp._plan(torch.bfloat16)
    monkeypatch.delenv("E3X_UVW16_NBUF")
    plan = tp._plan(torch.bfloat16)  # the defaults build, into the same directory
    assert (tmp_path / (plan.key + ".hsaco")).exists() and plan.family == "uvw_mfma"
