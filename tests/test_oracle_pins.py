"""Pins the CPU oracle: golden fixtures written from the reference, closed forms,
library routines and brute force.  No GPU, no product code."""
import math

import numpy as np
import pytest

from oracle import irreps as ir_
from oracle import tensor_product as otp
from oracle.message_passing import gather, scatter, tp_gather_scatter
from oracle.spherical_harmonics import spherical_harmonics as osh
from oracle.wigner import su2_clebsch_gordan, wigner_3j

RUN_CASES = [
    "fctp_cfg1", "fctp_small_cfg5_like", "fctp_per_sample_weights", "fctp_norm_path",
    "uvu_merged_cfg3_like_mul4", "uvu_builder_cfg3_like_mul4", "uvu_builderA_cfg4_like_mul2",
    "uvu_builderB_cfg4_like_mul2", "uvu_shared_v2", "uvu_mixed_weightless",
    "modes_uuu_uvuv_uuw_uvv", "modes_triangular", "empty_path_and_missing_output",
]  # fmt: skip


def spec_from_meta(m, **kw):
    upw = m.get("user_path_weights", [1.0] * len(m["instructions"]))
    ins = [tuple(t[:5]) + (pw,) for t, pw in zip(m["instructions"], upw)]
    return otp.make_spec(m["irreps_in1"], m["irreps_in2"], m["irreps_out"], ins, shared_weights=m["shared_weights"], **kw)


# ---------------------------------------------------------------- wigner 3j
def test_w3j_matches_reference_golden(golden_w3j):
    assert len(golden_w3j) > 60
    for key, ref in golden_w3j.items():
        l1, l2, l3 = map(int, key.split("_"))
        np.testing.assert_allclose(wigner_3j(l1, l2, l3), ref, atol=1e-13, rtol=0)


def test_w3j_closed_forms():
    eps = np.zeros((3, 3, 3))
    for a, b, c in ((0, 1, 2), (1, 2, 0), (2, 0, 1)):
        eps[a, b, c], eps[a, c, b] = 1, -1
    np.testing.assert_allclose(wigner_3j(1, 1, 1), eps / math.sqrt(6), atol=1e-14)
    for l in range(5):
        eye = np.eye(2 * l + 1) / math.sqrt(2 * l + 1)
        np.testing.assert_allclose(wigner_3j(0, l, l)[0], eye, atol=1e-14)
        np.testing.assert_allclose(wigner_3j(l, 0, l)[:, 0], eye, atol=1e-14)
        np.testing.assert_allclose(wigner_3j(l, l, 0)[:, :, 0], eye, atol=1e-14)


def test_w3j_norm_and_permutation_symmetry():
    for l1, l2, l3 in ((1, 2, 3), (2, 2, 2), (3, 3, 2), (1, 3, 3), (2, 3, 4)):
        c = wigner_3j(l1, l2, l3)
        assert abs(np.linalg.norm(c) - 1) < 1e-14
        s = (-1) ** (l1 + l2 + l3)
        np.testing.assert_allclose(c, np.transpose(wigner_3j(l2, l3, l1), (2, 0, 1)), atol=1e-14)
        np.testing.assert_allclose(c, s * np.transpose(wigner_3j(l2, l1, l3), (1, 0, 2)), atol=1e-14)
        np.testing.assert_allclose(c, s * np.transpose(wigner_3j(l1, l3, l2), (0, 2, 1)), atol=1e-14)


def test_su2_cg_matches_sympy():
    sympy_wigner = pytest.importorskip("sympy.physics.wigner")
    for j1, j2, j3 in ((1, 1, 2), (2, 1, 2), (2, 3, 3), (3, 3, 1)):
        c = su2_clebsch_gordan(j1, j2, j3)
        for m1 in range(-j1, j1 + 1):
            for m2 in range(-j2, j2 + 1):
                if abs(m1 + m2) <= j3:
                    ref = float(sympy_wigner.clebsch_gordan(j1, j2, j3, m1, m2, m1 + m2))
                    assert abs(c[j1 + m1, j2 + m2, j3 + m1 + m2] - ref) < 1e-13


# ---------------------------------------------------------------- irreps / structure
def test_sort_matches_reference_golden(golden_tp):
    for s, ref in golden_tp[0]["sort"].items():
        srt, p, inv = ir_.sort(ir_.parse(s))
        assert ir_.to_str(srt) == ref["irreps"] and list(p) == ref["p"] and list(inv) == ref["inv"]


def test_instruction_tables_match_reference_golden(golden_tp):
    meta = golden_tp[0]
    kw = {"fctp_norm_path": dict(irrep_normalization="norm", path_normalization="path")}
    n = 0
    for name, m in meta.items():
        if "instructions" not in m:
            continue
        spec = spec_from_meta(m, **kw.get(name, {}))
        assert spec.weight_numel == m["weight_numel"], name
        assert ir_.dim(spec.irreps_out) == ir_.dim(ir_.parse(m["irreps_out"]))
        for t, ref in zip(spec.instructions, m["instructions"]):
            assert abs(t.path_weight - ref[5]) <= 1e-15 * max(1, abs(ref[5])), name
            assert list(t.path_shape) == ref[6], name
        mask = otp.output_mask(spec)
        for sl, flag in zip(ir_.slices(spec.irreps_out), m["output_mask_blocks"]):
            if flag >= 0:
                assert (mask[sl] == flag).all(), name
        n += 1
    assert n >= 18


def test_builders_match_reference_golden(golden_tp):
    meta = golden_tp[0]
    m = meta["fctp_cfg1"]
    ins = otp.fully_connected_instructions(m["irreps_in1"], m["irreps_in2"], m["irreps_out"])
    assert [list(t[:3]) for t in ins] == [t[:3] for t in m["instructions"]]
    m = meta["fctp_cfg5_structure"]
    ins = otp.fully_connected_instructions(m["irreps_in1"], m["irreps_in2"], m["irreps_out"])
    assert [list(t[:3]) for t in ins] == [t[:3] for t in m["instructions"]] and len(ins) == 11
    assert m["weight_numel"] == 23068672
    for name, keep in (
        ("uvu_builder_cfg3_structure", {(0, 1), (1, -1), (2, 1)}),
        ("uvu_builderA_cfg4_structure", {(0, 1), (1, -1), (2, 1), (3, -1)}),
        ("uvu_builderB_cfg4_structure", {(l, p) for l in range(4) for p in (1, -1)}),
    ):
        m = meta[name]
        mid, ins = otp.convolution_instructions(m["irreps_in1"], m["irreps_in2"], lambda l, p: (l, p) in keep)
        assert ir_.to_str(mid) == m["irreps_out"], name
        assert [list(t[:3]) for t in ins] == [t[:3] for t in m["instructions"]], name
    assert meta["uvu_builderA_cfg4_structure"]["weight_numel"] == 2944
    assert meta["uvu_builderB_cfg4_structure"]["weight_numel"] == 4352
    assert meta["uvu_merged_cfg3_structure"]["weight_numel"] == 352


def test_fully_connected_normalization_identity():
    # reference tests/o3/tensor_product_sub_test.py:30-40
    a = otp.make_spec("10x0e", "10x0e", "0e", otp.fully_connected_instructions("10x0e", "10x0e", "0e"))
    b = otp.make_spec("3x0e+7x0e", "3x0e+7x0e", "0e", otp.fully_connected_instructions("3x0e+7x0e", "3x0e+7x0e", "0e"))
    x, y = np.random.default_rng(0).standard_normal((2, 4, 10))
    ra = otp.tp_forward(a, x, y, np.ones(a.weight_numel))
    rb = otp.tp_forward(b, x, y, np.ones(b.weight_numel))
    np.testing.assert_allclose(ra, rb, atol=1e-12)


# ---------------------------------------------------------------- contraction
@pytest.mark.parametrize("name", RUN_CASES)
def test_tp_forward_matches_reference_golden(golden_tp, name):
    meta, arr = golden_tp
    kw = dict(irrep_normalization="norm", path_normalization="path") if name == "fctp_norm_path" else {}
    spec = spec_from_meta(meta[name], **kw)
    out = otp.tp_forward(spec, arr[name + "/x1"], arr[name + "/x2"], arr[name + "/w"])
    assert out.shape == arr[name + "/out"].shape
    np.testing.assert_allclose(out, arr[name + "/out"], atol=1e-12, rtol=1e-12)


@pytest.mark.parametrize("name", ["fctp_small_cfg5_like", "uvu_merged_cfg3_like_mul4", "uvu_shared_v2", "fctp_per_sample_weights"])
def test_tp_forward_matches_brute_force_loops(golden_tp, name):
    meta, arr = golden_tp
    spec = spec_from_meta(meta[name])
    x1, x2, w = arr[name + "/x1"][:2], arr[name + "/x2"][:2], arr[name + "/w"]
    w = w if spec.shared_weights else w[:2]
    np.testing.assert_allclose(otp.tp_forward(spec, x1, x2, w), otp.tp_forward_loops(spec, x1, x2, w), atol=1e-12)


def test_tp_special_cases_reduce_to_library_routines():
    rng = np.random.default_rng(1)
    # 1o x 1o -> 1e, uuu: cross product / sqrt(6) * sqrt(3)   (component normalisation, one path)
    spec = otp.make_spec("4x1o", "4x1o", "4x1e", [(0, 0, 0, "uuu", False)])
    a, b = rng.standard_normal((2, 3, 12))
    ref = np.cross(a.reshape(3, 4, 3), b.reshape(3, 4, 3)).reshape(3, 12) / math.sqrt(2)
    np.testing.assert_allclose(otp.tp_forward(spec, a, b), ref, atol=1e-13)
    # l x l -> 0e: dot product / sqrt(2l+1)
    spec = otp.make_spec("1x2e", "1x2e", "1x0e", [(0, 0, 0, "uvw", True)])
    a, b = rng.standard_normal((2, 5, 5))
    np.testing.assert_allclose(otp.tp_forward(spec, a, b, np.array([2.0]))[:, 0], 2 * (a * b).sum(1) / math.sqrt(5), atol=1e-13)
    # all-scalar uvw: bilinear form / sqrt(U V)
    spec = otp.make_spec("3x0e", "2x0e", "4x0e", [(0, 0, 0, "uvw", True)])
    a, b, w = rng.standard_normal((5, 3)), rng.standard_normal((5, 2)), rng.standard_normal(24)
    ref = np.einsum("zu,zv,uvw->zw", a, b, w.reshape(3, 2, 4)) / math.sqrt(6)
    np.testing.assert_allclose(otp.tp_forward(spec, a, b, w), ref, atol=1e-13)
    # 0e x l -> l: scalar times vector (path weight sqrt(2l+1) cancels the 1/sqrt(2l+1) of the 3j)
    spec = otp.make_spec("1x0e", "1x1o", "1x1o", [(0, 0, 0, "uvu", True)], shared_weights=False)
    a, b, w = rng.standard_normal((5, 1)), rng.standard_normal((5, 3)), rng.standard_normal((5, 1))
    np.testing.assert_allclose(otp.tp_forward(spec, a, b, w), w * a * b, atol=1e-13)


def test_tp_output_variance_is_one():
    # reference _tensor_product.py:179-182 and tests/o3/tensor_product_test.py:81-85
    rng = np.random.default_rng(2)
    ins = otp.fully_connected_instructions("8x0e+8x1o", "0e+1o+2e", "8x0e+8x1o+8x2e")
    spec = otp.make_spec("8x0e+8x1o", "0e+1o+2e", "8x0e+8x1o+8x2e", ins)
    Z = 4000
    out = otp.tp_forward(spec, rng.standard_normal((Z, 32)), rng.standard_normal((Z, 9)), rng.standard_normal(spec.weight_numel))
    for sl in ir_.slices(spec.irreps_out):
        assert abs(out[:, sl].var() - 1) < 0.25


# ---------------------------------------------------------------- spherical harmonics
def test_sh_matches_reference_golden(golden_sh):
    pts = golden_sh["points"]
    for normalize in (True, False):
        for normalization in ("integral", "component", "norm"):
            ref = golden_sh[f"lmax8_{int(normalize)}_{normalization}"]
            got = osh(list(range(9)), pts, normalize, normalization)
            scale = np.maximum(1.0, np.abs(ref))
            assert (np.abs(got - ref) / scale).max() < 1e-11
            got3 = osh(list(range(4)), pts, normalize, normalization)  # closed forms
            assert (np.abs(got3 - ref[:, :16]) / scale[:, :16]).max() < 1e-12
    np.testing.assert_allclose(osh([2, 0, 3], pts, True, "component"), golden_sh["ls_2_0_3_1_component"], atol=1e-12)


def test_sh_matches_scipy_complex_harmonics():
    # docstring of the reference (_spherical_harmonics.py:142-148): equals the standard real
    # harmonics when evaluated with arguments ordered (y, z, x), 'integral' normalisation
    sp = pytest.importorskip("scipy.special")
    rng = np.random.default_rng(3)
    v = rng.standard_normal((50, 3))
    v /= np.linalg.norm(v, axis=1, keepdims=True)
    X, Y, Z = v[:, 2], v[:, 0], v[:, 1]  # e3nn (x, y, z) = standard (y, z, x)
    theta, phi = np.arccos(Z), np.arctan2(Y, X)  # polar, azimuth of the standard frame
    for l in range(6):
        got = osh(l, v, True, "integral")
        for m in range(-l, l + 1):
            if hasattr(sp, "sph_harm_y"):
                ylm = sp.sph_harm_y(l, abs(m), theta, phi)
            else:
                ylm = sp.sph_harm(abs(m), l, phi, theta)
            if m == 0:
                ref = ylm.real
            elif m > 0:
                ref = math.sqrt(2) * (-1) ** m * ylm.real
            else:
                ref = math.sqrt(2) * (-1) ** m * ylm.imag
            np.testing.assert_allclose(got[:, l + m], ref, atol=1e-12)


def test_sh_identities():
    rng = np.random.default_rng(4)
    v = rng.standard_normal((20, 3))
    for l in range(9):
        c = osh(l, v, True, "component")
        np.testing.assert_allclose((c**2).sum(1), 2 * l + 1, rtol=1e-12)  # reference test :83-92
        np.testing.assert_allclose(osh(l, -v, False, "component"), (-1) ** l * osh(l, v, False, "component"), atol=1e-9)
    z = osh([0, 1], np.zeros((1, 3)), False, "norm")  # reference test :45-48
    np.testing.assert_array_equal(z, [[1, 0, 0, 0]])
    z = osh([0, 1, 2], np.zeros((1, 3)), True, "component")
    assert z[0, 0] == 1 and not z[0, 1:].any()
    # recurrence with positive constant, reference test :124-137
    x = rng.standard_normal(3)
    for l in range(6):
        a = osh(l + 1, x, False, "component")
        b = np.einsum("ijk,j,k->i", wigner_3j(l + 1, l, 1), osh(l, x, False, "component"), x)
        np.testing.assert_allclose(a / np.linalg.norm(a), b / np.linalg.norm(b), atol=1e-12)


# ---------------------------------------------------------------- gather / scatter
def test_gather_scatter_integer_payload_is_exact():
    rng = np.random.default_rng(5)
    N, E, F = 13, 200, 7
    x = rng.integers(-50, 50, (N, F)).astype(np.float32)
    src, dst = rng.integers(0, N, E), rng.integers(0, N - 2, E)
    msg = gather(x, src)
    out = scatter(msg, dst, N)
    ref = np.zeros((N, F), np.float32)
    for e in range(E):
        ref[dst[e]] += x[src[e]]
    assert (out == ref).all() and not out[N - 2 :].any()
    assert (gather(x, src - N) == msg).all()  # negative indices wrap like torch indexing
    with pytest.raises(IndexError):
        gather(x, np.array([N]))
    with pytest.raises(IndexError):
        scatter(msg, dst + N, N)
    assert (scatter(msg, dst.astype(np.int32), N) == out).all()


def test_conv_matches_reference_golden(golden_tp):
    meta, arr = golden_tp
    spec = spec_from_meta(meta["conv_small"])
    g = {k.split("/")[1]: v for k, v in arr.items() if k.startswith("conv_small/")}
    np.testing.assert_allclose(osh([0, 1, 2], g["vec"], True, "component"), g["attr"], atol=1e-13)
    out = tp_gather_scatter(spec, g["node_x"], g["attr"], g["w"], g["src"], g["dst"], g["node_x"].shape[0])
    np.testing.assert_allclose(out, g["out"], atol=1e-12)
    assert not out[-1].any()


# ---------------------------------------------------------------- torch-CPU restatement (timed baseline, backward oracle)
TORCH_CASES = [  # every golden case whose instructions are all weighted uvu / uvw, the modes the restatement covers
    "fctp_cfg1", "fctp_small_cfg5_like", "fctp_per_sample_weights", "fctp_norm_path", "uvu_merged_cfg3_like_mul4",
    "uvu_builder_cfg3_like_mul4", "uvu_builderA_cfg4_like_mul2", "uvu_builderB_cfg4_like_mul2", "uvu_shared_v2",
]  # fmt: skip


@pytest.mark.parametrize("name", TORCH_CASES)
def test_torch_restatement_matches_reference_golden(golden_tp, name):
    import torch

    from oracle.torch_cpu import tp_forward_torch

    meta, arr = golden_tp
    kw = dict(irrep_normalization="norm", path_normalization="path") if name == "fctp_norm_path" else {}
    spec = spec_from_meta(meta[name], **kw)
    x1, x2, w = (torch.from_numpy(arr[f"{name}/{k}"]) for k in ("x1", "x2", "w"))
    assert x1.dtype == torch.float64
    out = tp_forward_torch(spec, x1, x2, w).numpy()
    assert out.shape == arr[name + "/out"].shape
    np.testing.assert_allclose(out, arr[name + "/out"], atol=1e-12, rtol=1e-12)


def test_torch_restatement_matches_numpy_oracle_on_the_benchmark_sets():
    # the instruction sets of the benchmark at reduced multiplicity, all five l-specialisations of the einsum strings
    import torch

    from oracle.torch_cpu import tp_forward_torch

    rng = np.random.default_rng(3)
    sh3 = "0e+1o+2e+3o"
    mid, ins = otp.convolution_instructions("6x0e+6x1o+6x2e+6x3o", sh3, lambda l, p: p == (-1) ** l and l <= 3)
    uvu = otp.make_spec("6x0e+6x1o+6x2e+6x3o", sh3, ir_.to_str(mid), ins, shared_weights=False)
    assert len(ins) == 23
    f = "5x0e+5x1o+5x2e"
    uvw = otp.make_spec(f, f, f, otp.fully_connected_instructions(f, f, f), shared_weights=True)
    for spec in (uvu, uvw):
        Z = 7
        x1 = rng.standard_normal((Z, ir_.dim(spec.irreps_in1)))
        x2 = rng.standard_normal((Z, ir_.dim(spec.irreps_in2)))
        w = rng.standard_normal((spec.weight_numel,) if spec.shared_weights else (Z, spec.weight_numel))
        ref = otp.tp_forward(spec, x1, x2, w)
        got = tp_forward_torch(spec, torch.from_numpy(x1), torch.from_numpy(x2), torch.from_numpy(w)).numpy()
        np.testing.assert_allclose(got, ref, atol=1e-12, rtol=1e-12)
        assert np.abs(ref).max() > 0.5  # not a comparison of zeros


def test_torch_gather_scatter_matches_reference_golden(golden_tp):
    import torch

    from oracle.torch_cpu import scatter_torch, tp_gather_scatter_torch

    meta, arr = golden_tp
    spec = spec_from_meta(meta["conv_small"])
    g = {k.split("/")[1]: v for k, v in arr.items() if k.startswith("conv_small/")}
    t = {k: torch.from_numpy(v) for k, v in g.items()}
    N = g["node_x"].shape[0]
    out = tp_gather_scatter_torch(spec, t["node_x"], t["attr"], t["w"], t["src"].long(), t["dst"].long(), N).numpy()
    np.testing.assert_allclose(out, g["out"], atol=1e-12)
    # int32 destinations are widened; integer payloads sum exactly
    msg = torch.arange(40, dtype=torch.float64).reshape(10, 4)
    dst = torch.tensor([3, 0, 3, 1, 0, 0, 4, 3, 1, 0], dtype=torch.int32)
    ref = np.zeros((6, 4))
    np.add.at(ref, dst.numpy(), msg.numpy())
    assert (scatter_torch(msg, dst.long(), 6).numpy() == ref).all()


def test_torch_spherical_harmonics_match_reference_golden(golden_sh):
    import torch

    from oracle.torch_cpu import spherical_harmonics_torch

    pts = torch.from_numpy(golden_sh["points"])
    for lmax in (1, 2, 3):
        n = (lmax + 1) ** 2
        for normalize in (True, False):
            ref = golden_sh[f"lmax8_{int(normalize)}_component"][:, :n]
            got = spherical_harmonics_torch(lmax, pts, normalize).numpy()
            assert (np.abs(got - ref) / np.maximum(1.0, np.abs(ref))).max() < 1e-12
    zero = spherical_harmonics_torch(3, torch.zeros(2, 3, dtype=torch.float64), True).numpy()
    assert (zero[:, 0] == 1).all() and not zero[:, 1:].any()  # reference _spherical_harmonics.py:96


# ---------------------------------------------------------------- rotations (equivariance tooling)
def test_wigner_D_is_a_representation_and_w3j_is_invariant():
    from oracle.rotation import irreps_D, random_rotation, wigner_D

    rng = np.random.default_rng(7)
    R1, R2 = random_rotation(rng), random_rotation(rng)
    np.testing.assert_allclose(wigner_D(1, R1), R1, atol=1e-12)  # reference tests/o3/wigner_test.py:28-32 (x,y,z order)
    for l in range(5):
        D1, D2, D12 = wigner_D(l, R1), wigner_D(l, R2), wigner_D(l, R1 @ R2)
        np.testing.assert_allclose(D1 @ D2, D12, atol=1e-10)
        np.testing.assert_allclose(D1 @ D1.T, np.eye(2 * l + 1), atol=1e-10)
    # C_ijk D_il D_jm D_kn = C_lmn  (reference tests/o3/wigner_test.py:15-25)
    for l1, l2, l3 in ((1, 1, 1), (1, 2, 3), (2, 2, 2), (3, 3, 2), (2, 3, 3), (1, 3, 3)):
        C = wigner_3j(l1, l2, l3)
        Cr = np.einsum("ijk,il,jm,kn->lmn", C, wigner_D(l1, R1), wigner_D(l2, R1), wigner_D(l3, R1))
        np.testing.assert_allclose(Cr, C, atol=1e-10)
    # the oracle tensor product is equivariant under rotation and inversion
    ins = otp.fully_connected_instructions("2x0e+2x1o+1x2e", "0e+1o+2e", "2x0e+2x1o+2x2e+1x1e")
    spec = otp.make_spec("2x0e+2x1o+1x2e", "0e+1o+2e", "2x0e+2x1o+2x2e+1x1e", ins)
    x1, x2, w = rng.standard_normal((4, 13)), rng.standard_normal((4, 9)), rng.standard_normal(spec.weight_numel)
    for improper in (False, True):
        Da, Db, Dc = (irreps_D(s, R1, improper) for s in ("2x0e+2x1o+1x2e", "0e+1o+2e", "2x0e+2x1o+2x2e+1x1e"))
        lhs = otp.tp_forward(spec, x1 @ Da.T, x2 @ Db.T, w)
        rhs = otp.tp_forward(spec, x1, x2, w) @ Dc.T
        np.testing.assert_allclose(lhs, rhs, atol=1e-10)


# ---- node-wise blocks either side of the message (oracle/nn.py) against fixtures written from the reference ----
import json as _json
import os as _os


def _nn_golden():
    here = _os.path.join(_os.path.dirname(_os.path.abspath(__file__)), "golden")
    return np.load(_os.path.join(here, "nn_cases.npz")), _json.load(open(_os.path.join(here, "nn_cases.json")))


@pytest.mark.parametrize("name", ["linear_mixed", "linear_path_norm", "linear_bias"])
def test_linear_matches_reference(name):
    from oracle import nn as onn

    arr, meta = _nn_golden()
    m = meta[name]
    kw = m["kwargs"]
    ins = onn.linear_instructions(m["irreps_in"], m["irreps_out"], None, kw.get("path_normalization", "element"))
    ref_ins = [t for t in m["instructions"] if t[0] != -1]
    assert [(a, b) for a, b, _, _ in ins] == [(t[0], t[1]) for t in ref_ins]
    np.testing.assert_allclose([t[3] for t in ins], [t[3] for t in ref_ins], rtol=1e-14)
    from oracle import irreps as oir

    biases = [bool(kw.get("biases")) and l == 0 for _, l, _ in oir.parse(m["irreps_out"])] if kw.get("biases") else None
    out = onn.linear_forward(m["irreps_in"], m["irreps_out"], arr[name + "/x"], arr[name + "/w"],
                             path_normalization=kw.get("path_normalization", "element"), bias=arr[name + "/bias"], biases=biases)  # fmt: skip
    np.testing.assert_allclose(out, arr[name + "/out"], rtol=1e-12, atol=1e-12)


def test_linear_closed_form_on_scalars():
    from oracle import nn as onn

    rng = np.random.default_rng(0)
    x, w = rng.normal(size=(5, 10)), rng.normal(size=30)
    np.testing.assert_allclose(onn.linear_forward("10x0e", "3x0e", x, w), x @ w.reshape(10, 3) / np.sqrt(10), rtol=1e-13)


def test_activation_constants_and_forward_match_reference():
    from oracle import nn as onn

    arr, meta = _nn_golden()
    for k, v in meta["cst"].items():
        assert onn.normalize2mom_const(k) == pytest.approx(v, rel=1e-13)
    m = meta["activation"]
    out, irreps_out = onn.activation_forward(m["irreps_in"], m["acts"], arr["activation/x"])
    from oracle import irreps as oir

    assert oir.to_str(irreps_out) == m["irreps_out"]
    np.testing.assert_allclose(out, arr["activation/out"], rtol=1e-12, atol=1e-13)


@pytest.mark.parametrize("name", ["gate_plain", "gate_parity", "gate_only_scalars", "gate_entries_as_given", "gate_gated_in_pieces"])
def test_gate_matches_reference(name):
    from oracle import irreps as oir
    from oracle import nn as onn

    arr, meta = _nn_golden()
    m = meta[name]
    out, irreps_in, irreps_out = onn.gate_forward(*m["args"], arr[name + "/x"])
    assert oir.to_str(irreps_in) == m["irreps_in"]
    assert oir.to_str(irreps_out) == m["irreps_out"] or oir.to_str(oir.simplify(irreps_out)) == oir.to_str(oir.simplify(oir.parse(m["irreps_out"])))
    np.testing.assert_allclose(out, arr[name + "/out"], rtol=1e-12, atol=1e-13)


def test_fully_connected_net_matches_reference():
    from oracle import nn as onn

    arr, meta = _nn_golden()
    out = onn.fc_forward([arr[f"fc/w{i}"] for i in range(3)], arr["fc/x"], meta["fc"]["act"])
    np.testing.assert_allclose(out, arr["fc/out"], rtol=1e-12, atol=1e-13)


def test_convolution_matches_reference():
    from oracle import nn as onn

    arr, meta = _nn_golden()
    a = meta["conv"]["args"]
    params = {k[len("conv/param/"):]: arr[k] for k in arr.files if k.startswith("conv/param/")}
    out = onn.convolution_forward(a[0], a[1], a[2], a[3], a[5], params, arr["conv/node_input"], arr["conv/node_attr"],
                                  arr["conv/src"], arr["conv/dst"], arr["conv/edge_attr"], arr["conv/edge_scalars"])  # fmt: skip
    np.testing.assert_allclose(out, arr["conv/out"], rtol=1e-11, atol=1e-12)
