"""GPU parity: o3.TensorProduct / FullyConnectedTensorProduct (HIP, through the C ABI) against the CPU oracle
and the golden outputs written from the reference."""
import numpy as np
import pytest
import torch

from e3nn_amd import o3
from oracle import tensor_product as otp
from tests import kernel_sets as ks
from tests.helpers import assert_close, oracle_spec, seeded

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

PLAIN_CASES = [c for c in ks.GOLDEN_GPU_CASES if c != "conv_small"]


@pytest.mark.parametrize("name", PLAIN_CASES)
def test_matches_reference_golden(golden_tp, name):
    meta, arr = golden_tp
    tp = ks.golden_tp(name, meta).to(DEV)
    x1 = torch.from_numpy(arr[name + "/x1"]).float().to(DEV)
    x2 = torch.from_numpy(arr[name + "/x2"]).float().to(DEV)
    w = torch.from_numpy(arr[name + "/w"]).float().to(DEV)
    if tp.internal_weights:
        with torch.no_grad():
            tp.weight.copy_(w)
        out = tp(x1, x2)
    elif tp.weight_numel:
        out = tp(x1, x2, w)
    else:
        out = tp(x1, x2)
    assert_close(out, arr[name + "/out"], what=name)
    # structure against the reference's tables
    m = meta[name]
    assert tp.weight_numel == m["weight_numel"]
    for t, ref in zip(tp.instructions, m["instructions"]):
        assert abs(t.path_weight - ref[5]) < 1e-14 and list(t.path_shape) == ref[6]
    for sl, flag in zip(tp.irreps_out.slices(), m["output_mask_blocks"]):
        if flag >= 0:
            assert (tp.output_mask[sl] == flag).all()


def test_general_connection_modes_against_oracle():
    # uvu + uvw + uvv + uuu + uuw (unweighted) in one instruction set, per-sample weights
    tp = ks.mixed_modes()
    x1, x2 = seeded(37, tp.irreps_in1.dim, seed=1), seeded(37, tp.irreps_in2.dim, seed=2)
    w = seeded(37, tp.weight_numel, seed=3)
    out = tp(x1.to(DEV), x2.to(DEV), w.to(DEV))
    ref = otp.tp_forward(oracle_spec(tp), x1.numpy(), x2.numpy(), w.numpy())
    assert_close(out, ref, what="mixed modes")


def test_cfg1_full_size_against_oracle():
    # FCTP('16x0e+16x1o', '0e+1o+2e' -> '16x0e+16x1o+16x2e'), batch 4096, x2 = SH(lmax 2) of unit vectors, seed 0
    g = torch.Generator().manual_seed(0)
    tp = ks.cfg1().to(DEV)
    w = torch.randn(tp.weight_numel, generator=g)
    x1 = torch.randn(4096, 64, generator=g)
    v = torch.randn(4096, 3, generator=g)
    v = v / v.norm(dim=1, keepdim=True)
    x2 = o3.spherical_harmonics([0, 1, 2], v.to(DEV), True, "component")
    with torch.no_grad():
        tp.weight.copy_(w)
    out = tp(x1.to(DEV), x2)
    ref = otp.tp_forward(oracle_spec(tp), x1.numpy(), x2.cpu().numpy(), w.numpy())
    assert_close(out, ref, what="cfg1")
    assert abs(out.var().item() - 1) < 0.2  # unit output variance


def test_batch_broadcasting_weight_lists_and_errors():
    tp = ks.golden_tp("fctp_per_sample_weights").to(DEV)  # shared_weights=False
    spec = oracle_spec(tp)
    x1 = seeded(3, 1, tp.irreps_in1.dim, seed=1)
    x2 = seeded(1, 4, tp.irreps_in2.dim, seed=2)
    w = seeded(3, 4, tp.weight_numel, seed=3)
    out = tp(x1.to(DEV), x2.to(DEV), w.to(DEV))
    assert out.shape == (3, 4, tp.irreps_out.dim)
    ref = otp.tp_forward(
        spec, x1.expand(3, 4, -1).reshape(12, -1).numpy(), x2.expand(3, 4, -1).reshape(12, -1).numpy(), w.reshape(12, -1).numpy()
    ).reshape(3, 4, -1)
    assert_close(out, ref)
    # weights given as a list of per-instruction tensors (the reference flattens their batch dims to one)
    x1f, x2f = x1.expand(3, 4, -1).reshape(12, -1).to(DEV), x2.expand(3, 4, -1).reshape(12, -1).to(DEV)
    wl = [v.contiguous() for v in tp.weight_views(w.reshape(12, -1).to(DEV))]
    assert torch.equal(tp(x1f, x2f, wl), out.reshape(12, -1))
    with pytest.raises(RuntimeError):
        tp(x1.to(DEV), x2.to(DEV))  # external weights are mandatory
    # shape checks are torch._assert like the reference's: AssertionError in eager mode
    with pytest.raises((RuntimeError, AssertionError)):
        tp(x1.to(DEV), x2.to(DEV), w.to(DEV)[..., :-1])
    with pytest.raises((RuntimeError, AssertionError)):
        tp(x1.to(DEV), x2.to(DEV), w.to(DEV)[0, 0])  # no batch dimension on per-sample weights
    with pytest.raises((RuntimeError, AssertionError)):
        tp(x1.to(DEV)[..., :-1], x2.to(DEV), w.to(DEV))
    # "weird" batch dimensions broadcast like the reference (tests/o3/tensor_product_test.py:346-358)
    a, b, c = seeded(2, 1, 4, tp.irreps_in1.dim, seed=5).to(DEV), seeded(2, 3, 1, tp.irreps_in2.dim, seed=6).to(DEV), seeded(3, 4, tp.weight_numel, seed=7).to(DEV)
    full = tp(a.expand(2, 3, 4, -1).reshape(24, -1), b.expand(2, 3, 4, -1).reshape(24, -1), c[None].expand(2, 3, 4, -1).reshape(24, -1))
    assert torch.equal(tp(a, b, c).reshape(24, -1), full)
    with pytest.raises(RuntimeError):
        tp(x1, x2, w)  # CPU tensors: no silent fallback
    shared = ks.golden_tp("fctp_cfg1").to(DEV)
    with pytest.raises((RuntimeError, AssertionError)):
        shared(seeded(2, 64).to(DEV), seeded(2, 9).to(DEV), seeded(2, shared.weight_numel).to(DEV))
    # empty batch
    assert shared(torch.zeros(0, 64, device=DEV), torch.zeros(0, 9, device=DEV)).shape == (0, 144)


def test_product_without_instructions_gives_zeros():
    # no path is allowed by parity (e3nn builds such a product without complaint): zeros forward, zero gradients
    tp = o3.FullyConnectedTensorProduct("8x3o", "64x2e", "16x2e").to(DEV)
    assert len(tp.instructions) == 0 and tp.weight_numel == 0
    x1 = seeded(5, tp.irreps_in1.dim).to(DEV).requires_grad_(True)
    x2 = seeded(5, tp.irreps_in2.dim, seed=1).to(DEV).requires_grad_(True)
    out = tp(x1, x2)
    assert out.shape == (5, 80) and not out.any()
    g1, g2 = torch.autograd.grad(out, (x1, x2), torch.ones_like(out), allow_unused=True)
    assert (g1 is None or not g1.any()) and (g2 is None or not g2.any())


def test_missing_output_paths_are_exact_zeros():
    tp = ks.golden_tp("empty_path_and_missing_output").to(DEV)
    out = tp(seeded(6, tp.irreps_in1.dim).to(DEV), seeded(6, tp.irreps_in2.dim, seed=1).to(DEV))
    sl = tp.irreps_out.slices()[1]
    assert not out[:, sl].any() and out[:, tp.irreps_out.slices()[0]].any()
    assert tp.output_mask[sl].sum() == 0


def test_bilinearity_and_weight_linearity():
    tp = ks.cfg3(True)
    Z = 257
    x1, x1b = seeded(Z, 288, seed=1).to(DEV), seeded(Z, 288, seed=2).to(DEV)
    x2 = seeded(Z, 9, seed=3).to(DEV)
    w, wb = seeded(Z, 352, seed=4).to(DEV), seeded(Z, 352, seed=5).to(DEV)
    a = tp(x1 + 0.5 * x1b, x2, w)
    b = tp(x1, x2, w) + 0.5 * tp(x1b, x2, w)
    assert (a - b).abs().max().item() < 2e-5
    a = tp(x1, x2, w + 2 * wb)
    b = tp(x1, x2, w) + 2 * tp(x1, x2, wb)
    assert (a - b).abs().max().item() < 5e-5


@pytest.mark.parametrize("maker,Z", [(lambda: ks.cfg3(True), 1000), (lambda: ks.cfg3(False), 333), (lambda: ks.cfg4("A"), 130),
                                     (lambda: ks.cfg4("B"), 70), (ks.odd_mul, 129)])  # fmt: skip
def test_plain_uvu_benchmark_instruction_sets(maker, Z):
    tp = maker()
    x1 = seeded(Z, tp.irreps_in1.dim, seed=11)
    x2 = seeded(Z, tp.irreps_in2.dim, seed=12)
    w = seeded(Z, tp.weight_numel, seed=13)
    out = tp(x1.to(DEV), x2.to(DEV), w.to(DEV))
    ref = otp.tp_forward(oracle_spec(tp), x1.numpy(), x2.numpy(), w.numpy())
    # |out| reaches ~50 for these un-normalised random inputs: the relative term matters
    assert_close(out, ref, atol=1e-4, rtol=1e-5, what=str(tp))


def test_bf16_storage_variant():
    tp = ks.cfg3(True)
    Z = 500
    x1, x2, w = seeded(Z, 288, seed=1), seeded(Z, 9, seed=2), seeded(Z, 352, seed=3)
    xb, yb, wb = (t.to(DEV).to(torch.bfloat16) for t in (x1, x2, w))
    out = tp(xb, yb, wb)
    assert out.dtype == torch.bfloat16
    # oracle on the bf16-rounded inputs; the output is rounded to bf16 once
    ref = otp.tp_forward(oracle_spec(tp), xb.float().cpu().numpy(), yb.float().cpu().numpy(), wb.float().cpu().numpy())
    assert_close(out, ref, atol=1e-2, rtol=1e-2, what="bf16 storage")


def _fan_in_weights(tp, seed=0):
    # N(0, 1/fan_in) per instruction, fan_in = U*V  (benchmark definition of the dense uvw configuration)
    g = torch.Generator().manual_seed(seed)
    w = torch.randn(tp.weight_numel, generator=g)
    off = 0
    for t in tp.instructions:
        n = t.path_shape[0] * t.path_shape[1] * t.path_shape[2]
        w[off : off + n] /= (t.path_shape[0] * t.path_shape[1]) ** 0.5
        off += n
    return w


@pytest.mark.parametrize(
    "maker,Z,family",
    [(ks.mfma_small, 150, "uvw_mfma"), (ks.cfg5, 70, "uvw_mfma"), (ks.wide_k, 130, "uvw_mfma"), (ks.outer_split, 200, "uvw_mfma"),
     # every multiplicity a multiple of 64: the matrix steps on split operands (also on restaged K blocks)
     (ks.mfma_full_tiles, 150, "uvw_mfma"), (ks.wide_k_full_tiles, 130, "uvw_mfma"),
     # an l = 3 output: seven accumulator tiles per wave, two waves per SIMD
     (ks.mfma_l3_out, 210, "uvw_mfma"),
     # scalar second input: the node-wise kernel; batches that end inside a wave's 64 rows, inside a workgroup's 256
     # rows, and below one wave
     (ks.node_fctp, 333, "uvw_node"), (ks.node_fctp, 17, "uvw_node"), (ks.node_fctp, 1280, "uvw_node"),
     (ks.radial_layer, 1000, "uvw_node"), (ks.node_block, 200, "uvw_node"), (ks.node_wide_out, 77, "uvw_node"), (ks.node_narrow, 301, "uvw_node"),
     (ks.node_partial_tile, 129, "uvw_node"), (ks.node_many_species, 260, "uvw_node")],
)  # fmt: skip
def test_uvw_matrix_core_kernel_against_oracle(maker, Z, family):
    tp = maker().to(DEV)
    assert tp._plan(torch.float32).family == family
    w = _fan_in_weights(tp)
    with torch.no_grad():
        tp.weight.copy_(w)
    x1, x2 = seeded(Z, tp.irreps_in1.dim, seed=21), seeded(Z, tp.irreps_in2.dim, seed=22)
    out = tp(x1.to(DEV), x2.to(DEV))
    ref = otp.tp_forward(oracle_spec(tp), x1.numpy(), x2.numpy(), w.numpy())
    assert_close(out, ref, what=str(tp))


@pytest.mark.parametrize("maker,Z", [(ks.node_fctp, 333), (ks.node_fctp, 1), (ks.node_wide_out, 130), (ks.node_narrow, 301), (ks.node_partial_tile, 257),
                                     (ks.node_many_species, 140)])  # fmt: skip
def test_node_wise_kernel_in_bf16_storage_against_oracle(maker, Z):
    # rows, scalars and weights stored as bf16 (8-byte pieces; weight rows element by element where the channel
    # counts are no multiples of 4), fp32 matrix instructions on the converted values, one rounding of the output
    tp = maker().to(DEV)
    w = _fan_in_weights(tp)
    tpb = maker().to(DEV).to(torch.bfloat16)
    assert tpb._plan(torch.bfloat16).family == "uvw_node"
    with torch.no_grad():
        tpb.weight.copy_(w.to(torch.bfloat16))
    xb = seeded(Z, tp.irreps_in1.dim, seed=41).to(DEV).to(torch.bfloat16)
    yb = seeded(Z, tp.irreps_in2.dim, seed=42).to(DEV).to(torch.bfloat16)
    out = tpb(xb, yb)
    assert out.dtype == torch.bfloat16 and out.shape == (Z, tp.irreps_out.dim)
    ref = otp.tp_forward(oracle_spec(tp), xb.float().cpu().numpy(), yb.float().cpu().numpy(), tpb.weight.detach().float().cpu().numpy())
    scale = float(np.abs(ref).max())
    # bf16 rounds to nearest with 8 significant bits: at most 2^-8 relative; the absolute term covers elements near zero
    assert_close(out, ref, atol=2.0**-9 * scale, rtol=2.0**-8, what=f"bf16 node-wise {tp}")


def test_uvw_full_size_dense_configuration():
    # FCTP(128x0e+128x1o+128x2e x same -> same), batch 65536, weights N(0, 1/fan_in), inputs N(0, 1)
    tp = ks.cfg5().to(DEV)
    w = _fan_in_weights(tp)
    with torch.no_grad():
        tp.weight.copy_(w)
    Z = 65536
    g = torch.Generator(device=DEV).manual_seed(0)
    x1 = torch.randn(Z, 1152, device=DEV, generator=g)
    x2 = torch.randn(Z, 1152, device=DEV, generator=g)
    out = tp(x1, x2)
    # rows are independent: the oracle on a few rows from both ends and the middle
    rows = torch.tensor([0, 1, 63, 64, 32767, 32768, 65471, 65535])
    ref = otp.tp_forward(oracle_spec(tp), x1[rows].cpu().numpy(), x2[rows].cpu().numpy(), w.numpy())
    assert_close(out[rows], ref, what="cfg5 rows")
    # size-independent properties: bilinearity in (x1, x2), output scale
    out2 = tp(2.0 * x1, -0.5 * x2)
    # powers of two commute with every rounding, so scaling alone is exact; the sign is not: the matrix passes run on
    # bf16 matrix instructions (three-way split operands), whose internal sums are not symmetric under negation
    assert torch.equal(tp(2.0 * x1, 0.5 * x2), out)
    assert float((out2 + out).detach().abs().max()) <= 1e-5 * float(out.detach().abs().max())  # measured 3.4e-6: the size of the rounding errors
    # weights N(0, 1/fan_in) on top of the path normalisation 1/sqrt(fan_in * paths): variance 1/fan_in
    assert abs(out.var().item() * 16384 - 1.0) < 0.1
    # batch slices give the same rows
    assert torch.equal(tp(x1[1000:1100], x2[1000:1100]), out[1000:1100])


@pytest.mark.parametrize("maker", [ks.mfma_full_tiles, ks.cfg5, ks.node_block])
def test_split_operand_kernels_over_the_exponent_range_and_on_non_finite_rows(maker):
    # the fp32 plans of these sets form each product from three bf16 pieces per operand.  (i) The pieces keep the
    # exponent range of fp32: rows scaled by 1e-30 ... 1e30 come out with fp32 accuracy relative to their own scale.
    # (ii) A row holding inf or NaN comes out non-finite and leaves every other row untouched, bit for bit.  Where the
    # reference's einsum gives +-inf for such a row (all products of one sign) these kernels give NaN: the piece
    # h = bf16(inf) is inf and the next piece is inf - inf; finite |x| above 3.39e38, which round to inf in bf16, behave
    # the same way.  A sum of products of an inf with factors of both signs is NaN in the reference as well.
    tp = maker().to(DEV)
    w = _fan_in_weights(tp)
    with torch.no_grad():
        tp.weight.copy_(w)
    Z = 70
    x1, x2 = seeded(Z, tp.irreps_in1.dim, seed=31), seeded(Z, tp.irreps_in2.dim, seed=32)
    scales = torch.tensor([1e-30, 1e-15, 1.0, 1e15, 1e30]).repeat(Z // 5)[:, None]
    out = tp((x1 * scales).to(DEV), x2.to(DEV))
    ref = otp.tp_forward(oracle_spec(tp), x1.numpy(), x2.numpy(), w.numpy())
    rel = out.cpu().double() / scales.double()
    assert_close(rel, ref, what=f"{maker.__name__}: rows scaled by 1e-30 ... 1e30, relative to their scale")
    clean = tp(x1.to(DEV), x2.to(DEV))
    bad = x1.clone()
    bad[3, 0], bad[40, 5] = float("inf"), float("nan")
    got = tp(bad.to(DEV), x2.to(DEV))
    keep = torch.ones(Z, dtype=torch.bool)
    keep[[3, 40]] = False
    assert torch.equal(got[keep], clean[keep])
    assert not torch.isfinite(got[3]).all() and not torch.isfinite(got[40]).all()


def _uvw_weight_gradient_fp64(tp, x1, x2, cot):
    """d/dW of sum(cot * tp(x1, x2, W)) for shared uvw weights, written out from the definition
    out[z, w, k] = pw sum_uv W[u, v, w] sum_ij C[i, j, k] x1[z, u, i] x2[z, v, j]:
    gW[u, v, w] = pw sum_ij (x1_i (x) x2_j)^T [z, (u, v)] @ (sum_k C[i, j, k] cot[z, w, k]), one GEMM per (i, j)."""
    from oracle.wigner import wigner_3j

    s1, s2, so = tp.irreps_in1.slices(), tp.irreps_in2.slices(), tp.irreps_out.slices()
    Z, blocks = x1.shape[0], []
    for t in tp.instructions:
        (U, ir1), (V, ir2), (W, iro) = tp.irreps_in1[t.i_in1], tp.irreps_in2[t.i_in2], tp.irreps_out[t.i_out]
        a, b, g = x1[:, s1[t.i_in1]].reshape(Z, U, -1), x2[:, s2[t.i_in2]].reshape(Z, V, -1), cot[:, so[t.i_out]].reshape(Z, W, -1)
        C = wigner_3j(ir1.l, ir2.l, iro.l)
        gw = np.zeros((U * V, W))
        for i in range(ir1.dim):
            for j in range(ir2.dim):
                if np.any(C[i, j]):
                    gw += (a[:, :, None, i] * b[:, None, :, j]).reshape(Z, U * V).T @ (g @ C[i, j])
        blocks.append(t.path_weight * gw.reshape(-1))
    return np.concatenate(blocks)


def test_uvw_weight_gradient_on_the_dense_configuration():
    # the weight gradient of config 5's own instruction set (11 paths of 128 x 128 x 128, 23 M weights) on the
    # split-operand matrix-core kernel; 300 rows end inside a batch chunk of the kernel.  The float64 reference is the
    # definition written out (one GEMM per pair of input components), itself checked here against autograd of the
    # einsum restatement on a small set
    from oracle.torch_cpu import tp_forward_torch

    small = ks.mfma_small()
    x1, x2, cot = (seeded(9, d, seed=s).double() for d, s in ((small.irreps_in1.dim, 1), (small.irreps_in2.dim, 2), (small.irreps_out.dim, 3)))
    wd = seeded(small.weight_numel, seed=4).double().requires_grad_()
    (auto,) = torch.autograd.grad(tp_forward_torch(oracle_spec(small), x1, x2, wd), wd, cot)
    assert np.abs(_uvw_weight_gradient_fp64(small, x1.numpy(), x2.numpy(), cot.numpy()) - auto.numpy()).max() < 1e-12

    tp = ks.cfg5().to(DEV)
    Z = 300
    x1, x2, cot = seeded(Z, 1152, seed=41), seeded(Z, 1152, seed=42), seeded(Z, 1152, seed=43)
    wg = _fan_in_weights(tp).to(DEV).requires_grad_()
    (got,) = torch.autograd.grad(tp(x1.to(DEV), x2.to(DEV), wg), wg, cot.to(DEV))
    ref = _uvw_weight_gradient_fp64(tp, x1.double().numpy(), x2.double().numpy(), cot.double().numpy())
    # a sum over the batch: tolerance scaled by its size
    assert_close(got, ref, atol=1e-4 * max(1.0, float(np.abs(ref).max())), what="cfg5 weight gradient, 300 rows")


def _bf16_uvw(seed_w=0, make=ks.cfg5):
    tp = make().to(DEV)
    w = _fan_in_weights(tp, seed=seed_w)
    tpb = make().to(DEV).to(torch.bfloat16)
    with torch.no_grad():
        tpb.weight.copy_(w.to(torch.bfloat16))
    return tp, tpb, tpb.weight.detach().float().cpu().numpy()


def _oracle_chunks(spec, x1, x2, w, chunk=48):
    return np.concatenate([otp.tp_forward(spec, x1[b : b + chunk], x2[b : b + chunk], w) for b in range(0, x1.shape[0], chunk)])


def test_uvw_bf16_storage():
    # two full 128-row workgroup tiles and a ragged tail of 77 rows; outputs have standard deviation 1/128, so the
    # tolerance is tied to the output scale: atol = 1e-2 max|ref| (a dropped path of the 11 shifts outputs by ~0.5 sigma,
    # ten times this), rtol 1e-2 for the single bf16 rounding of the output
    tp, tpb, wq = _bf16_uvw()
    Z = 333
    x1, x2 = seeded(Z, 1152, seed=31), seeded(Z, 1152, seed=32)
    xb, yb = x1.to(DEV).to(torch.bfloat16), x2.to(DEV).to(torch.bfloat16)
    out = tpb(xb, yb)
    assert out.dtype == torch.bfloat16
    ref = _oracle_chunks(oracle_spec(tp), xb.float().cpu().numpy(), yb.float().cpu().numpy(), wq)
    scale = float(np.abs(ref).max())
    assert 0.02 < scale < 0.08
    assert_close(out, ref, atol=1e-2 * scale, rtol=1e-2, what="bf16 uvw, Z = 333")
    # every path matters at this tolerance: the oracle without the last instruction fails it
    spec = oracle_spec(tp)
    short = otp.make_spec(str(tp.irreps_in1), str(tp.irreps_in2), str(tp.irreps_out),
                          [(t.i_in1, t.i_in2, t.i_out, t.connection_mode, t.has_weight, 0.0 if n == 10 else 1.0) for n, t in enumerate(tp.instructions)],
                          shared_weights=True)  # fmt: skip
    assert len(spec.instructions) == 11
    miss = _oracle_chunks(short, xb[:48].float().cpu().numpy(), yb[:48].float().cpu().numpy(), wq)
    assert (np.abs(out[:48].detach().float().cpu().numpy() - miss) > 1e-2 * scale + 1e-2 * np.abs(miss)).any()


def test_uvw_bf16_storage_full_size():
    # batch 65536: rows from both ends, tile boundaries and the middle against the oracle; slices give the same rows
    tp, tpb, wq = _bf16_uvw()
    Z = 65536
    g = torch.Generator(device=DEV).manual_seed(0)
    xb = torch.randn(Z, 1152, device=DEV, generator=g).to(torch.bfloat16)
    yb = torch.randn(Z, 1152, device=DEV, generator=g).to(torch.bfloat16)
    out = tpb(xb, yb)
    rows = torch.tensor([0, 127, 128, 32767, 32768, 40001, 65408, 65535])
    ref = otp.tp_forward(oracle_spec(tp), xb[rows].float().cpu().numpy(), yb[rows].float().cpu().numpy(), wq)
    scale = float(np.abs(ref).max())
    assert_close(out[rows], ref, atol=1e-2 * scale, rtol=1e-2, what="bf16 uvw, 8 rows of Z = 65536")
    # a batch slice gives the same rows up to the accumulation order (workgroups start at different outer-index
    # blocks depending on their position in the grid): within one bf16 rounding step of the output
    part = tpb(xb[4096 : 4096 + 256], yb[4096 : 4096 + 256]).float()
    assert (part - out[4096 : 4096 + 256].float()).abs().max().item() <= 2.0**-7 * scale
    assert abs(out.float().var().item() * 16384 - 1.0) < 0.1


@pytest.mark.parametrize("Z", [8192 + 1, 16384 + 130, 16384 + 256 + 127])
def test_uvw_bf16_storage_ragged_batches_in_256_row_workgroups(Z):
    # from 8192 rows on the 0e and 1o outputs are computed by workgroups of 256 rows (two row tiles per wavefront);
    # the last workgroup here holds 1 row, a full first tile and 2 rows of the second, or a full first tile less one row
    tp, tpb, wq = _bf16_uvw()
    g = torch.Generator(device=DEV).manual_seed(Z)
    xb = torch.randn(Z, 1152, device=DEV, generator=g).to(torch.bfloat16)
    yb = torch.randn(Z, 1152, device=DEV, generator=g).to(torch.bfloat16)
    out = tpb(xb, yb)
    assert out.shape == (Z, 1152) and torch.isfinite(out.float()).all()
    rows = torch.cat([torch.tensor([0, 127, 128, 255, 256, 8191]), torch.arange(Z - 140, Z)])
    ref = _oracle_chunks(oracle_spec(tp), xb[rows].float().cpu().numpy(), yb[rows].float().cpu().numpy(), wq)
    scale = float(np.abs(ref).max())
    assert_close(out[rows], ref, atol=1e-2 * scale, rtol=1e-2, what=f"bf16 uvw, Z = {Z}")
    # the same rows as a batch below the switch (workgroups of 128 rows): equal up to the accumulation order
    part = tpb(xb[-400:], yb[-400:]).float()
    assert (part - out[-400:].float()).abs().max().item() <= 2.0**-7 * scale


def test_uvw_bf16_storage_small_multiplicities_in_256_row_workgroups():
    # multiplicities 32 and 64 (fewer weight chunks per stage than wavefronts, two and four matrix steps per outer
    # index), four output irreps of which 0e, 1o and 1e take the 256-row workgroups; ragged last workgroup
    tp, tpb, wq = _bf16_uvw(make=ks.mfma_small)
    Z = 16384 + 128 + 77
    g = torch.Generator(device=DEV).manual_seed(3)
    xb = torch.randn(Z, tp.irreps_in1.dim, device=DEV, generator=g).to(torch.bfloat16)
    yb = torch.randn(Z, tp.irreps_in2.dim, device=DEV, generator=g).to(torch.bfloat16)
    out = tpb(xb, yb)
    rows = torch.cat([torch.arange(0, 16384, 333), torch.arange(16384 - 2, Z)])
    ref = _oracle_chunks(oracle_spec(tp), xb[rows].float().cpu().numpy(), yb[rows].float().cpu().numpy(), wq, chunk=512)
    scale = float(np.abs(ref).max())
    assert_close(out[rows], ref, atol=1e-2 * scale, rtol=1e-2, what="bf16 uvw, small multiplicities")
    part = tpb(xb[-300:], yb[-300:]).float()
    assert (part - out[-300:].float()).abs().max().item() <= 2.0**-7 * scale


@pytest.mark.parametrize("Z", [300, 16384 + 77])
def test_uvw_bf16_storage_tiles_of_32_channels(Z):
    # irreps of 32 and 96 channels: their last workgroup tile holds 32 channels instead of 64 (both row tilings)
    tp, tpb, wq = _bf16_uvw(make=ks.mfma_half_tiles)
    assert tpb._plan(torch.bfloat16).family == "uvw_mfma"
    g = torch.Generator(device=DEV).manual_seed(Z)
    xb = torch.randn(Z, tp.irreps_in1.dim, device=DEV, generator=g).to(torch.bfloat16)
    yb = torch.randn(Z, tp.irreps_in2.dim, device=DEV, generator=g).to(torch.bfloat16)
    out = tpb(xb, yb)
    assert torch.isfinite(out.float()).all()
    rows = torch.cat([torch.arange(0, min(Z, 16384), 97), torch.arange(max(0, Z - 200), Z)])
    ref = _oracle_chunks(oracle_spec(tp), xb[rows].float().cpu().numpy(), yb[rows].float().cpu().numpy(), wq, chunk=512)
    scale = float(np.abs(ref).max())
    assert_close(out[rows], ref, atol=1e-2 * scale, rtol=1e-2, what=f"bf16 uvw, 32-channel tiles, Z = {Z}")


def test_provider_binding_runs_the_same_kernels():
    # modules built by the provider from (Irreps, Instruction) data give the product's own results, with e3nn's
    # broadcasting of leading dimensions -- also after the pickle round trip e3nn puts its generated modules through
    import pickle

    from e3nn_amd import provider

    for tp, shared in ((ks.cfg1().to(DEV), True), (ks.cfg3(True), False)):
        gm = provider.hip_provider(tp.irreps_in1, tp.irreps_in2, tp.irreps_out, tp.instructions, shared, True, True)
        x1 = seeded(5, 1, tp.irreps_in1.dim, seed=1).to(DEV)
        x2 = seeded(1, 3, tp.irreps_in2.dim, seed=2).to(DEV)
        w = tp.weight.detach() if shared else seeded(5, 3, tp.weight_numel, seed=3).to(DEV)
        ref = tp(x1, x2) if shared else tp(x1, x2, w)
        for mod in (gm, pickle.loads(pickle.dumps(gm))):
            got = mod(x1, x2, w)
            assert got.shape == (5, 3, tp.irreps_out.dim) and torch.equal(got, ref)
        with pytest.raises(RuntimeError, match="share one dtype"):
            gm(x1, x2.bfloat16(), w)
        with pytest.raises(RuntimeError, match="float32 or bfloat16"):
            gm(x1.double(), x2.double(), w.double())


def test_provider_binding_is_differentiable():
    # a reference TensorProduct served by the provider must train: gradients of all three arguments through
    # gm(x1, x2, w) are the package TensorProduct's own (config 1: shared uvw weights; config 3: per-sample uvu
    # weights), and both agree with float64 autograd of the einsum restatement
    from e3nn_amd import provider
    from oracle.torch_cpu import tp_forward_torch

    for tp, shared in ((ks.cfg1().to(DEV), True), (ks.cfg3(True), False)):
        gm = provider.hip_provider(tp.irreps_in1, tp.irreps_in2, tp.irreps_out, tp.instructions, shared, True, True)
        x1 = seeded(40, tp.irreps_in1.dim, seed=1)
        x2 = seeded(40, tp.irreps_in2.dim, seed=2)
        w = seeded(*((tp.weight_numel,) if shared else (40, tp.weight_numel)), seed=3)
        cot = seeded(40, tp.irreps_out.dim, seed=4)
        grads = []
        for f in (gm, tp):
            args = [t.to(DEV).requires_grad_() for t in (x1, x2, w)]
            out = f(*args)
            assert out.grad_fn is not None
            grads.append(torch.autograd.grad(out, args, cot.to(DEV)))
        for got, ref, name in zip(grads[0], grads[1], ("x1", "x2", "w")):
            if shared and name == "w":  # batch slices meet in fp32 atomics: last-bit differences between two runs
                assert (got - ref).abs().max().item() <= 1e-5 * ref.abs().max().item(), name
            else:
                assert torch.equal(got, ref), name
        spec = oracle_spec(tp)
        a, b, c = (t.double().requires_grad_() for t in (x1, x2, w))
        oracle_grads = torch.autograd.grad(tp_forward_torch(spec, a, b, c), (a, b, c), cot.double())
        for got, ref, name in zip(grads[0], oracle_grads, ("x1", "x2", "w")):
            atol = 1e-4 * max(1.0, float(ref.abs().max())) if shared and name == "w" else 1e-4  # batch sum / contraction
            assert_close(got, ref.numpy(), atol=atol, what=f"provider, d/d{name}")


def test_provider_right_binding():
    from e3nn_amd import provider

    tp = ks.right_small().to(DEV)
    gm = provider.hip_provider_right(tp.irreps_in1, tp.irreps_in2, tp.irreps_out, tp.instructions, True, True, True)
    x1 = seeded(6, tp.irreps_in1.dim, seed=1).to(DEV)
    x2 = seeded(6, tp.irreps_in2.dim, seed=2).to(DEV)
    mats = gm(x2, tp.weight.detach())
    assert mats.shape == (6, tp.irreps_in1.dim, tp.irreps_out.dim) and torch.equal(mats, tp.right(x2))
    ref = otp.tp_forward(oracle_spec(tp), x1.cpu().numpy(), x2.cpu().numpy(), tp.weight.detach().cpu().numpy())
    assert_close(torch.einsum("zi,zik->zk", x1, mats), ref, what="x @ right(y) through the provider")
