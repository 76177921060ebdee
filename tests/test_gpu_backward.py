"""GPU parity of the backward pass: gradients from the HIP kernels against torch autograd (float64) through the
CPU restatement of the reference's einsum graph (oracle/torch_cpu.py)."""
import numpy as np
import pytest
import torch

from e3nn_amd.nn import DstSortedEdges
from oracle.torch_cpu import tp_forward_torch, tp_gather_scatter_torch
from tests import kernel_sets as ks
from tests.helpers import assert_close, oracle_spec, seeded

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _oracle_grads(fn, tensors, cot):
    ts = [t.double().clone().requires_grad_(True) for t in tensors]
    out = fn(*ts)
    out.backward(cot.double())
    return out.detach(), [t.grad for t in ts]


@pytest.mark.parametrize("maker,Z", [
    (lambda: ks.golden_tp("uvu_merged_cfg3_like_mul4"), 9), (lambda: ks.golden_tp("uvu_builderA_cfg4_like_mul2"), 7),
    (lambda: ks.cfg3(True), 130), (lambda: ks.cfg3(False), 65), (lambda: ks.cfg4("A"), 17), (ks.odd_mul, 33),
])  # fmt: skip
def test_uvu_plain_gradients(maker, Z):
    tp = maker()
    spec = oracle_spec(tp)
    x1, x2, w = seeded(Z, tp.irreps_in1.dim, seed=1), seeded(Z, tp.irreps_in2.dim, seed=2), seeded(Z, tp.weight_numel, seed=3)
    cot = seeded(Z, tp.irreps_out.dim, seed=4)
    ref_out, (r1, r2, rw) = _oracle_grads(lambda a, b, c: tp_forward_torch(spec, a, b, c), (x1, x2, w), cot)
    a, b, c = (t.to(DEV).requires_grad_(True) for t in (x1, x2, w))
    out = tp(a, b, c)
    # the weight gradient is written without a zero fill: hand the allocator a NaN-filled block of its size first,
    # so that an element the kernel skipped would show
    junk = torch.full((Z, tp.weight_numel), float("nan"), device=DEV)
    del junk
    out.backward(cot.to(DEV))
    # per-sample contractions: the benchmark's tolerance for contractions, |err| <= 1e-4 + 1e-5 |ref|
    assert_close(out, ref_out.numpy())
    assert_close(a.grad, r1.numpy(), what="d/dx1")
    assert_close(b.grad, r2.numpy(), what="d/dx2")
    assert_close(c.grad, rw.numpy(), what="d/dw")


@pytest.mark.parametrize("maker,N,E,idx", [(lambda: ks.cfg3(True), 120, 3000, torch.int64), (lambda: ks.cfg3(False), 50, 900, torch.int32),
                                           (lambda: ks.cfg4("A"), 25, 300, torch.int32),
                                           # multiplicities that leave lane groups partly filled (80, 24, 5): every
                                           # weight-gradient column must still be written (the buffer is not zero-filled)
                                           (ks.odd_mul, 40, 600, torch.int32), (ks.narrow_message, 60, 900, torch.int64)])  # fmt: skip
def test_fused_message_gradients(maker, N, E, idx):
    tp = maker()
    spec = oracle_spec(tp)
    g = torch.Generator().manual_seed(7)
    src, dst = torch.randint(0, N, (E,), generator=g), torch.randint(0, N - 2, (E,), generator=g)
    node_x, attr, w = seeded(N, tp.irreps_in1.dim, seed=1), seeded(E, tp.irreps_in2.dim, seed=2), seeded(E, tp.weight_numel, seed=3)
    cot = seeded(N, tp.irreps_out.dim, seed=4)
    ref_out, (r1, r2, rw) = _oracle_grads(lambda a, b, c: tp_gather_scatter_torch(spec, a, b, c, src, dst, N), (node_x, attr, w), cot)
    a, b, c = (t.to(DEV).requires_grad_(True) for t in (node_x, attr, w))
    edges = DstSortedEdges(src.to(idx).to(DEV), dst.to(idx).to(DEV), N)
    out = tp.forward_gather_scatter(a, b, c, edges=edges)
    junk = torch.full((E, tp.weight_numel), float("nan"), device=DEV)  # see test_uvu_plain_gradients
    del junk
    out.backward(cot.to(DEV))
    scale = lambda r: max(1.0, float(r.abs().max()))  # noqa: E731
    assert_close(out, ref_out.numpy(), atol=1e-4 * scale(ref_out))
    assert_close(a.grad, r1.numpy(), atol=1e-4 * scale(r1), what="d/dnode_x")
    # sums over the edges of a node are held to a tolerance scaled by their size (the order of summation differs
    # from scatter_add_), per-edge contractions to the benchmark's 1e-4 + 1e-5 |ref|
    assert_close(b.grad, r2.numpy(), what="d/dedge_attr")
    assert_close(c.grad, rw.numpy(), what="d/dweight")
    # only some inputs require a gradient
    a2, c2 = node_x.to(DEV).requires_grad_(True), w.to(DEV)
    tp.forward_gather_scatter(a2, attr.to(DEV), c2, edges=edges).backward(cot.to(DEV))
    # (another kernel than above where one kernel writes every gradient: the lane groups of a wavefront are combined
    # in another order, so the last bits may differ)
    assert_close(a2.grad, a.grad.cpu().numpy(), atol=1e-5 * scale(r1), what="d/dnode_x alone")
    # node features and weights but not the edge attributes (training without forces): one kernel on the transposed
    # plan writes both gradients where the instruction set fits it (a lane group owning a whole row)
    a4, c4 = node_x.to(DEV).requires_grad_(True), w.to(DEV).requires_grad_(True)
    tp.forward_gather_scatter(a4, attr.to(DEV), c4, edges=edges).backward(cot.to(DEV))
    assert_close(a4.grad, r1.numpy(), atol=1e-4 * scale(r1), what="d/dnode_x, one backward kernel")
    assert_close(c4.grad, rw.numpy(), what="d/dweight, one backward kernel")
    # negative source indices wrap in the gather; the gradient scatters onto the wrapped rows
    neg = torch.where(torch.arange(E) % 3 == 0, src - N, src)
    a3 = node_x.to(DEV).requires_grad_(True)
    tp.forward_gather_scatter(a3, attr.to(DEV), c2, edges=DstSortedEdges(neg.to(idx).to(DEV), dst.to(idx).to(DEV), N)).backward(cot.to(DEV))
    assert torch.equal(a3.grad, a2.grad)
    a5, c5 = node_x.to(DEV).requires_grad_(True), w.to(DEV).requires_grad_(True)
    tp.forward_gather_scatter(a5, attr.to(DEV), c5, edges=DstSortedEdges(neg.to(idx).to(DEV), dst.to(idx).to(DEV), N)).backward(cot.to(DEV))
    assert torch.equal(a5.grad, a4.grad) and torch.equal(c5.grad, c4.grad)


@pytest.mark.parametrize("maker,Z", [(lambda: ks.golden_tp("fctp_small_cfg5_like"), 6), (ks.cfg1, 50), (ks.mfma_small, 70),
                                     (lambda: ks.golden_tp("fctp_per_sample_weights"), 5), (ks.node_fctp, 90), (ks.radial_layer, 77), (ks.node_wide_out, 45), (ks.node_narrow, 40)])  # fmt: skip
def test_uvw_input_gradients(maker, Z):
    tp = maker().to(DEV)
    spec = oracle_spec(tp)
    x1, x2 = seeded(Z, tp.irreps_in1.dim, seed=1), seeded(Z, tp.irreps_in2.dim, seed=2)
    w = seeded(*((Z,) if not tp.shared_weights else ()), tp.weight_numel, seed=3) / 4
    cot = seeded(Z, tp.irreps_out.dim, seed=4)
    ref_out, (r1, r2) = _oracle_grads(lambda a, b: tp_forward_torch(spec, a, b, w.double()), (x1, x2), cot)
    a, b = (t.to(DEV).requires_grad_(True) for t in (x1, x2))
    out = tp(a, b, w.to(DEV))
    out.backward(cot.to(DEV))
    assert_close(out, ref_out.numpy())
    assert_close(a.grad, r1.numpy(), what="d/dx1")
    assert_close(b.grad, r2.numpy(), what="d/dx2")


@pytest.mark.parametrize("maker,Z", [(lambda: ks.golden_tp("fctp_small_cfg5_like"), 6), (ks.cfg1, 50), (ks.cfg1, 4099),
                                     (lambda: ks.golden_tp("fctp_per_sample_weights"), 5), (ks.mfma_small, 70),
                                     (ks.mfma_small, 1500), (ks.mfma_full_tiles, 70), (ks.mfma_full_tiles, 1237), (ks.node_fctp, 700), (ks.node_block, 333), (ks.node_block, 20), (ks.outer_split, 410), (ks.radial_layer, 513), (ks.node_wide_out, 300), (ks.node_narrow, 260),
                                     (ks.node_partial_tile, 100), (ks.unaligned_mfma, 300), (ks.unaligned_offsets, 129)])  # fmt: skip
def test_uvw_weight_gradients(maker, Z):
    tp = maker().to(DEV)
    spec = oracle_spec(tp)
    x1, x2 = seeded(Z, tp.irreps_in1.dim, seed=1), seeded(Z, tp.irreps_in2.dim, seed=2)
    w = seeded(*((Z,) if not tp.shared_weights else ()), tp.weight_numel, seed=3) / 4
    cot = seeded(Z, tp.irreps_out.dim, seed=4)
    _, (r1, r2, rw) = _oracle_grads(lambda a, b, c: tp_forward_torch(spec, a, b, c), (x1, x2, w), cot)
    a, b, c = (t.to(DEV).requires_grad_(True) for t in (x1, x2, w))
    tp(a, b, c).backward(cot.to(DEV))
    # shared weights: the gradient is a sum over the batch, held to a tolerance scaled by its size; everything else
    # is a per-sample contraction (1e-4 + 1e-5 |ref|)
    w_atol = 1e-4 * max(1.0, float(rw.abs().max())) if tp.shared_weights else 1e-4
    assert_close(c.grad, rw.numpy(), atol=w_atol, what="d/dw")
    assert_close(a.grad, r1.numpy(), what="d/dx1")
    assert_close(b.grad, r2.numpy(), what="d/dx2")
    # the weights alone
    c2 = w.to(DEV).requires_grad_(True)
    tp(x1.to(DEV), x2.to(DEV), c2).backward(cot.to(DEV))
    assert_close(c2.grad, rw.numpy(), atol=w_atol, what="d/dw alone")


def test_internal_weights_train():
    tp = ks.cfg1().to(DEV)
    x1, x2 = seeded(40, 64).to(DEV), seeded(40, 9).to(DEV)
    tp(x1, x2).square().sum().backward()
    assert tp.weight.grad is not None and tp.weight.grad.shape == tp.weight.shape and bool(tp.weight.grad.abs().sum() > 0)


def test_shared_uvu_weight_gradient():
    tp = ks.golden_tp("uvu_shared_v2").to(DEV)
    assert tp.shared_weights and tp.weight_numel
    spec = oracle_spec(tp)
    Z = 300
    x1, x2, w = seeded(Z, tp.irreps_in1.dim, seed=1), seeded(Z, tp.irreps_in2.dim, seed=2), seeded(tp.weight_numel, seed=3)
    cot = seeded(Z, tp.irreps_out.dim, seed=4)
    _, (r1, r2, rw) = _oracle_grads(lambda a, b, c: tp_forward_torch(spec, a, b, c), (x1, x2, w), cot)
    a, b, c = (t.to(DEV).requires_grad_(True) for t in (x1, x2, w))
    tp(a, b, c).backward(cot.to(DEV))
    assert_close(c.grad, rw.numpy(), atol=1e-4 * max(1.0, float(rw.abs().max())), what="d/dw (shared, summed over the batch)")
    assert_close(a.grad, r1.numpy(), what="d/dx1")
    assert_close(b.grad, r2.numpy(), what="d/dx2")


@pytest.mark.parametrize("maker", [ks.mixed_modes, lambda: ks.golden_tp("modes_uuu_uvuv_uuw_uvv"), lambda: ks.golden_tp("modes_triangular")])
def test_general_mode_gradients(maker):
    """Connection modes outside pure uvu / pure uvw are differentiated through the equivalent uvw product with structured
    weights.  The map is trilinear, so central differences of the float64 oracle along a direction are exact."""
    from oracle import tensor_product as otp

    tp = maker().to(DEV)
    assert tp._live_mode() == "general"
    spec = oracle_spec(tp)
    Z = 37
    wshape = (tp.weight_numel,) if tp.shared_weights else (Z, tp.weight_numel)
    x1, x2, w = seeded(Z, tp.irreps_in1.dim, seed=1), seeded(Z, tp.irreps_in2.dim, seed=2), seeded(*wshape, seed=3)
    cot = seeded(Z, tp.irreps_out.dim, seed=4)
    a, b, c = (t.to(DEV).requires_grad_(True) for t in (x1, x2, w))
    out = tp(a, b, c)
    f = lambda p, q, r: otp.tp_forward(spec, p, q, r if tp.weight_numel else None)  # noqa: E731
    n1, n2, nw = (t.numpy().astype(np.float64) for t in (x1, x2, w))
    assert_close(out, f(n1, n2, nw), what="forward through the dense equivalent")
    with torch.no_grad():
        assert_close(tp(a, b, c), f(n1, n2, nw), what="forward, mode-specific kernel")
    out.backward(cot.to(DEV))
    rng = np.random.default_rng(5)
    c64 = cot.numpy().astype(np.float64)
    for got, which in ((a.grad, 0), (b.grad, 1), (c.grad, 2)):
        if which == 2 and not tp.weight_numel:
            continue
        for _ in range(3):
            args = [n1, n2, nw]
            v = rng.normal(size=args[which].shape)
            plus, minus = list(args), list(args)
            plus[which], minus[which] = args[which] + v, args[which] - v
            want = ((f(*plus) - f(*minus)) * c64).sum() / 2
            assert float((got.cpu().double().numpy() * v).sum()) == pytest.approx(want, rel=2e-4, abs=1e-3)


@pytest.mark.parametrize("maker", [lambda **kw: ks.golden_tp("fctp_small_cfg5_like", **kw), lambda **kw: ks.golden_tp("uvu_merged_cfg3_like_mul4", **kw), ks.mixed_modes])
def test_right(maker):
    """right(y, w) is the matrix with forward(x, y, w) == x @ right(y, w) (the reference's own test of right(),
    tests/o3/tensor_product_test.py, checks this identity); the forward side is the oracle's."""
    from oracle import tensor_product as otp

    with pytest.raises(AssertionError):  # as in the reference, right() is there only when asked for at construction
        maker().right(seeded(1, maker().irreps_in2.dim).to(DEV))
    tp = maker(compile_right=True).to(DEV)
    spec = oracle_spec(tp)
    Z = 5
    wshape = (tp.weight_numel,) if tp.shared_weights else (Z, tp.weight_numel)
    x1, x2, w = seeded(Z, tp.irreps_in1.dim, seed=1), seeded(Z, tp.irreps_in2.dim, seed=2), seeded(*wshape, seed=3)
    with torch.no_grad():
        r = tp.right(x2.to(DEV), w.to(DEV) if tp.weight_numel else None)
    assert r.shape == (Z, tp.irreps_in1.dim, tp.irreps_out.dim)
    got = torch.einsum("zik,zi->zk", r.cpu().double(), x1.double())
    want = otp.tp_forward(spec, *(t.numpy().astype(np.float64) for t in (x1, x2)), w.numpy().astype(np.float64) if tp.weight_numel else None)
    assert_close(got, want, what="x @ right(y, w)")
    # rows of the operator that belong to an input irrep no instruction reads are zero
    assert torch.isfinite(r).all()


@pytest.mark.parametrize("lmax", [1, 2, 3])
@pytest.mark.parametrize("normalize,normalization", [(True, "component"), (False, "integral"), (True, "norm")])
def test_spherical_harmonics_gradient(lmax, normalize, normalization):
    from e3nn_amd import o3
    from oracle.torch_cpu import spherical_harmonics_torch
    import math

    x = seeded(301, 3, seed=lmax)
    cot = seeded(301, (lmax + 1) ** 2, seed=9)

    def ref_fn(v):
        y = spherical_harmonics_torch(lmax, v, normalize)
        if normalization == "integral":
            y = y / math.sqrt(4 * math.pi)
        elif normalization == "norm":
            y = y / torch.cat([math.sqrt(2 * l + 1) * torch.ones(2 * l + 1, dtype=y.dtype) for l in range(lmax + 1)])
        return y

    _, (rx,) = _oracle_grads(ref_fn, (x,), cot)
    xd = x.to(DEV).requires_grad_(True)
    o3.spherical_harmonics(list(range(lmax + 1)), xd, normalize, normalization).backward(cot.to(DEV))
    assert_close(xd.grad, rx.numpy(), atol=1e-4 * max(1.0, float(rx.abs().max())), what="d/dxyz")
    # float64 finite differences of the oracle agree with its autograd (the reference's gradcheck, test :62-80)
    eps = 1e-6
    xp = x.double().clone()
    xp[0, 1] += eps
    fd = ((ref_fn(xp) - ref_fn(x.double()))[0] * cot[0].double()).sum() / eps
    assert abs(fd - rx[0, 1]) < 1e-4 * max(1.0, abs(float(fd)))


@pytest.mark.parametrize("ls,normalize,normalization", [
    ([0, 1, 2, 3, 4, 5], True, "component"), ([6], False, "integral"), ([2, 2, 0, 7], True, "norm"), ([1, 3], False, "component"),
    (list(range(11)), True, "integral"), (list(range(13)), True, "component"), ([12, 11], False, "norm"),
])  # fmt: skip
def test_spherical_harmonics_gradient_any_l_list(ls, normalize, normalization):
    """l lists beyond 0..3 take the reverse sweep of the recurrence: against central differences of the float64 oracle
    along random directions, point by point."""
    from e3nn_amd import o3
    from oracle import spherical_harmonics as osh

    n = 203
    x = seeded(n, 3, seed=len(ls))
    n_out = sum(2 * l + 1 for l in ls)
    cot = seeded(n, n_out, seed=11)
    xd = x.to(DEV).requires_grad_(True)
    out = o3.spherical_harmonics(ls, xd, normalize, normalization)
    assert out.shape == (n, n_out)
    out.backward(cot.to(DEV))
    got = xd.grad.cpu().double().numpy()
    x64, c64 = x.numpy().astype(np.float64), cot.numpy().astype(np.float64)
    rng = np.random.default_rng(7)
    f = lambda p: osh.spherical_harmonics(ls, p, normalize, normalization)  # noqa: E731
    for _ in range(3):
        v = rng.normal(size=x64.shape)
        eps = 1e-6
        want = ((f(x64 + eps * v) - f(x64 - eps * v)) * c64).sum(axis=1) / (2 * eps)
        have = (got * v).sum(axis=1)
        scale = max(1.0, float(np.abs(want).max()))
        assert np.abs(have - want).max() < 2e-4 * scale, (np.abs(have - want).max(), scale)


@pytest.mark.parametrize("maker,Z,shared", [(ks.mfma_small, 300, True), (lambda: ks.golden_tp("uvu_shared_v2"), 200, True),
                                            (lambda: ks.cfg3(True), 130, False), (ks.wide_k_l3, 150, True)])  # fmt: skip
def test_gradients_in_bf16_storage(maker, Z, shared):
    """bf16 storage, fp32 accumulation: every gradient against float64 autograd of the oracle on the same (bf16-rounded)
    inputs, to the bf16 tolerance rel 1e-2 of the largest entry (inputs, outputs and gradients are rounded to bf16)."""
    tp = maker().to(DEV)
    spec = oracle_spec(tp)
    bf = torch.bfloat16
    wshape = (tp.weight_numel,) if shared else (Z, tp.weight_numel)
    x1, x2 = seeded(Z, tp.irreps_in1.dim, seed=1).to(bf), seeded(Z, tp.irreps_in2.dim, seed=2).to(bf)
    w, cot = seeded(*wshape, seed=3).to(bf), seeded(Z, tp.irreps_out.dim, seed=4).to(bf)
    _, (r1, r2, rw) = _oracle_grads(lambda a, b, c: tp_forward_torch(spec, a, b, c), (x1.float(), x2.float(), w.float()), cot.float())
    a, b, c = (t.to(DEV).requires_grad_(True) for t in (x1, x2, w))
    tp(a, b, c).backward(cot.to(DEV))
    for got, ref, what in ((a.grad, r1, "d/dx1"), (b.grad, r2, "d/dx2"), (c.grad, rw, "d/dw")):
        assert got.dtype == bf
        err = (got.float().cpu().double() - ref).abs().max().item()
        assert err <= 2e-2 * max(1.0, ref.abs().max().item()), f"{what}: {err} vs {ref.abs().max().item()}"
