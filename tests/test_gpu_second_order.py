"""GPU parity of second derivatives: what a loss on forces (-dE/dpos) differentiates.

Every check has the same shape.  For a map f with inputs (x_i) take F = <cot, f(x)>, its gradients g_i = dF/dx_i with
``create_graph=True``, the scalar H = sum_i <c_i, g_i> for fixed cotangents c_i, and compare dH/dx_j -- every second
derivative of F contracted with the c_i -- with the same quantity from torch autograd in float64 through the CPU
restatement of the reference's graph (oracle/torch_cpu.py; reference: einsums e3nn/o3/_tensor_product/_codegen.py:148-187,
polynomial chain e3nn/o3/_spherical_harmonics.py:193-249, gather/scatter e3nn/nn/models/v2106/points_convolution.py:13-17,105-106).
"""
import math

import numpy as np
import pytest
import torch

from e3nn_amd import nn, o3
from e3nn_amd.nn import DstSortedEdges
from oracle import nn as onn
from oracle.torch_cpu import spherical_harmonics_torch, tp_forward_torch, tp_gather_scatter_torch
from tests import kernel_sets as ks
from tests.helpers import assert_close, oracle_spec, seeded

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def second_order(fn, inputs, cot, cots_in):
    """(first gradients, gradients of H = sum <c_i, dF/dx_i>) for F = <cot, fn(*inputs)>."""
    inputs = [t.clone().requires_grad_() for t in inputs]
    g = torch.autograd.grad(fn(*inputs), inputs, cot, create_graph=True)
    H = sum((gi * ci).sum() for gi, ci in zip(g, cots_in))
    gg = torch.autograd.grad(H, inputs, allow_unused=True)
    return [t.detach() for t in g], [None if t is None else t.detach() for t in gg]


def compare(fn_gpu, fn_ref, inputs, cot, what, tol=1e-4):
    cots_in = [seeded(*t.shape, seed=70 + i) for i, t in enumerate(inputs)]
    g_ref, gg_ref = second_order(fn_ref, [t.double() for t in inputs], cot.double(), [c.double() for c in cots_in])
    g_gpu, gg_gpu = second_order(fn_gpu, [t.to(DEV) for t in inputs], cot.to(DEV), [c.to(DEV) for c in cots_in])
    for i, (a, b) in enumerate(zip(g_gpu, g_ref)):
        assert_close(a, b.numpy(), atol=tol * max(1.0, float(b.abs().max())), what=f"{what}: dF/dx{i}")
    for i, (a, b) in enumerate(zip(gg_gpu, gg_ref)):
        if b is None:
            assert a is None or not a.any()
            continue
        assert a is not None, f"{what}: dH/dx{i} missing"
        assert_close(a, b.numpy(), atol=tol * max(1.0, float(b.abs().max())), what=f"{what}: dH/dx{i} (second order)")


@pytest.mark.parametrize("maker,Z", [
    (lambda: ks.golden_tp("uvu_merged_cfg3_like_mul4"), 9), (lambda: ks.cfg3(True), 70), (lambda: ks.golden_tp("uvu_shared_v2"), 40),
    (ks.cfg1, 50), (ks.mfma_small, 70), (lambda: ks.golden_tp("fctp_per_sample_weights"), 5), (ks.mixed_modes, 12),
])  # fmt: skip
def test_tensor_product_second_derivatives(maker, Z):
    # uvu with per-sample and with shared weights, uvw on the vector-ALU and on the matrix-core kernels with shared and
    # with per-sample weights, and a mixture of connection modes (differentiated through its dense equivalent)
    tp = maker().to(DEV)
    x1, x2 = seeded(Z, tp.irreps_in1.dim, seed=1), seeded(Z, tp.irreps_in2.dim, seed=2)
    w = seeded(*(() if tp.shared_weights else (Z,)), tp.weight_numel, seed=3) / 2
    cot = seeded(Z, tp.irreps_out.dim, seed=4)
    if tp._live_mode() == "general":
        from oracle import tensor_product as otp

        # the einsum restatement covers uvu / uvw; other modes are checked against central differences of the first
        # gradients of the float64 numpy oracle along one random direction per argument
        inputs = [t.to(DEV).requires_grad_() for t in (x1, x2, w)]
        g = torch.autograd.grad(tp(*inputs), inputs, cot.to(DEV), create_graph=True)
        cs = [seeded(*t.shape, seed=70 + i) for i, t in enumerate(inputs)]
        H = sum((gi * ci.to(DEV)).sum() for gi, ci in zip(g, cs))
        gg = torch.autograd.grad(H, inputs)
        spec, c64 = oracle_spec(tp), cot.numpy().astype(np.float64)
        F = lambda a, b, c: float((otp.tp_forward(spec, a, b, c) * c64).sum())  # noqa: E731
        base = [t.numpy().astype(np.float64) for t in (x1, x2, w)]
        dirs = [c.numpy().astype(np.float64) for c in cs]
        eps = 1e-4

        def H64(args):  # sum_i <c_i, dF/dx_i> by central differences of F along c_i
            tot = 0.0
            for i in range(3):
                hi, lo = list(args), list(args)
                hi[i], lo[i] = args[i] + eps * dirs[i], args[i] - eps * dirs[i]
                tot += (F(*hi) - F(*lo)) / (2 * eps)
            return tot

        rng = np.random.default_rng(0)
        for j in range(3):
            v = rng.normal(size=base[j].shape)
            hi, lo = list(base), list(base)
            hi[j], lo[j] = base[j] + eps * v, base[j] - eps * v
            fd = (H64(hi) - H64(lo)) / (2 * eps)
            assert float((gg[j].cpu().double().numpy() * v).sum()) == pytest.approx(fd, rel=2e-3, abs=2e-3), j
        return
    spec = oracle_spec(tp)
    compare(lambda a, b, c: tp(a, b, c), lambda a, b, c: tp_forward_torch(spec, a, b, c), [x1, x2, w], cot, str(tp))


@pytest.mark.parametrize("maker,N,E,idx", [(lambda: ks.cfg3(True), 60, 1500, torch.int64), (lambda: ks.cfg3(False), 40, 700, torch.int32)])
def test_message_second_derivatives(maker, N, E, idx):
    tp = maker()
    spec = oracle_spec(tp)
    g = torch.Generator().manual_seed(7)
    src, dst = torch.randint(0, N, (E,), generator=g), torch.randint(0, N - 2, (E,), generator=g)
    node_x, attr, w = seeded(N, tp.irreps_in1.dim, seed=1), seeded(E, tp.irreps_in2.dim, seed=2), seeded(E, tp.weight_numel, seed=3) / 2
    cot = seeded(N, tp.irreps_out.dim, seed=4)
    edges = DstSortedEdges(src.to(idx).to(DEV), dst.to(idx).to(DEV), N)
    compare(lambda a, b, c: tp.forward_gather_scatter(a, b, c, edges=edges),
            lambda a, b, c: tp_gather_scatter_torch(spec, a, b, c, src, dst, N), [node_x, attr, w], cot, "message")  # fmt: skip


@pytest.mark.parametrize("lmax", [1, 2, 3])
@pytest.mark.parametrize("normalize,normalization", [(True, "component"), (False, "component"), (True, "integral"), (False, "norm")])
def test_spherical_harmonics_second_derivatives(lmax, normalize, normalization):
    x = seeded(301, 3, seed=5) * (1.0 if normalize else 0.8)
    n_out = (lmax + 1) ** 2
    cot = seeded(301, n_out, seed=6)
    scale = torch.cat([torch.full((2 * l + 1,), {"component": 1.0, "integral": 1 / math.sqrt(4 * math.pi), "norm": 1 / math.sqrt(2 * l + 1)}[normalization])
                       for l in range(lmax + 1)]).double()  # fmt: skip
    ls = list(range(lmax + 1))
    if lmax == 1 and not normalize:
        # linear in the vector: the second derivative vanishes identically (float64 autograd has nothing to differentiate)
        xd = x.to(DEV).requires_grad_()
        (gx,) = torch.autograd.grad(o3.spherical_harmonics(ls, xd, False, normalization), xd, cot.to(DEV), create_graph=True)
        (g2,) = torch.autograd.grad((gx * seeded(301, 3, seed=8).to(DEV)).sum(), xd)
        assert not g2.any()
        return
    compare(lambda v: o3.spherical_harmonics(ls, v, normalize, normalization),
            lambda v: spherical_harmonics_torch(lmax, v, normalize) * scale, [x], cot, f"harmonics lmax {lmax} {normalization}")  # fmt: skip
    # the derivative of the backward pass with respect to the output gradient as well
    xd, gd = x.to(DEV).requires_grad_(), cot.to(DEV).requires_grad_()
    (gx,) = torch.autograd.grad(o3.spherical_harmonics(ls, xd, normalize, normalization), xd, gd, create_graph=True)
    c = seeded(301, 3, seed=8)
    (gg,) = torch.autograd.grad((gx * c.to(DEV)).sum(), gd)
    x64 = x.double().requires_grad_()
    g64 = cot.double().requires_grad_()
    (gx64,) = torch.autograd.grad(spherical_harmonics_torch(lmax, x64, normalize) * scale, x64, g64, create_graph=True)
    (gg64,) = torch.autograd.grad((gx64 * c.double()).sum(), g64)
    assert_close(gg, gg64.numpy(), atol=1e-4 * max(1.0, float(gg64.abs().max())), what="harmonics: d/dgrad_out of the backward pass")
    # a third derivative is refused, not dropped
    (gx,) = torch.autograd.grad(o3.spherical_harmonics(ls, xd, normalize, normalization), xd, cot.to(DEV), create_graph=True)
    (g2,) = torch.autograd.grad((gx * c.to(DEV)).sum(), xd, create_graph=True)
    with pytest.raises(RuntimeError, match="once_differentiable|does not require grad"):
        g2.sum().backward()


def _act64(name):
    f = {"silu": torch.nn.functional.silu, "tanh": torch.tanh, "sigmoid": torch.sigmoid, "abs": torch.abs, "relu": torch.relu}[name]
    cst = onn.normalize2mom_const(name)
    return lambda t: cst * f(t)


def _gate64(x, sc, gates, gated):
    """torch restatement of Gate for ("16x0e+4x0o", [silu, tanh]), ("8x0e+4x0o", [sigmoid, tanh]), "8x1o+4x2e": input
    columns sorted by (l, p): 4x0o (scalars tanh), 4x0o (gates tanh) | 16x0e (scalars silu), 8x0e (gates sigmoid) | 8x1o | 4x2e."""
    s_o, g_o, s_e, g_e = x[:, 0:4], x[:, 4:8], x[:, 8:24], x[:, 24:32]
    y1, y2 = x[:, 32:56].reshape(-1, 8, 3), x[:, 56:76].reshape(-1, 4, 5)
    out_s = torch.cat([_act64("silu")(s_e), _act64("tanh")(s_o)], dim=1)
    return torch.cat([out_s, (_act64("sigmoid")(g_e)[:, :, None] * y1).reshape(-1, 24), (_act64("tanh")(g_o)[:, :, None] * y2).reshape(-1, 20)], dim=1)


def test_gate_second_derivatives():
    args = ("16x0e+4x0o", ["silu", "tanh"], "8x0e+4x0o", ["sigmoid", "tanh"], "8x1o+4x2e")
    gate = nn.Gate(*args)
    assert str(gate.irreps_in) == "8x0o+24x0e+8x1o+4x2e"
    x = seeded(33, gate.irreps_in.dim, seed=3)
    # the restatement used as the float64 reference gives the pinned oracle's values
    ref, _, _ = onn.gate_forward(*args, x.numpy())
    assert np.abs(_gate64(x.double(), *args[::2]).numpy() - ref).max() < 1e-12
    cot = seeded(33, gate.irreps_out.dim, seed=4)
    compare(lambda v: gate(v), lambda v: _gate64(v, *args[::2]), [x], cot, "gate")


def _fc64(x, ws, act, vi=1, vo=1):
    """torch restatement of FullyConnectedNet without output activation (e3nn/nn/_fc.py:38-48,70-88)."""
    n = len(ws)
    var_in = vi
    for i, w in enumerate(ws):
        last = i == n - 1
        var_out = vo if last else 1
        if not last:
            x = _act64(act)(x @ w / math.sqrt(w.shape[0] * var_in))
        else:
            x = x @ w / math.sqrt(w.shape[0] * var_in / var_out)
        var_in = var_out
    return x


@pytest.mark.parametrize("hs,act", [([8, 64, 352], "silu"), ([5, 100, 50], "silu"), ([8, 512, 16], "silu")])
def test_fully_connected_net_second_derivatives(hs, act):
    # one-layer kernels with the activation attached to the next layer, and (512 hidden units) the tensor-product kernels
    torch.manual_seed(5)
    net = nn.FullyConnectedNet(hs, {"silu": torch.nn.functional.silu, "tanh": torch.tanh}[act]).to(DEV)
    ws = [getattr(net, f"layer{i}").weight.detach().cpu() for i in range(len(hs) - 1)]
    x = seeded(77, hs[0], seed=9)
    ref = onn.fc_forward([w.numpy().astype(np.float64) for w in ws], x.numpy(), act)
    assert np.abs(_fc64(x.double(), [w.double() for w in ws], act).numpy() - ref).max() < 1e-10
    cot = seeded(77, hs[-1], seed=10)

    def gpu(v, *weights):  # the given weights are substituted for the parameters, so that they carry the graph
        return torch.func.functional_call(net, {f"layer{i}.weight": w for i, w in enumerate(weights)}, (v,))

    compare(gpu, lambda v, *weights: _fc64(v, weights, act), [x] + ws, cot, f"fully connected net {hs}", tol=2e-4)


def test_forces_can_be_trained_on():
    # positions -> edge vectors -> harmonics (inside the message kernel) and radial network of the lengths -> message
    # -> energy; forces = -dE/dpos with create_graph, a loss on the forces differentiated with respect to the node
    # features and the weights of the radial network: against float64 autograd of the restatement
    tp = ks.cfg3(True)
    spec = oracle_spec(tp)
    N, E = 50, 900
    g = torch.Generator().manual_seed(3)
    src, dst = torch.randint(0, N, (E,), generator=g), torch.randint(0, N, (E,), generator=g)
    dst = torch.where(dst == src, (dst + 1) % N, dst)
    pos, node_x = seeded(N, 3, seed=1) * 2, seeded(N, tp.irreps_in1.dim, seed=2)
    w1, w2 = seeded(8, 64, seed=3), seeded(64, tp.weight_numel, seed=4)
    readout, target = seeded(N, tp.irreps_out.dim, seed=5), seeded(N, 3, seed=6)
    centers = torch.linspace(0.5, 4.0, 8)

    def loss_and_grads(p, x, a, b, energy_of):
        p, x, a, b = (t.clone().requires_grad_() for t in (p, x, a, b))
        energy = energy_of(p, x, a, b)
        (de,) = torch.autograd.grad(energy, p, create_graph=True)
        loss = ((-de - target.to(de)) ** 2).sum()
        return (-de).detach(), torch.autograd.grad(loss, (p, x, a, b))

    def energy64(p, x, a, b):
        vec = p[src] - p[dst]
        scalars = torch.exp(-((vec.norm(dim=1, keepdim=True) - centers.double()) ** 2))
        w = _fc64(scalars, [a, b], "silu")
        out = tp_gather_scatter_torch(spec, x, spherical_harmonics_torch(2, vec, True), w, src, dst, N)
        return (out * readout.double()).sum()

    net = nn.FullyConnectedNet([8, 64, tp.weight_numel], torch.nn.functional.silu).to(DEV)
    edges = DstSortedEdges(src.to(DEV), dst.to(DEV), N)

    def energy_gpu(p, x, a, b):
        vec = p[src.to(DEV)] - p[dst.to(DEV)]
        scalars = torch.exp(-((vec.norm(dim=1, keepdim=True) - centers.to(DEV)) ** 2))
        w = torch.func.functional_call(net, {"layer0.weight": a, "layer1.weight": b}, (scalars,))
        out = tp.forward_gather_scatter_sh(x, vec, w, edges, True, "component")
        return (out * readout.to(DEV)).sum()

    f64, g64 = loss_and_grads(pos.double(), node_x.double(), w1.double(), w2.double(), energy64)
    f32, g32 = loss_and_grads(pos.to(DEV), node_x.to(DEV), w1.to(DEV), w2.to(DEV), energy_gpu)
    assert_close(f32, f64.numpy(), atol=2e-4 * max(1.0, float(f64.abs().max())), what="forces")
    for a, b, name in zip(g32, g64, ("positions", "node features", "radial layer 0", "radial layer 1")):
        assert_close(a, b.numpy(), atol=2e-4 * max(1.0, float(b.abs().max())), what=f"d loss(forces) / d {name}")


def test_convolution_block_second_derivatives():
    # the block's own autograd nodes (lin2 + alpha as one node, the mixing as one node) under create_graph: the mixing
    # against its formula in float64, the joint lin2 + alpha node against the two modules on their own (whose second
    # derivatives are those of the tensor product, checked above)
    from e3nn_amd.nn.convolution import _Mix

    N, C = 40, 12
    sc, alpha, conv = seeded(N, C, seed=1), seeded(N, 1, seed=2), seeded(N, C, seed=3)
    m = (torch.arange(C) % 3 != 0).float()
    c0, c1 = (1 - m) * 0.3, m * 0.09
    compare(lambda a, b, c: _Mix.apply(a, b, c, c0.to(DEV), c1.to(DEV)),
            lambda a, b, c: a + (c0.double() + b * c1.double()) * c, [sc, alpha, conv], seeded(N, C, seed=4), "mixing")  # fmt: skip

    block = ks.conv_wide().to(DEV)
    with torch.no_grad():
        block.alpha.weight.normal_()
    N, E = 60, 900
    g = torch.Generator().manual_seed(11)
    src, dst = torch.randint(0, N, (E,), generator=g).to(DEV), torch.randint(0, N, (E,), generator=g).to(DEV)
    node_input, node_attr = seeded(N, 288, seed=1).to(DEV), seeded(N, 4, seed=2).to(DEV)
    edge_attr = o3.spherical_harmonics([0, 1, 2], seeded(E, 3, seed=3).to(DEV), True, "component")
    edge_scalars = seeded(E, 8, seed=4).to(DEV)
    cot, c_x, c_s = seeded(N, 288, seed=5).to(DEV), seeded(N, 288, seed=6).to(DEV), seeded(E, 8, seed=7).to(DEV)
    params = [p for p in block.parameters()]

    def run():
        x, s = node_input.clone().requires_grad_(), edge_scalars.clone().requires_grad_()
        out = block(x, node_attr, src, dst, edge_attr, s)
        gx, gs = torch.autograd.grad(out, (x, s), cot, create_graph=True)
        H = (gx * c_x).sum() + (gs * c_s).sum()
        return [t.detach() for t in (gx, gs)] + list(torch.autograd.grad(H, [x, s] + params, allow_unused=True))

    assert block._alpha_head is not None
    joint = run()
    head, block.__dict__["_alpha_head"] = block._alpha_head, None
    separate = run()
    block.__dict__["_alpha_head"] = head
    assert any(t is not None and bool(t.abs().sum() > 0) for t in joint[2:])
    for a, b in zip(joint, separate):
        assert (a is None) == (b is None)
        if a is not None:
            assert (a - b).abs().max().item() <= 2e-5 * max(1.0, b.abs().max().item())
