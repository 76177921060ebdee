"""GPU parity of the node-wise blocks either side of the message (o3.Linear, nn.Activation, nn.Gate,
nn.FullyConnectedNet, the v2106 Convolution): the modules on the HIP kernels against fixtures written from the
reference and against the fp64 oracle (oracle/nn.py); gradients against central differences of the oracle."""
import numpy as np
import pytest
import torch

from e3nn_amd import nn, o3
from oracle import nn as onn
from tests import kernel_sets as ks
from tests.helpers import assert_close, seeded

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _t(a):
    return torch.from_numpy(np.asarray(a)).float().to(DEV)


@pytest.mark.parametrize("name", ["linear_mixed", "linear_path_norm", "linear_bias"])
def test_linear_against_reference_fixture(name):
    arr, meta = ks.nn_golden()
    m = meta[name]
    lin = o3.Linear(m["irreps_in"], m["irreps_out"], **m["kwargs"]).to(DEV)
    assert lin.weight_numel == m["weight_numel"]
    with torch.no_grad():
        lin.weight.copy_(_t(arr[name + "/w"]))
        if lin.bias_numel:
            lin.bias.copy_(_t(arr[name + "/bias"]))
    assert_close(lin(_t(arr[name + "/x"])), arr[name + "/out"], what=name)


def test_linear_on_the_matrix_cores():
    lin = dict(ks.nn_modules())["linear_wide"].to(DEV)
    assert lin._tp._plan(torch.float32).family == "uvw_node"
    x = seeded(300, lin.irreps_in.dim, seed=5)
    ref = onn.linear_forward(str(lin.irreps_in), str(lin.irreps_out), x.numpy(), lin.weight.detach().cpu().numpy())
    xd = x.to(DEV).requires_grad_(True)
    out = lin(xd)
    assert_close(out, ref, what="linear_wide")
    # the map is linear in x and in w: <cot, L(x)> differentiates to L^T cot and to x (x) cot
    cot = seeded(300, lin.irreps_out.dim, seed=6)
    out.backward(cot.to(DEV))
    ref_gx = onn.linear_forward(str(lin.irreps_in), str(lin.irreps_out), np.eye(lin.irreps_in.dim), lin.weight.detach().cpu().numpy())
    assert_close(xd.grad, cot.numpy().astype(np.float64) @ ref_gx.T, atol=2e-4, what="d/dx")
    w = lin.weight.detach().cpu().numpy().astype(np.float64)
    rng = np.random.default_rng(0)
    dw = rng.normal(size=w.shape)
    fd = (onn.linear_forward(str(lin.irreps_in), str(lin.irreps_out), x.numpy(), dw) * cot.numpy()).sum()
    assert float((lin.weight.grad.cpu().double().numpy() * dw).sum()) == pytest.approx(fd, rel=2e-4)


@pytest.mark.parametrize("norm", ["element", "path"])
def test_linear_with_input_and_output_channels(norm):
    # f_in / f_out (e3nn/o3/_linear.py:117-118): features [..., f_in, irreps_in.dim] -> [..., f_out, irreps_out.dim], weights
    # [f_in, f_out, weight_numel], every path weight 1 / sqrt(f_in * fan-in) (:152-161), einsum "xyuw,zxui->zywi" (:448);
    # checked against that einsum written out in float64
    f_in, f_out = 3, 2
    lin = ks.linear_channels(norm).to(DEV)
    irreps_in, irreps_out = lin.irreps_in, lin.irreps_out
    assert lin.weight.shape == (f_in, f_out, lin.weight_numel) and lin.bias.shape == (f_out, 5)
    assert lin.weight_numel == 4 * 5 + 2 * 5 + 3 * 2 and lin.output_mask.shape == (irreps_out.dim,) and bool(lin.output_mask.all())
    with torch.no_grad():
        lin.bias.copy_(seeded(f_out, 5, seed=3))
    x = seeded(7 * f_in, irreps_in.dim, seed=1).reshape(7, f_in, irreps_in.dim)
    w = lin.weight.detach().cpu().double().numpy()
    xs, ref = x.double().numpy(), np.zeros((7, f_out, irreps_out.dim))
    off = 0
    for ins in lin.instructions:
        if ins.i_in == -1:
            continue
        U, W = ins.path_shape
        sl_in, sl_out = irreps_in.slices()[ins.i_in], irreps_out.slices()[ins.i_out]
        d = irreps_in[ins.i_in].ir.dim
        fan = sum(irreps_in[i.i_in if norm == "element" else ins.i_in].mul for i in lin.instructions if i.i_in != -1 and i.i_out == ins.i_out)
        assert ins.path_weight == pytest.approx((f_in * fan) ** -0.5)
        blk = w[:, :, off : off + U * W].reshape(f_in, f_out, U, W)
        ref[:, :, sl_out] += ins.path_weight * np.einsum("xyuw,zxui->zywi", blk, xs[:, :, sl_in].reshape(7, f_in, U, d)).reshape(7, f_out, W * d)
        off += U * W
    ref[:, :, :5] += lin.bias.detach().cpu().double().numpy()
    xd = x.to(DEV).requires_grad_(True)
    out = lin(xd)
    assert out.shape == (7, f_out, irreps_out.dim)
    assert_close(out, ref, what=f"Linear f_in f_out {norm}")
    out.square().sum().backward()  # gradients reach the input and the [f_in, f_out, numel] parameter
    assert xd.grad.shape == x.shape and lin.weight.grad.shape == lin.weight.shape and bool(lin.weight.grad.abs().sum() > 0)
    with pytest.raises(ValueError):
        o3.Linear(irreps_in, irreps_out, f_in=3)


def test_activation_and_gate_against_reference_fixtures():
    arr, meta = ks.nn_golden()
    acts = {"silu": torch.nn.functional.silu, "tanh": torch.tanh, "sigmoid": torch.sigmoid, "abs": torch.abs, "relu": torch.relu}
    m = meta["activation"]
    act = nn.Activation(m["irreps_in"], [acts[a] if a else None for a in m["acts"]])
    assert str(act.irreps_out) == m["irreps_out"]
    assert_close(act(_t(arr["activation/x"])), arr["activation/out"], what="activation")
    for name in ("gate_plain", "gate_parity", "gate_only_scalars", "gate_entries_as_given", "gate_gated_in_pieces"):
        sc, a_s, ga, a_g, gd = meta[name]["args"]
        gate = nn.Gate(sc, [acts[k] for k in a_s], ga, [acts[k] for k in a_g], gd)
        assert str(gate.irreps_in) == meta[name]["irreps_in"], name
        assert str(gate.irreps_out.simplify()) == str(o3.Irreps(meta[name]["irreps_out"]).simplify()), name
        assert_close(gate(_t(arr[name + "/x"])), arr[name + "/out"], what=name)


def test_gate_gradient_against_central_differences():
    args = ("16x0e+4x0o", ["silu", "tanh"], "8x0e+4x0o", ["sigmoid", "tanh"], "8x1o+4x2e")
    gate = nn.Gate(args[0], args[1], args[2], args[3], args[4])
    x = seeded(33, gate.irreps_in.dim, seed=3)
    cot = seeded(33, gate.irreps_out.dim, seed=4)
    xd = x.to(DEV).requires_grad_(True)
    out = gate(xd)
    ref, _, _ = onn.gate_forward(*args, x.numpy())
    assert_close(out, ref, what="gate")
    out.backward(cot.to(DEV))
    rng = np.random.default_rng(1)
    x64, c64 = x.numpy().astype(np.float64), cot.numpy().astype(np.float64)
    for _ in range(3):
        v = rng.normal(size=x64.shape)
        eps = 1e-5
        fd = ((onn.gate_forward(*args, x64 + eps * v)[0] - onn.gate_forward(*args, x64 - eps * v)[0]) * c64).sum() / (2 * eps)
        assert float((xd.grad.cpu().double().numpy() * v).sum()) == pytest.approx(fd, rel=1e-4, abs=1e-4)


@pytest.mark.parametrize("case", range(len(ks.FUSED_FC_CASES)))
def test_fully_connected_net_one_kernel(case):
    """Without a gradient the whole network is one kernel: against the oracle and against the layer-by-layer kernels,
    on batch sizes around the 64-row wave tile and the 512-row workgroup tile."""
    hs, act, out_act, vi, vo = ks.FUSED_FC_CASES[case]
    net = ks.fused_fc_nets()[case].to(DEV)
    assert net.fused_plan().handle is not None, net.fused_plan().reason
    ws = [getattr(net, f"layer{i}").weight.detach().cpu().numpy() for i in range(len(hs) - 1)]
    for Z in (0, 1, 63, 513, 20011):
        x = seeded(max(Z, 1), hs[0], seed=100 + case)[:Z]
        with torch.no_grad():
            out = net(x.to(DEV))
        assert out.shape == (Z, hs[-1])
        if Z == 0:
            continue
        want = onn.fc_forward(ws, x.numpy(), act, variance_in=vi, variance_out=vo, out_act=out_act)
        assert_close(out, want, what=f"one-kernel fc {hs} Z={Z}")
        layered = net(x.to(DEV).requires_grad_(True)).detach()
        assert_close(out, layered.cpu().numpy(), what=f"one-kernel fc vs layers {hs} Z={Z}")
    # leading batch dimensions and a view that is not 16-byte aligned
    x = seeded(7 * 11 * hs[0] + 1, 1, seed=5).reshape(-1)[1:].reshape(7, 11, hs[0])
    with torch.no_grad():
        out = net(x.to(DEV)[:, 1:])
    want = onn.fc_forward(ws, x[:, 1:].numpy().reshape(-1, hs[0]), act, variance_in=vi, variance_out=vo, out_act=out_act)
    assert_close(out.reshape(-1, hs[-1]), want, what="one-kernel fc, batch dims")


def test_split_operand_layer_is_as_accurate_as_the_fp32_product():
    """The 64 -> 352 layer runs as six bf16 matrix products of three-way split operands accumulated in fp32.  Against the
    float64 product its error is that of an fp32 matrix product (here: torch's), not that of bf16 arithmetic, also for
    operands with a wide spread of magnitudes."""
    from e3nn_amd.nn.fc import _FusedPlan

    plan = _FusedPlan([64, 352], "identity", False, 1, 1)
    assert plan.handle is not None and plan.workspace_bytes == 64 * 352 * 6  # three bf16 planes: the split path
    g = torch.Generator().manual_seed(7)
    Z = 4099
    x = torch.randn(Z, 64, generator=g) * torch.exp(3.0 * torch.randn(Z, 64, generator=g))  # magnitudes over several decades
    w = torch.randn(64, 352, generator=g) * torch.exp(2.0 * torch.randn(64, 352, generator=g))
    exact = (x.double() @ w.double()) / 8.0
    got = plan.forward(x.to(DEV), [w.to(DEV)]).cpu().double()
    fp32 = ((x.to(DEV) @ w.to(DEV)) / 8.0).cpu().double()
    scale = (x.double().abs() @ w.double().abs()) / 8.0  # what an error of one rounding per product is measured against
    err_split = ((got - exact).abs() / scale).max().item()
    err_fp32 = ((fp32 - exact).abs() / scale).max().item()
    # (errors relative to sum |x||w|: fp32 accumulation of 64 terms alone gives a few 1e-7)
    assert err_split < 2e-6, err_split  # bf16 arithmetic would sit near 4e-3, two-way splits near 2e-5
    assert err_split < 4 * err_fp32 + 2e-7, (err_split, err_fp32)
    print(f"split-operand product: {err_split:.2e}, fp32 product: {err_fp32:.2e}")


@pytest.mark.parametrize("case", range(len(ks.FUSED_FC_CASES)))
def test_fully_connected_net_gradients(case):
    """Under autograd the dense layers run on the one-layer kernels (x @ W, g @ W^T, x^T g): every gradient against
    central differences of the float64 oracle along random directions, on a batch with ragged row tiles."""
    hs, act, out_act, vi, vo = ks.FUSED_FC_CASES[case]
    net = ks.fused_fc_nets()[case].to(DEV)
    n_layers = len(hs) - 1
    assert all(getattr(net, f"layer{i}").dense_plans()[0] for i in range(n_layers))
    Z = 1237
    x = seeded(Z, hs[0], seed=40 + case)
    ws = [getattr(net, f"layer{i}").weight.detach().cpu().numpy().astype(np.float64) for i in range(n_layers)]
    f = lambda xx, ww: onn.fc_forward(ww, xx, act, variance_in=vi, variance_out=vo, out_act=out_act)  # noqa: E731
    xd = x.to(DEV).requires_grad_(True)
    out = net(xd)
    assert_close(out, f(x.numpy(), ws), what="layer-by-layer forward")
    if n_layers > 1 and act is not None:
        # hidden activations are differentiated inside the epilogue of the next layer's input-gradient kernel
        seen, todo = set(), [out.grad_fn]
        while todo:
            fn = todo.pop()
            if fn is not None and fn not in seen:
                seen.add(fn)
                todo += [g for g, _ in fn.next_functions]
        assert sum("_ActDenseFn" in type(fn).__name__ for fn in seen) == n_layers - 1
    cot = seeded(Z, hs[-1], seed=60 + case)
    out.backward(cot.to(DEV))
    rng = np.random.default_rng(case)
    x64, c64 = x.numpy().astype(np.float64), cot.numpy().astype(np.float64)
    eps = 1e-6  # small: relu has kinks, and a step across one biases the difference quotient
    v = rng.normal(size=x64.shape)
    fd = ((f(x64 + eps * v, ws) - f(x64 - eps * v, ws)) * c64).sum() / (2 * eps)
    assert float((xd.grad.cpu().double().numpy() * v).sum()) == pytest.approx(fd, rel=3e-4, abs=1e-3)
    for i in range(n_layers):
        dw = rng.normal(size=ws[i].shape)
        wp = [w + eps * dw if k == i else w for k, w in enumerate(ws)]
        wm = [w - eps * dw if k == i else w for k, w in enumerate(ws)]
        fd = ((f(x64, wp) - f(x64, wm)) * c64).sum() / (2 * eps)
        got = getattr(net, f"layer{i}").weight.grad.cpu().double().numpy()
        assert float((got * dw).sum()) == pytest.approx(fd, rel=3e-4, abs=1e-3), f"layer {i}"


@pytest.mark.parametrize("Z", [1, 15, 16, 17, 33])
def test_dense_layer_gradients_on_batches_around_one_trip(Z):
    """The dense weight-gradient kernel walks the batch in trips of 16 rows shared by four waves, the input-gradient
    kernel in tiles of 32: batches of less than a trip, exactly one, and one row more, against the float64 oracle's
    analytic gradients (the network is y = act(x W0 s0) W1 s1, so they are three matrix products)."""
    net = ks.fused_fc_nets()[0].to(DEV)  # 8 -> 64 -> 352, SiLU
    x = seeded(Z, 8, seed=90 + Z)
    cot = seeded(Z, 352, seed=190 + Z)
    xd = x.to(DEV).requires_grad_(True)
    net(xd).backward(cot.to(DEV))
    w0, w1 = (getattr(net, f"layer{i}").weight.detach().cpu().double().numpy() for i in range(2))
    x64, c64 = x.double().numpy(), cot.double().numpy()
    z = x64 @ w0 / np.sqrt(8.0)
    cst = onn.normalize2mom_const("silu")
    sg = 1.0 / (1.0 + np.exp(-z))
    h = cst * z * sg
    assert_close(net(x.to(DEV)), onn.fc_forward([w0, w1], x64, "silu"), what=f"fc forward, Z = {Z}")
    gh = c64 @ w1.T / 8.0
    gz = gh * cst * sg * (1.0 + z * (1.0 - sg))
    assert_close(net.layer1.weight.grad, h.T @ c64 / 8.0, what=f"dense weight gradient 64x352, Z = {Z}")
    assert_close(net.layer0.weight.grad, x64.T @ gz / np.sqrt(8.0), what=f"dense weight gradient 8x64, Z = {Z}")
    assert_close(xd.grad, gz @ w0.T / np.sqrt(8.0), what=f"dense input gradient, Z = {Z}")


def test_fully_connected_net_wide_hidden_layer():
    """Outside the limits of the fused kernel every layer runs on the tensor-product kernels, forward and backward."""
    fc = dict(ks.nn_modules())["fc_wide_hidden"].to(DEV)
    assert fc.fused_plan().handle is None and not fc.layer0.dense_plans()[0]
    x = seeded(300, 8, seed=21)
    ws = [fc.layer0.weight.detach().cpu().numpy(), fc.layer1.weight.detach().cpu().numpy()]
    with torch.no_grad():
        assert_close(fc(x.to(DEV)), onn.fc_forward(ws, x.numpy(), "silu"), what="wide fc, no grad")
    xd = x.to(DEV).requires_grad_(True)
    out = fc(xd)
    assert_close(out, onn.fc_forward(ws, x.numpy(), "silu"), what="wide fc")
    cot = seeded(300, 16, seed=22)
    out.backward(cot.to(DEV))
    rng = np.random.default_rng(3)
    x64, c64 = x.numpy().astype(np.float64), cot.numpy().astype(np.float64)
    v, eps = rng.normal(size=x64.shape), 1e-5
    fd = ((onn.fc_forward(ws, x64 + eps * v) - onn.fc_forward(ws, x64 - eps * v)) * c64).sum() / (2 * eps)
    assert float((xd.grad.cpu().double().numpy() * v).sum()) == pytest.approx(fd, rel=2e-4)
    dw = rng.normal(size=ws[1].shape)
    fd = ((onn.fc_forward([ws[0], ws[1] + eps * dw], x64) - onn.fc_forward([ws[0], ws[1] - eps * dw], x64)) * c64).sum() / (2 * eps)
    assert float((fc.layer1.weight.grad.cpu().double().numpy() * dw).sum()) == pytest.approx(fd, rel=2e-4)


def test_fully_connected_net():
    arr, meta = ks.nn_golden()
    fc = nn.FullyConnectedNet(meta["fc"]["hs"], torch.nn.functional.silu).to(DEV)
    with torch.no_grad():
        for i in range(3):
            getattr(fc, f"layer{i}").weight.copy_(_t(arr[f"fc/w{i}"]))
    assert_close(fc(_t(arr["fc/x"])), arr["fc/out"], what="fc fixture")
    # radial-network shape: 8 -> 64 -> 352, the second layer on the matrix cores
    fc = dict(ks.nn_modules())["fc_radial"].to(DEV)
    assert fc.layer1._tp._plan(torch.float32).family == "uvw_node"
    x = seeded(1000, 8, seed=8)
    ws = [fc.layer0.weight.detach().cpu().numpy(), fc.layer1.weight.detach().cpu().numpy()]
    xd = x.to(DEV).requires_grad_(True)
    out = fc(xd)
    assert_close(out, onn.fc_forward(ws, x.numpy(), "silu"), what="fc radial")
    cot = seeded(1000, 352, seed=9)
    out.backward(cot.to(DEV))
    rng = np.random.default_rng(2)
    x64, c64 = x.numpy().astype(np.float64), cot.numpy().astype(np.float64)
    v = rng.normal(size=x64.shape)
    eps = 1e-5
    fd = ((onn.fc_forward(ws, x64 + eps * v) - onn.fc_forward(ws, x64 - eps * v)) * c64).sum() / (2 * eps)
    assert float((xd.grad.cpu().double().numpy() * v).sum()) == pytest.approx(fd, rel=2e-4)
    dw = rng.normal(size=ws[0].shape)
    fd = ((onn.fc_forward([ws[0] + eps * dw, ws[1]], x64) - onn.fc_forward([ws[0] - eps * dw, ws[1]], x64)) * c64).sum() / (2 * eps)
    assert float((fc.layer0.weight.grad.cpu().double().numpy() * dw).sum()) == pytest.approx(fd, rel=2e-4)
    dw = rng.normal(size=ws[1].shape)
    fd = ((onn.fc_forward([ws[0], ws[1] + eps * dw], x64) - onn.fc_forward([ws[0], ws[1] - eps * dw], x64)) * c64).sum() / (2 * eps)
    assert float((fc.layer1.weight.grad.cpu().double().numpy() * dw).sum()) == pytest.approx(fd, rel=2e-4)
    assert fc.layer1.dense_plans()[0], "the dense layers of the radial network run on the one-layer kernels"


def _conv_oracle(conv, args, params, node_input, node_attr, src, dst, edge_attr, edge_scalars):
    return onn.convolution_forward(args[0], args[1], args[2], args[3], args[5], params, node_input, node_attr, src, dst,
                                   edge_attr, edge_scalars)  # fmt: skip


def test_convolution_against_reference_fixture():
    arr, meta = ks.nn_golden()
    a = meta["conv"]["args"]
    conv = nn.Convolution(a[0], a[1], a[2], a[3], a[4], a[5]).to(DEV)
    assert str(conv.tp.irreps_out) == meta["conv"]["irreps_mid"]
    assert [[i.i_in1, i.i_in2, i.i_out] for i in conv.tp.instructions] == meta["conv"]["tp_instructions"]
    sd = {k[len("conv/param/"):]: _t(arr[k]) for k in arr.files if k.startswith("conv/param/")}
    missing = conv.load_state_dict(sd, strict=False)
    assert not [k for k in missing.unexpected_keys], missing
    own = conv.state_dict()
    assert not [k for k in missing.missing_keys if k.endswith("weight") and "_tp" not in k and own[k].numel()], missing
    out = conv(_t(arr["conv/node_input"]), _t(arr["conv/node_attr"]), torch.from_numpy(arr["conv/src"]).to(DEV),
               torch.from_numpy(arr["conv/dst"]).to(DEV), _t(arr["conv/edge_attr"]), _t(arr["conv/edge_scalars"]))  # fmt: skip
    assert_close(out, arr["conv/out"], atol=2e-4, what="convolution fixture")


def test_convolution_block_forward_and_backward():
    conv = ks.conv_wide().to(DEV)
    with torch.no_grad():
        conv.alpha.weight.normal_()
    N, E = 150, 2500
    g = torch.Generator().manual_seed(11)
    src, dst = torch.randint(0, N, (E,), generator=g), torch.randint(0, N, (E,), generator=g)
    node_input, node_attr = seeded(N, 288, seed=1), seeded(N, 4, seed=2)
    vec = seeded(E, 3, seed=3)
    edge_attr = o3.spherical_harmonics([0, 1, 2], vec.to(DEV), True, "component").cpu()
    edge_scalars = seeded(E, 8, seed=4)
    params = {k: v.detach().cpu().numpy().astype(np.float64) for k, v in conv.state_dict().items() if k.endswith("weight") and v.numel()}
    a = ("32x0e+32x1o+32x2e", "4x0e", ks.SH2, "32x0e+32x1o+32x2e", [8, 64], 37.5)
    run = lambda x, p=params: _conv_oracle(conv, a, p, x, node_attr.numpy(), src.numpy(), dst.numpy(), edge_attr.numpy(), edge_scalars.numpy())  # noqa: E731
    xd = node_input.to(DEV).requires_grad_(True)
    out = conv(xd, node_attr.to(DEV), src.to(DEV), dst.to(DEV), edge_attr.to(DEV), edge_scalars.to(DEV))
    ref = run(node_input.numpy())
    assert_close(out, ref, atol=1e-4 * max(1.0, float(np.abs(ref).max())), what="convolution block")
    # without gradients the radial network runs inside the message kernel
    with torch.no_grad():
        assert conv.tp.prepare_gather_scatter_radial(conv.fc)
        out2 = conv(node_input.to(DEV), node_attr.to(DEV), src.to(DEV), dst.to(DEV), edge_attr.to(DEV), edge_scalars.to(DEV))
    assert_close(out2, ref, atol=1e-4 * max(1.0, float(np.abs(ref).max())), what="convolution block, inference path")
    cot = seeded(N, 288, seed=5)
    out.backward(cot.to(DEV))
    rng = np.random.default_rng(3)
    x64, c64 = node_input.numpy().astype(np.float64), cot.numpy().astype(np.float64)
    v = rng.normal(size=x64.shape)
    eps = 1e-5
    fd = ((run(x64 + eps * v) - run(x64 - eps * v)) * c64).sum() / (2 * eps)
    assert float((xd.grad.cpu().double().numpy() * v).sum()) == pytest.approx(fd, rel=5e-4)
    for key, par in (("fc.layer0.weight", conv.fc.layer0.weight), ("lin1.weight", conv.lin1.weight), ("alpha.weight", conv.alpha.weight),
                     ("lin2.weight", conv.lin2.weight), ("sc.weight", conv.sc.weight)):
        dw = rng.normal(size=params[key].shape)
        hi, lo = dict(params), dict(params)
        hi[key], lo[key] = params[key] + eps * dw, params[key] - eps * dw
        fd = ((run(x64, hi) - run(x64, lo)) * c64).sum() / (2 * eps)
        got = float((par.grad.cpu().double().numpy().reshape(dw.shape) * dw).sum())
        assert got == pytest.approx(fd, rel=5e-4, abs=1e-3), key
    # lin2 and alpha as one node of the autograd graph (taken above) against the two modules on their own
    assert conv._alpha_head is not None
    joint = [xd.grad.clone()] + [p.grad.clone() for p in conv.parameters()]
    xd.grad = None
    conv.zero_grad(set_to_none=True)
    conv.__dict__["_alpha_head"] = None
    conv(xd, node_attr.to(DEV), src.to(DEV), dst.to(DEV), edge_attr.to(DEV), edge_scalars.to(DEV)).backward(cot.to(DEV))
    for a_, b_ in zip(joint, [xd.grad] + [p.grad for p in conv.parameters()]):
        assert_close(a_, b_.cpu().numpy(), atol=1e-5 * max(1.0, float(b_.abs().max())), what="joint lin2 + alpha")


# bf16 storage of the node-wise blocks: rows and parameters are stored as bf16, the kernels compute in fp32.  The
# reference is the same module on the same (bf16-representable) numbers held as fp32.  Every stage that stores its
# result as bf16 rounds it by at most 2^-8 of its size (eight significant bits, round to nearest), and the next stage
# sums such values: the tolerance is 2^-8 of the largest reference value per stored stage, plus rel 1e-2 as for the
# bf16 message kernels.
def _bf16_tol(ref, stages=1):
    return dict(atol=stages * 2.0**-8 * float(ref.detach().abs().max()), rtol=1e-2)


def test_gate_and_activation_in_bf16_storage():
    gate = nn.Gate("16x0e+4x0o", ["silu", "tanh"], "8x0e+4x0o", ["sigmoid", "tanh"], "8x1o+4x2e")
    x = seeded(257, gate.irreps_in.dim, seed=3).bfloat16()
    cot = seeded(257, gate.irreps_out.dim, seed=4).bfloat16()
    xb, xf = x.to(DEV).requires_grad_(True), x.float().to(DEV).requires_grad_(True)
    ob, of = gate(xb), gate(xf)
    assert ob.dtype == torch.bfloat16
    # one rounding of the fp32 result to bf16: at most 2^-8 of the value
    assert_close(ob, of.detach().cpu().numpy(), atol=1e-30, rtol=2.0**-8, what="gate, bf16 storage")
    ob.backward(cot.to(DEV))
    of.backward(cot.float().to(DEV))
    assert xb.grad.dtype == torch.bfloat16
    assert_close(xb.grad, xf.grad.cpu().numpy(), atol=2.0**-8 * float(xf.grad.abs().max()), rtol=2.0**-8, what="gate gradient, bf16 storage")
    act = nn.Activation("64x0e+8x1o", [torch.nn.functional.silu, None])
    y = seeded(100, act.irreps_in.dim, seed=5).bfloat16().to(DEV)
    assert_close(act(y), act(y.float()).cpu().numpy(), atol=1e-30, rtol=2.0**-8, what="activation, bf16 storage")
    # second derivative (a loss on a gradient), against the fp32 kernels on the same numbers
    res = []
    for t in (x.to(DEV), x.float().to(DEV)):
        t = t.requires_grad_(True)
        (g1,) = torch.autograd.grad(gate(t).square().sum(), t, create_graph=True)
        (g2,) = torch.autograd.grad(g1.square().sum(), t)
        res.append(g2)
    assert_close(res[0], res[1].cpu().numpy(), **_bf16_tol(res[1], 3), what="gate second derivative, bf16 storage")
    with pytest.raises(NotImplementedError):
        gate(x.half().to(DEV))


def test_node_wise_blocks_in_bf16_storage():
    import copy

    lin = dict(ks.nn_modules())["linear_wide"].to(DEV)
    x = seeded(300, lin.irreps_in.dim, seed=6).bfloat16().to(DEV)
    with torch.no_grad():
        lin.weight.copy_(lin.weight.bfloat16().float())
    ref_in = x.float().requires_grad_(True)
    ref = lin(ref_in)
    ref.backward(torch.ones_like(ref))
    lb = copy.deepcopy(lin).to(torch.bfloat16)
    xb = x.clone().requires_grad_(True)
    out = lb(xb)
    assert out.dtype == torch.bfloat16
    assert_close(out, ref.detach().cpu().numpy(), **_bf16_tol(ref), what="linear, bf16 storage")
    out.backward(torch.ones_like(out))
    assert_close(xb.grad, ref_in.grad.cpu().numpy(), **_bf16_tol(ref_in.grad), what="linear d/dx, bf16 storage")
    assert_close(lb.weight.grad, lin.weight.grad.cpu().numpy(), **_bf16_tol(lin.weight.grad), what="linear d/dw, bf16 storage")

    net = dict(ks.nn_modules())["fc_radial"].to(DEV)
    with torch.no_grad():
        for p in net.parameters():
            p.copy_(p.bfloat16().float())
    s = seeded(1000, 8, seed=7).bfloat16().to(DEV)
    ref = net(s.float())
    nb = copy.deepcopy(net).to(torch.bfloat16)
    assert_close(nb(s), ref.detach().cpu().numpy(), **_bf16_tol(ref, 2), what="radial network, bf16 storage")
    with torch.no_grad():
        assert_close(nb(s), ref.detach().cpu().numpy(), **_bf16_tol(ref, 2), what="radial network without gradients, bf16 storage")

    conv = ks.conv_wide().to(DEV)
    with torch.no_grad():
        conv.alpha.weight.normal_()
        for p in conv.parameters():
            p.copy_(p.bfloat16().float())
    N, E = 150, 2500
    g = torch.Generator().manual_seed(11)
    src, dst = torch.randint(0, N, (E,), generator=g).to(DEV), torch.randint(0, N, (E,), generator=g).to(DEV)
    node_input, node_attr = seeded(N, 288, seed=1).bfloat16().to(DEV), seeded(N, 4, seed=2).bfloat16().to(DEV)
    edge_attr = o3.spherical_harmonics([0, 1, 2], seeded(E, 3, seed=3).to(DEV), True, "component").bfloat16()
    edge_scalars = seeded(E, 8, seed=4).bfloat16().to(DEV)
    xf = node_input.float().requires_grad_(True)
    ref = conv(xf, node_attr.float(), src, dst, edge_attr.float(), edge_scalars.float())
    cot = seeded(N, 288, seed=5).bfloat16().to(DEV)
    ref.backward(cot.float())
    cb = copy.deepcopy(conv).to(torch.bfloat16)
    xb = node_input.clone().requires_grad_(True)
    out = cb(xb, node_attr, src, dst, edge_attr, edge_scalars)
    assert out.dtype == torch.bfloat16
    # five bf16-stored stages in a row forward (lin1, radial weights, message, lin2 / alpha, mix), as many again backward
    assert_close(out, ref.detach().cpu().numpy(), **_bf16_tol(ref, 5), what="convolution block, bf16 storage")
    out.backward(cot)
    assert_close(xb.grad, xf.grad.cpu().numpy(), **_bf16_tol(xf.grad, 10), what="convolution block d/dx, bf16 storage")
    for (name, pb), pf in zip(cb.named_parameters(), conv.parameters()):
        if pf.grad is None or not pf.numel():
            continue
        assert pb.grad.dtype == torch.bfloat16, name
        assert_close(pb.grad, pf.grad.cpu().numpy(), **_bf16_tol(pf.grad, 10), what=f"convolution block d/d{name}, bf16 storage")
