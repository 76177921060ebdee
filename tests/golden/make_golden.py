"""Writes the golden fixtures in this directory from the reference implementation.

Run once, in the build container only (the reference never leaves it):

    python tests/golden/make_golden.py [/root/reference]

The reference imports ``opt_einsum_fx`` at module scope; that package only re-orders
einsum contractions (no arithmetic of its own) and is not installed here, so an
in-memory module with identity ``jitable`` / ``optimize_einsums_full`` is registered
before the import.  Everything is evaluated in float64.  The fixtures hold inputs and
expected outputs only:

* w3j.npz          wigner_3j(l1, l2, l3) for every valid triple with l <= 4
* sh.npz           spherical_harmonics on 24 fixed points, l <= 8, all option combinations
* tp_cases.json    instruction tables (path weights, shapes, weight_numel, sorted output
                   irreps, output_mask) incl. the five benchmark configurations
* tp_cases.npz     seeded inputs and outputs of small TensorProducts and of
                   gather -> TensorProduct -> scatter
* nn_cases.npz/json  (``python tests/golden/make_golden.py nn``) o3.Linear, nn.Activation, nn.Gate,
                   nn.FullyConnectedNet and the v2106 Convolution: parameters, inputs, outputs, irreps strings
* state_dict_keys.json  (``python tests/golden/make_golden.py state``) names and shapes of the entries of
                   ``TensorProduct.state_dict()`` (weights, output mask and the constant buffers of the generated
                   modules) for a list of constructor arguments
"""
import json
import os
import sys
import types

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def import_reference(path):
    stub = types.ModuleType("opt_einsum_fx")
    stub.jitable = lambda m: m
    stub.optimize_einsums_full = lambda m, example_inputs: m
    sys.modules["opt_einsum_fx"] = stub
    sys.path.insert(0, path)
    torch.set_default_dtype(torch.float64)
    import e3nn  # noqa: F401
    from e3nn import o3

    return o3


def conv_builder(o3, irreps_in, irreps_edge, keep):
    # call-site instruction builder, as the reference model code does it
    irreps_in, irreps_edge = o3.Irreps(irreps_in), o3.Irreps(irreps_edge)
    keep = [o3.Irrep(k) for k in keep]
    mid, ins = [], []
    for i, (mul, ir_in) in enumerate(irreps_in):
        for j, (_, ir_edge) in enumerate(irreps_edge):
            for ir_out in ir_in * ir_edge:
                if ir_out in keep:
                    ins.append((i, j, len(mid), "uvu", True))
                    mid.append((mul, ir_out))
    mid = o3.Irreps(mid)
    mid, p, _ = mid.sort()
    return mid, [(a, b, p[c], m, t) for a, b, c, m, t in ins]


def merged_uvu(o3, irreps_in, irreps_edge, irreps_out):
    irreps_in, irreps_edge, irreps_out = o3.Irreps(irreps_in), o3.Irreps(irreps_edge), o3.Irreps(irreps_out)
    return [
        (i, j, k, "uvu", True)
        for i, (_, a) in enumerate(irreps_in)
        for j, (_, b) in enumerate(irreps_edge)
        for k, (_, c) in enumerate(irreps_out)
        if c in a * b
    ]


def describe(tp):
    return {
        "irreps_in1": str(tp.irreps_in1),
        "irreps_in2": str(tp.irreps_in2),
        "irreps_out": str(tp.irreps_out),
        "instructions": [
            [t.i_in1, t.i_in2, t.i_out, t.connection_mode, bool(t.has_weight), float(t.path_weight), list(t.path_shape)]
            for t in tp.instructions
        ],
        "weight_numel": int(tp.weight_numel),
        "shared_weights": bool(tp.shared_weights),
        "internal_weights": bool(tp.internal_weights),
        # one flag per output irrep block (the mask is constant inside a block)
        "output_mask_blocks": [int(tp.output_mask[s.start]) if s.stop > s.start else -1 for s in tp.irreps_out.slices()],
    }


STATE_CASES = [
    # (name, irreps_in1, irreps_in2, irreps_out, instructions, kwargs)
    ("fctp_l2", "2x0e+2x1o+2x2e", "0e+1o+2e", "2x0e+2x1o+2x2e", None, {}),
    ("fctp_l2_unspecialized", "2x0e+2x1o+2x2e", "0e+1o+2e", "2x0e+2x1o+2x2e", None, {"_specialized_code": False}),
    ("fctp_right", "2x0e+2x1o", "0e+1o", "2x0e+2x1o+1x2e", None, {"compile_right": True}),
    ("uvu_mixed", "3x0e+3x1o", "2x0e+2x1o", "3x0e+3x1o",
     [(0, 0, 0, "uvu", True), (0, 1, 1, "uvu", True), (1, 0, 1, "uvu", False), (1, 1, 0, "uvu", True), (1, 1, 0, "uvu", False)], {}),
    ("modes", "3x1o+3x2e+3x0e", "3x1o+3x0e", "3x1e+3x2e+9x1o+2x2o+3x1o+3x0e+1x0e",
     [(0, 0, 0, "uuu", True), (1, 1, 1, "uuu", False), (0, 1, 2, "uvuv", True), (1, 0, 3, "uuw", True), (0, 1, 4, "uvv", True),
      (2, 1, 5, "uuu", False), (0, 0, 6, "uuw", False), (1, 1, 1, "uvv", False)], {}),
    ("modes_right", "3x1o+3x2e", "3x1o+3x0e", "3x1e+3x2e+9x1o+2x2o+3x1o",
     [(0, 0, 0, "uuu", True), (1, 1, 1, "uuu", False), (0, 1, 2, "uvuv", True), (1, 0, 3, "uuw", True), (0, 1, 4, "uvv", True)],
     {"compile_right": True}),
    ("triangular", "4x1o+4x0e", "4x1o+4x0e", "6x1e+3x2e+6x0e", [(0, 0, 0, "uvu<v", True), (0, 0, 1, "u<vw", True), (1, 1, 2, "uvu<v", False)], {}),
    ("empty_paths", "2x0e+0x1o", "1o", "2x1o+3x2e", [(0, 0, 0, "uvu", True), (1, 0, 1, "uvw", True)], {}),
    ("external_weights", "2x0e+2x1o", "0e+1o", "2x0e+2x1o", None, {"internal_weights": False, "shared_weights": False}),
]


def main_state():
    ref = sys.argv[2] if len(sys.argv) > 2 else "/root/reference"
    o3 = import_reference(ref)
    out = {}
    for name, i1, i2, io, ins, kw in STATE_CASES:
        tp = o3.FullyConnectedTensorProduct(i1, i2, io, **kw) if ins is None else o3.TensorProduct(i1, i2, io, ins, **kw)
        out[name] = {
            "args": [i1, i2, io, ins, kw],
            "state_dict": {k: list(v.shape) for k, v in tp.state_dict().items()},
        }
    # node-wise blocks: module constructors by name, positional arguments as JSON
    from e3nn import nn
    from e3nn.nn.models.v2106.points_convolution import Convolution

    silu, sigmoid, tanh = torch.nn.functional.silu, torch.sigmoid, torch.tanh
    modules = {
        "linear": (o3.Linear, ["2x0e+2x1o", "3x0e+1x1o"], {"biases": True}),
        "linear_l2": (o3.Linear, ["2x0e+2x1o+2x2e", "3x0e+1x1o+2x2e"], {}),
        "fc": (nn.FullyConnectedNet, [[4, 8, 2], silu], {}),
        "gate": (nn.Gate, ["4x0e+2x0o", [silu, tanh], "3x0e", [sigmoid], "2x1o+1x2e"], {}),
        "activation": (nn.Activation, ["4x0e+2x0o", [silu, tanh]], {}),
        "convolution_l1": (Convolution, ["4x0e+4x1o", "2x0e", "0e+1o", "4x0e+4x1o", [3, 8], 3.0], {}),
        "convolution_l2": (Convolution, ["4x0e+4x1o+4x2e", "2x0e", "0e+1o+2e", "4x0e+4x1o+4x2e", [3, 8], 3.0], {}),
    }
    for name, (ctor, args, kw) in modules.items():
        m = ctor(*args, **kw)
        out["module_" + name] = {"state_dict": {k: list(v.shape) for k, v in m.state_dict().items()}}
    with open(os.path.join(HERE, "state_dict_keys.json"), "w") as f:
        json.dump(out, f, indent=1)
    print("wrote state_dict_keys.json:", {k: len(v["state_dict"]) for k, v in out.items()})


def main():
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    o3 = import_reference(ref)
    g = torch.Generator().manual_seed(0)

    # ---- wigner 3j ---------------------------------------------------------------
    w3j = {}
    for l1 in range(5):
        for l2 in range(5):
            for l3 in range(abs(l1 - l2), min(4, l1 + l2) + 1):
                w3j[f"{l1}_{l2}_{l3}"] = o3.wigner_3j(l1, l2, l3).numpy()
    np.savez_compressed(os.path.join(HERE, "w3j.npz"), **w3j)

    # ---- spherical harmonics -----------------------------------------------------
    pts = torch.randn(20, 3, generator=g)
    pts = torch.cat([pts, torch.zeros(1, 3), torch.tensor([[0.0, 1.0, 0.0], [1e-20, 0.0, 0.0], [3.0, -4.0, 12.0]])])
    sh = {"points": pts.numpy()}
    for normalize in (True, False):
        for normalization in ("integral", "component", "norm"):
            out = o3.spherical_harmonics(list(range(9)), pts, normalize, normalization)
            sh[f"lmax8_{int(normalize)}_{normalization}"] = out.numpy()
    sh["ls_2_0_3_1_component"] = o3.spherical_harmonics([2, 0, 3], pts, True, "component").numpy()
    np.savez_compressed(os.path.join(HERE, "sh.npz"), **sh)

    # ---- tensor products ---------------------------------------------------------
    meta, arrays = {}, {}

    def add_case(name, tp, Z, extra=None, run=True):
        d = describe(tp)
        if extra:
            d.update(extra)
        meta[name] = d
        if not run:
            return
        x1 = torch.randn(Z, tp.irreps_in1.dim, generator=g)
        x2 = torch.randn(Z, tp.irreps_in2.dim, generator=g)
        if tp.weight_numel and not tp.internal_weights:
            w = torch.randn(*(() if tp.shared_weights else (Z,)), tp.weight_numel, generator=g)
            out = tp(x1, x2, w)
        elif tp.weight_numel:
            w = tp.weight.detach().clone()
            out = tp(x1, x2)
        else:
            w = torch.zeros(0)
            out = tp(x1, x2)
        arrays[name + "/x1"], arrays[name + "/x2"] = x1.numpy(), x2.numpy()
        arrays[name + "/w"], arrays[name + "/out"] = w.numpy(), out.detach().numpy()

    # configuration 1 (rows of it), and the structure of configuration 5
    tp = o3.FullyConnectedTensorProduct("16x0e+16x1o", "0e+1o+2e", "16x0e+16x1o+16x2e")
    add_case("fctp_cfg1", tp, 16)
    tp = o3.FullyConnectedTensorProduct("128x0e+128x1o+128x2e", "128x0e+128x1o+128x2e", "128x0e+128x1o+128x2e")
    add_case("fctp_cfg5_structure", tp, 0, run=False)
    tp = o3.FullyConnectedTensorProduct("3x0e+3x1o+3x2e", "3x0e+3x1o+3x2e", "3x0e+3x1o+3x2e")
    add_case("fctp_small_cfg5_like", tp, 5)
    tp = o3.FullyConnectedTensorProduct("2x0e+3x1o", "2x0e+1x1o+1x1e", "2x0e+2x1o+3x1e+1x2e", shared_weights=False)
    add_case("fctp_per_sample_weights", tp, 6)
    tp = o3.FullyConnectedTensorProduct("4x0e+2x1o+1x2e", "0e+1o", "3x0e+5x1o", irrep_normalization="norm", path_normalization="path")
    add_case("fctp_norm_path", tp, 4)

    # configuration 3: merged outputs, and the call-site builder with sorted per-path blocks
    sh2, sh3 = str(o3.Irreps.spherical_harmonics(2)), str(o3.Irreps.spherical_harmonics(3))
    for mul, tag, run in ((32, "cfg3_structure", False), (4, "cfg3_like_mul4", True)):
        feats = f"{mul}x0e+{mul}x1o+{mul}x2e"
        tp = o3.TensorProduct(feats, sh2, feats, merged_uvu(o3, feats, sh2, feats), internal_weights=False, shared_weights=False)
        add_case("uvu_merged_" + tag, tp, 7, run=run)
        mid, ins = conv_builder(o3, feats, sh2, ["0e", "1o", "2e"])
        tp = o3.TensorProduct(feats, sh2, mid, ins, internal_weights=False, shared_weights=False)
        add_case("uvu_builder_" + tag, tp, 7, run=run)
    # configuration 4: MACE-scale, targets 0e 1o 2e 3o (A) and every l <= 3 of both parities (B)
    for mul, tag, run in ((128, "cfg4_structure", False), (2, "cfg4_like_mul2", True)):
        feats = f"{mul}x0e+{mul}x1o+{mul}x2e+{mul}x3o"
        mid, ins = conv_builder(o3, feats, sh3, ["0e", "1o", "2e", "3o"])
        tp = o3.TensorProduct(feats, sh3, mid, ins, internal_weights=False, shared_weights=False)
        add_case("uvu_builderA_" + tag, tp, 5, run=run)
        mid, ins = conv_builder(o3, feats, sh3, ["0e", "0o", "1e", "1o", "2e", "2o", "3e", "3o"])
        tp = o3.TensorProduct(feats, sh3, mid, ins, internal_weights=False, shared_weights=False)
        add_case("uvu_builderB_" + tag, tp, 5, run=run)

    # uvu with in2 multiplicity > 1 and shared weights; unweighted uvu
    tp = o3.TensorProduct("3x0e+3x1o", "2x0e+2x1o", "3x0e+3x1o", [(0, 0, 0, "uvu", True), (0, 1, 1, "uvu", True), (1, 0, 1, "uvu", True), (1, 1, 0, "uvu", True)])
    add_case("uvu_shared_v2", tp, 5)
    tp = o3.TensorProduct("3x1o", "2x1o", "3x1e+3x2e", [(0, 0, 0, "uvu", False), (0, 0, 1, "uvu", True, 2.5)], internal_weights=False, shared_weights=True)
    add_case("uvu_mixed_weightless", tp, 5, extra={"user_path_weights": [1.0, 2.5]})
    # the other connection modes
    tp = o3.TensorProduct("3x1o+3x2e", "3x1o+3x0e", "3x1e+3x2e+9x1o+2x2o+3x1o", [
        (0, 0, 0, "uuu", True), (1, 1, 1, "uuu", False), (0, 1, 2, "uvuv", True), (1, 0, 3, "uuw", True), (0, 1, 4, "uvv", True)])
    add_case("modes_uuu_uvuv_uuw_uvv", tp, 4)
    tp = o3.TensorProduct("4x1o", "4x1o", "6x1e+3x2e", [(0, 0, 0, "uvu<v", True), (0, 0, 1, "u<vw", True)])
    add_case("modes_triangular", tp, 4)
    tp = o3.TensorProduct("2x0e+0x1o", "1o", "2x1o+3x2e", [(0, 0, 0, "uvu", True), (1, 0, 1, "uvw", True)])
    add_case("empty_path_and_missing_output", tp, 3)

    # gather -> TP -> scatter, with the reference's scatter()
    feats = "4x0e+4x1o+4x2e"
    mid, ins = conv_builder(o3, feats, sh2, ["0e", "1o", "2e"])
    tp = o3.TensorProduct(feats, sh2, mid, ins, internal_weights=False, shared_weights=False)
    N, E = 6, 17
    node_x = torch.randn(N, tp.irreps_in1.dim, generator=g)
    vec = torch.randn(E, 3, generator=g)
    attr = o3.spherical_harmonics(list(range(3)), vec, True, "component")
    w = torch.randn(E, tp.weight_numel, generator=g)
    src = torch.randint(0, N, (E,), generator=g)
    dst = torch.randint(0, N - 1, (E,), generator=g)  # node N-1 receives nothing
    msg = tp(node_x[src], attr, w)
    out = msg.new_zeros(N, msg.shape[1]).scatter_add_(0, dst.reshape(-1, 1).expand_as(msg), msg)
    meta["conv_small"] = describe(tp)
    for k, v in dict(node_x=node_x, vec=vec, attr=attr, w=w, src=src, dst=dst, out=out).items():
        arrays["conv_small/" + k] = v.numpy()

    meta["sort"] = {}
    for s in ("2o+1e+0e+1e", "1e+0e+1e", "4x0e+4x1o+4x2e+4x1o+4x0e+4x2o+1x0o"):
        r = o3.Irreps(s).sort()
        meta["sort"][s] = {"irreps": str(r.irreps), "p": list(r.p), "inv": list(r.inv)}

    np.savez_compressed(os.path.join(HERE, "tp_cases.npz"), **arrays)
    with open(os.path.join(HERE, "tp_cases.json"), "w") as f:
        json.dump(meta, f, separators=(",", ":"))
    print("wrote", sorted(os.listdir(HERE)))


def main_nn(ref="/root/reference"):
    """Node-wise blocks around the message: fixtures for the oracle's restatements in oracle/nn.py."""
    o3 = import_reference(ref)
    from e3nn import nn
    from e3nn.nn.models.v2106.points_convolution import Convolution

    g = torch.Generator().manual_seed(1234)
    rn = lambda *shape: torch.randn(*shape, generator=g)  # noqa: E731
    arrays, meta = {}, {}

    for name, (a, b, kw) in {
        "linear_mixed": ("4x0e+3x1o+2x0e", "5x0e+2x1o+3x1o+1x2e", {}),
        "linear_path_norm": ("4x0e+3x1o+2x0e", "5x0e+2x1o", {"path_normalization": "path"}),
        "linear_bias": ("6x0e+2x1e", "3x0e+2x1e+2x0e", {"biases": True}),
    }.items():
        lin = o3.Linear(a, b, **kw)
        if lin.bias_numel:
            with torch.no_grad():
                lin.bias.copy_(rn(lin.bias_numel))
        x = rn(7, lin.irreps_in.dim)
        arrays[name + "/x"], arrays[name + "/w"], arrays[name + "/out"] = x.numpy(), lin.weight.detach().numpy(), lin(x).detach().numpy()
        arrays[name + "/bias"] = lin.bias.detach().numpy()
        meta[name] = {"irreps_in": a, "irreps_out": b, "kwargs": kw, "weight_numel": lin.weight_numel,
                      "instructions": [[i.i_in, i.i_out, list(i.path_shape), i.path_weight] for i in lin.instructions]}  # fmt: skip

    acts = {"silu": torch.nn.functional.silu, "tanh": torch.tanh, "sigmoid": torch.sigmoid, "abs": torch.abs, "relu": torch.relu}
    from e3nn.math import normalize2mom
    meta["cst"] = {k: normalize2mom(f).cst for k, f in acts.items()}

    act = nn.Activation("5x0e+3x0o+2x1e+4x0o", [torch.nn.functional.silu, torch.tanh, None, torch.abs])
    x = rn(6, act.irreps_in.dim)
    arrays["activation/x"], arrays["activation/out"] = x.numpy(), act(x).numpy()
    meta["activation"] = {"irreps_in": str(act.irreps_in), "acts": ["silu", "tanh", None, "abs"], "irreps_out": str(act.irreps_out)}

    for name, (sc, a_s, ga, a_g, gd) in {
        "gate_plain": ("6x0e", ["silu"], "5x0e", ["sigmoid"], "3x1o+2x2e"),
        "gate_parity": ("4x0e+2x0o", ["silu", "tanh"], "3x0e+4x0o", ["sigmoid", "tanh"], "2x1o+3x1e+2x2e"),
        "gate_only_scalars": ("7x0e", ["relu"], "", [], ""),
    }.items():
        gate = nn.Gate(sc, [acts[k] for k in a_s], ga, [acts[k] for k in a_g], gd)
        x = rn(5, gate.irreps_in.dim)
        arrays[name + "/x"], arrays[name + "/out"] = x.numpy(), gate(x).numpy()
        meta[name] = {"args": [sc, a_s, ga, a_g, gd], "irreps_in": str(gate.irreps_in), "irreps_out": str(gate.irreps_out)}

    fc = nn.FullyConnectedNet([3, 16, 8, 5], torch.nn.functional.silu)
    x = rn(9, 3)
    arrays["fc/x"], arrays["fc/out"] = x.numpy(), fc(x).detach().numpy()
    for i in range(3):
        arrays[f"fc/w{i}"] = getattr(fc, f"layer{i}").weight.detach().numpy()
    meta["fc"] = {"hs": [3, 16, 8, 5], "act": "silu"}

    conv = Convolution("4x0e+3x1o+2x1e", "2x0e", "0e+1o+2e", "5x0e+2x1o+3x2e", [3, 8], 4.0)
    with torch.no_grad():
        conv.alpha.weight.copy_(rn(conv.alpha.weight_numel))  # the reference zero-initialises it: exercise the path
    N, E = 11, 40
    node_input, node_attr = rn(N, conv.irreps_node_input.dim), rn(N, 2)
    src, dst = torch.randint(0, N, (E,), generator=g), torch.randint(0, N, (E,), generator=g)
    vec = rn(E, 3)
    edge_attr = o3.spherical_harmonics([0, 1, 2], vec, True, "component")
    edge_scalars = rn(E, 3)
    out = conv(node_input, node_attr, src, dst, edge_attr, edge_scalars)
    for k, v in dict(node_input=node_input, node_attr=node_attr, src=src, dst=dst, edge_attr=edge_attr,
                     edge_scalars=edge_scalars, out=out.detach()).items():  # fmt: skip
        arrays["conv/" + k] = v.numpy()
    for k, v in conv.state_dict().items():
        if k.endswith("weight") and v.numel():
            arrays["conv/param/" + k] = v.numpy()
    meta["conv"] = {"args": ["4x0e+3x1o+2x1e", "2x0e", "0e+1o+2e", "5x0e+2x1o+3x2e", [3, 8], 4.0],
                    "irreps_mid": str(conv.tp.irreps_out), "tp_instructions": [[i.i_in1, i.i_in2, i.i_out] for i in conv.tp.instructions]}  # fmt: skip

    # (the module parameters above are drawn from the global generator, unseeded: a new run of this section writes
    # other, equally valid values for them; the committed files keep the values of the first run and gained the cases below)
    # gates whose scalars / gate scalars are not in simplified form: neighbouring entries of one irrep with different
    # activation functions, gated irreps given in pieces (drawn last, from a generator of their own, so that the cases
    # above keep their values)
    g2 = torch.Generator().manual_seed(1234)
    for name, (sc, a_s, ga, a_g, gd) in {
        "gate_entries_as_given": ("3x0e+2x0e+2x0o", ["silu", "relu", "tanh"], "2x0o+3x0o+1x0e", ["tanh", "abs", "sigmoid"], "1x2e+1x3o+3x1e+1x2o"),
        "gate_gated_in_pieces": ("", [], "4x0e+2x0e", ["sigmoid", "tanh"], "3x1e+1x1e+2x2o"),
    }.items():
        gate = nn.Gate(sc, [acts[k] for k in a_s], ga, [acts[k] for k in a_g], gd)
        x = torch.randn(5, gate.irreps_in.dim, generator=g2)
        arrays[name + "/x"], arrays[name + "/out"] = x.numpy(), gate(x).numpy()
        meta[name] = {"args": [sc, a_s, ga, a_g, gd], "irreps_in": str(gate.irreps_in), "irreps_out": str(gate.irreps_out)}

    np.savez_compressed(os.path.join(HERE, "nn_cases.npz"), **arrays)
    with open(os.path.join(HERE, "nn_cases.json"), "w") as f:
        json.dump(meta, f, separators=(",", ":"))
    print("wrote nn_cases", len(arrays), "arrays")


if __name__ == "__main__":
    if len(sys.argv) > 1 and sys.argv[1] == "state":
        main_state()
    elif len(sys.argv) > 1 and sys.argv[1] == "nn":
        main_nn(*sys.argv[2:])
    else:
        main()
