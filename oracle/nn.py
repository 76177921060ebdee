"""Oracle: the node-wise blocks either side of the message.  TEST INFRASTRUCTURE ONLY.

numpy (fp64) restatements of

* ``o3.Linear``               reference e3nn/o3/_linear.py:133-165 (instructions, alpha^(-1/2)), :348-498 (the einsum
                              "uw,zui->zwi" per path, biases added to scalar outputs)
* ``normalize2mom``           reference e3nn/math/_normalize_activation.py:9-19,42-57
* ``nn.Activation``           reference e3nn/nn/_activation.py:33-104
* ``nn.Gate``                 reference e3nn/nn/_gate.py:8-24 (sorted, simplified input), :103-144
                              (+ ElementwiseTensorProduct pairing, e3nn/o3/_tensor_product/_sub.py:115-142)
* ``nn.FullyConnectedNet``    reference e3nn/nn/_fc.py:38-48,70-88
* v2106 ``Convolution``       reference e3nn/nn/models/v2106/points_convolution.py:56-113

Pin status: every function here is pinned by golden outputs written from the reference (tests/golden/nn_cases.*), and
Linear additionally by its closed form on scalars (W^T x / sqrt(fan_in)).
"""
import numpy as np
import torch

from . import irreps as ir_
from . import message_passing as mp_
from . import tensor_product as tp_

ACTS = {
    "silu": lambda x: x / (1.0 + np.exp(-x)),
    "tanh": np.tanh,
    "sigmoid": lambda x: 1.0 / (1.0 + np.exp(-x)),
    "abs": np.abs,
    "relu": lambda x: np.maximum(x, 0.0),
}
_PARITY = {"silu": 0, "tanh": -1, "sigmoid": 0, "abs": 1, "relu": 0}
_TORCH = {"silu": torch.nn.functional.silu, "tanh": torch.tanh, "sigmoid": torch.sigmoid, "abs": torch.abs, "relu": torch.relu}


def normalize2mom_const(name):
    # _normalize_activation.py:9-19: second moment over 1e6 normal samples from a torch generator seeded with 0
    # (the sample stream is torch's, so torch draws it); :42-48 snaps constants within 1e-4 of 1 to the identity
    gen = torch.Generator(device="cpu").manual_seed(0)
    z = torch.randn(1_000_000, generator=gen, dtype=torch.float64)
    cst = float(_TORCH[name](z).pow(2).mean().pow(-0.5))
    return 1.0 if abs(cst - 1) < 1e-4 else cst


def linear_instructions(irreps_in, irreps_out, instructions=None, path_normalization="element"):
    i_in, i_out = ir_.parse(irreps_in), ir_.parse(irreps_out)
    if instructions is None:  # _linear.py:133-140
        instructions = [(a, b) for a, ta in enumerate(i_in) for b, tb in enumerate(i_out) if ta[1:] == tb[1:]]
    out = []
    for a, b in instructions:  # _linear.py:152-165
        x = sum(i_in[a2 if path_normalization == "element" else a][0] for a2, b2 in instructions if b2 == b)
        out.append((a, b, (i_in[a][0], i_out[b][0]), (1.0 if x == 0 else x) ** -0.5))
    return out


def linear_forward(irreps_in, irreps_out, x, w, instructions=None, path_normalization="element", bias=None, biases=None):
    i_in, i_out = ir_.parse(irreps_in), ir_.parse(irreps_out)
    ins = linear_instructions(i_in, i_out, instructions, path_normalization)
    sl_in, sl_out = ir_.slices(i_in), ir_.slices(i_out)
    x = np.asarray(x, np.float64)
    out = np.zeros(x.shape[:-1] + (ir_.dim(i_out),))
    off = 0
    for a, b, (u, wn), pw in ins:
        d = 2 * i_in[a][1] + 1
        W = np.asarray(w[off : off + u * wn], np.float64).reshape(u, wn)
        off += u * wn
        xa = x[..., sl_in[a]].reshape(x.shape[:-1] + (u, d))
        out[..., sl_out[b]] += pw * np.einsum("uw,...ui->...wi", W, xa).reshape(x.shape[:-1] + (wn * d,))
    if biases:  # _linear.py:176-188: one bias per channel of the flagged scalar outputs, in output order
        boff = 0
        for flag, sl in zip(biases, sl_out):
            if flag:
                n = sl.stop - sl.start
                out[..., sl] += np.asarray(bias[boff : boff + n], np.float64)
                boff += n
    return out


def activation_forward(irreps_in, acts, x):
    """acts: one name or None per irrep.  Returns (out, irreps_out)."""
    i_in = ir_.parse(irreps_in)
    x = np.asarray(x, np.float64)
    out = x.copy()
    irreps_out = []
    for (mul, l, p), sl, name in zip(i_in, ir_.slices(i_in), acts):
        if name is None:
            irreps_out.append((mul, l, p))
            continue
        assert l == 0
        p_out = _PARITY[name] if p == -1 else p  # _activation.py:49-59
        assert p_out != 0
        irreps_out.append((mul, 0, p_out))
        out[..., sl] = normalize2mom_const(name) * ACTS[name](x[..., sl])
    return out, irreps_out


def gate_forward(irreps_scalars, act_scalars, irreps_gates, act_gates, irreps_gated, x):
    """Returns (out, irreps_in, irreps_out) with the reference's sorted + simplified input layout."""
    given = [ir_.parse(g) for g in (irreps_scalars, irreps_gates, irreps_gated)]
    groups = [ir_.simplify(g) for g in given]  # _gate.py:14: the cut is made on the simplified groups ...
    cat = [t for g in groups for t in g]
    srt, p, _ = ir_.sort(cat)  # _gate.py:19-22
    sl = ir_.slices(srt)
    x = np.asarray(x, np.float64)
    parts, pos = [], 0
    for g in groups:  # Extract (_gate.py:22): entry i of the concatenation sits at sorted position p[i]
        cols = [x[..., sl[p[pos + i]]] for i in range(len(g))]
        parts.append(np.concatenate(cols, axis=-1) if cols else np.zeros(x.shape[:-1] + (0,)))
        pos += len(g)
    # ... and the activations act on the irreps as given (_gate.py:108-112): same columns, possibly more entries
    scalars, out_s = activation_forward([t for t in given[0] if t[0]], [a for t, a in zip(given[0], act_scalars) if t[0]], parts[0])
    gates, out_g = activation_forward([t for t in given[1] if t[0]], [a for t, a in zip(given[1], act_gates) if t[0]], parts[1])
    # ElementwiseTensorProduct(gated, gates): copy u of the gated irreps times gate scalar u; component
    # normalisation makes the factor exactly 1 (sqrt(2l+1) * delta / sqrt(2l+1))
    gated_cols, out_gated = [], []
    gate_par = [pp for mul, _, pp in out_g for _ in range(mul)]
    u = 0
    col = 0
    for mul, l, pp in groups[2]:
        d = 2 * l + 1
        blk = parts[2][..., col : col + mul * d].reshape(x.shape[:-1] + (mul, d))
        gated_cols.append((blk * gates[..., u : u + mul, None]).reshape(x.shape[:-1] + (mul * d,)))
        run = 0  # output irreps: runs split where the gate parity changes (_sub.py:118-142)
        for k in range(mul):
            if k + 1 == mul or gate_par[u + k + 1] != gate_par[u + k]:
                out_gated.append((k + 1 - run, l, pp * gate_par[u + k]))
                run = k + 1
        u += mul
        col += mul * d
    out = np.concatenate([scalars] + gated_cols, axis=-1)
    return out, ir_.simplify(srt), out_s + out_gated


def fc_forward(weights, x, act="silu", variance_in=1, variance_out=1, out_act=False):
    # _fc.py:70-88 (layer list) and :38-48 (one layer)
    x = np.asarray(x, np.float64)
    cst = normalize2mom_const(act) if act is not None else 1.0
    var_in = variance_in
    n = len(weights)
    for i, W in enumerate(weights):
        W = np.asarray(W, np.float64)
        last = i == n - 1
        var_out = variance_out if last else 1
        a = act if (not last or out_act) else None
        if a is not None:
            x = x @ (W / (W.shape[0] * var_in) ** 0.5)
            x = cst * ACTS[a](x) * var_out**0.5
        else:
            x = x @ (W / (W.shape[0] * var_in / var_out) ** 0.5)
        var_in = var_out
    return x


def _fctp(irreps_in1, irreps_in2, irreps_out, x1, x2, w):
    spec = tp_.make_spec(irreps_in1, irreps_in2, irreps_out, tp_.fully_connected_instructions(irreps_in1, irreps_in2, irreps_out))
    return tp_.tp_forward(spec, x1, x2, w), spec


def convolution_forward(irreps_node_input, irreps_node_attr, irreps_edge_attr, irreps_node_output, num_neighbors, params,
                        node_input, node_attr, edge_src, edge_dst, edge_attr, edge_scalars):
    """params: 'sc.weight', 'lin1.weight', 'lin2.weight', 'alpha.weight', 'fc.layer{i}.weight'."""
    i_in, i_out = ir_.parse(irreps_node_input), ir_.parse(irreps_node_output)
    N = np.asarray(node_input).shape[0]
    n_fc = len([k for k in params if k.startswith("fc.layer")])
    weight = fc_forward([params[f"fc.layer{i}.weight"] for i in range(n_fc)], edge_scalars, "silu")  # :86,100
    sc, sc_spec = _fctp(i_in, irreps_node_attr, i_out, node_input, node_attr, params["sc.weight"])  # :56,102
    x, _ = _fctp(i_in, irreps_node_attr, i_in, node_input, node_attr, params["lin1.weight"])  # :58,103
    outs = {(l, p) for _, l, p in i_out} | {(0, 1)}
    mid, ins = tp_.convolution_instructions(i_in, irreps_edge_attr, lambda l, p: (l, p) in outs)  # :60-76
    spec = tp_.make_spec(i_in, irreps_edge_attr, mid, ins, shared_weights=False)
    x = mp_.tp_gather_scatter(spec, x, edge_attr, weight, edge_src, edge_dst, N) / num_neighbors**0.5  # :105-106
    conv, _ = _fctp(mid, irreps_node_attr, i_out, x, node_attr, params["lin2.weight"])  # :89,108
    alpha, _ = _fctp(mid, irreps_node_attr, "0e", x, node_attr, params["alpha.weight"])  # :92,109
    m = tp_.output_mask(sc_spec)  # :111-113
    alpha = (1 - m) + alpha * m
    return sc + alpha * conv
