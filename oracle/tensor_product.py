"""Oracle: TensorProduct construction + forward.  TEST INFRASTRUCTURE ONLY.

Restates
* instruction parsing and path normalisation, reference
  e3nn/o3/_tensor_product/_tensor_product.py:236-324;
* weight bookkeeping (:403) and output_mask (:412-428);
* the per-instruction contraction of e3nn/o3/_tensor_product/_codegen.py:107-343 in
  its generic (non-specialised) form.  The reference's l = 0 / (1,1,1) special cases
  (:150-163, :169-182) substitute delta/sqrt(dim) and epsilon/sqrt(6) for the same
  Wigner tensor, so the generic form is numerically the same map;
* the instruction lists of FullyConnectedTensorProduct (e3nn/o3/_tensor_product/_sub.py:53-59)
  and of the message-passing call site (e3nn/nn/models/v2106/points_convolution.py:60-76).
"""
from collections import namedtuple
from math import sqrt

import numpy as np

from . import irreps as ir_
from .wigner import wigner_3j

Instruction = namedtuple("Instruction", "i_in1 i_in2 i_out mode has_weight path_weight path_shape")
Spec = namedtuple("Spec", "irreps_in1 irreps_in2 irreps_out instructions weight_numel shared_weights")

MODES = ("uvw", "uvu", "uvv", "uuw", "uuu", "uvuv", "uvu<v", "u<vw")


def _path_shape(mode, m1, m2, mo):
    # reference _tensor_product.py:245-254
    return {
        "uvw": (m1, m2, mo),
        "uvu": (m1, m2),
        "uvv": (m1, m2),
        "uuw": (m1, mo),
        "uuu": (m1,),
        "uvuv": (m1, m2),
        "uvu<v": (m1 * (m2 - 1) // 2,),
        "u<vw": (m1 * (m2 - 1) // 2, mo),
    }[mode]


def _num_elements(mode, m1, m2):
    # reference _tensor_product.py:277-287
    return {
        "uvw": m1 * m2,
        "uvu": m2,
        "uvv": m1,
        "uuw": m1,
        "uuu": 1,
        "uvuv": 1,
        "uvu<v": 1,
        "u<vw": m1 * (m2 - 1) // 2,
    }[mode]


def make_spec(
    irreps_in1,
    irreps_in2,
    irreps_out,
    instructions,
    in1_var=None,
    in2_var=None,
    out_var=None,
    irrep_normalization="component",
    path_normalization="element",
    shared_weights=True,
):
    i1, i2, io = ir_.parse(irreps_in1), ir_.parse(irreps_in2), ir_.parse(irreps_out)
    in1_var = [1.0] * len(i1) if in1_var is None else [float(v) for v in in1_var]
    in2_var = [1.0] * len(i2) if in2_var is None else [float(v) for v in in2_var]
    out_var = [1.0] * len(io) if out_var is None else [float(v) for v in out_var]
    raw = [tuple(t) if len(t) == 6 else tuple(t) + (1.0,) for t in instructions]  # :236
    for a, b, c, mode, _, _ in raw:
        assert mode in MODES
        assert i1[a][2] * i2[b][2] == io[c][2]
        assert abs(i1[a][1] - i2[b][1]) <= io[c][1] <= i1[a][1] + i2[b][1]
    out = []
    for a, b, c, mode, has_w, pw in raw:
        l1, l2, lo = i1[a][1], i2[b][1], io[c][1]
        # :298-303
        alpha = {"component": 2 * lo + 1, "norm": (2 * l1 + 1) * (2 * l2 + 1), "none": 1}[irrep_normalization]
        # :305-311
        if path_normalization == "element":
            x = sum(
                in1_var[a2] * in2_var[b2] * _num_elements(m2_, i1[a2][0], i2[b2][0])
                for a2, b2, c2, m2_, _, _ in raw
                if c2 == c
            )
        elif path_normalization == "path":
            x = in1_var[a] * in2_var[b] * _num_elements(mode, i1[a][0], i2[b][0])
            x *= len([1 for t in raw if t[2] == c])
        else:
            x = 1
        if x > 0.0:
            alpha /= x
        alpha *= out_var[c]
        alpha *= pw
        out.append(Instruction(a, b, c, mode, bool(has_w), sqrt(alpha), _path_shape(mode, i1[a][0], i2[b][0], io[c][0])))
    wn = sum(int(np.prod(t.path_shape)) for t in out if t.has_weight)  # :403
    return Spec(i1, i2, io, out, wn, shared_weights)


def fully_connected_instructions(irreps_in1, irreps_in2, irreps_out):
    # reference _sub.py:53-59: loop order in1 -> in2 -> out
    i1, i2, io = ir_.parse(irreps_in1), ir_.parse(irreps_in2), ir_.parse(irreps_out)
    return [
        (a, b, c, "uvw", True, 1.0)
        for a, (_, l1, p1) in enumerate(i1)
        for b, (_, l2, p2) in enumerate(i2)
        for c, (_, lo, po) in enumerate(io)
        if (lo, po) in ir_.product((l1, p1), (l2, p2))
    ]


def convolution_instructions(irreps_node_input, irreps_edge_attr, keep):
    """uvu instruction list + sorted per-path output irreps of the message TP.

    reference points_convolution.py:60-76; ``keep(l, p)`` plays the role of the
    ``ir_out in irreps_node_output or ir_out == 0e`` filter (:64).
    """
    i1, i2 = ir_.parse(irreps_node_input), ir_.parse(irreps_edge_attr)
    mid, ins = [], []
    for a, (mul, l1, p1) in enumerate(i1):
        for b, (_, l2, p2) in enumerate(i2):
            for lo, po in ir_.product((l1, p1), (l2, p2)):
                if keep(lo, po):
                    ins.append((a, b, len(mid), "uvu", True))
                    mid.append((mul, lo, po))
    mid_sorted, p, _ = ir_.sort(mid)
    ins = [(a, b, p[c], mode, tr) for a, b, c, mode, tr in ins]
    return mid_sorted, ins


def output_mask(spec):
    # reference _tensor_product.py:412-428
    parts = []
    for c, (mul, l, _) in enumerate(spec.irreps_out):
        hit = any(t.i_out == c and t.path_weight != 0 and 0 not in t.path_shape for t in spec.instructions)
        parts.append(np.full(mul * (2 * l + 1), 1.0 if hit else 0.0))
    return np.concatenate(parts) if parts else np.ones(0)


def tp_forward(spec, x1, x2, w=None, dtype=np.float64):
    """out[Z, dim_out] for x1[Z, dim1], x2[Z, dim2]; w is [weight_numel] (shared) or [Z, weight_numel]."""
    x1 = np.asarray(x1, dtype=dtype)
    x2 = np.asarray(x2, dtype=dtype)
    Z = x1.shape[0]
    i1, i2, io = spec.irreps_in1, spec.irreps_in2, spec.irreps_out
    s1, s2, so = ir_.slices(i1), ir_.slices(i2), ir_.slices(io)
    out = np.zeros((Z, ir_.dim(io)), dtype=dtype)
    if w is not None:
        w = np.asarray(w, dtype=dtype)
        w = w.reshape(-1, spec.weight_numel) if spec.weight_numel else w
    z = "" if spec.shared_weights else "z"
    off = 0
    # instructions with an empty path are dropped before offsets are counted (_codegen.py:51)
    for t in [t for t in spec.instructions if 0 not in t.path_shape]:
        (m1, l1, _), (m2, l2, _), (mo, lo, _) = i1[t.i_in1], i2[t.i_in2], io[t.i_out]
        if t.has_weight:
            n = int(np.prod(t.path_shape))
            wt = w[:, off : off + n].reshape(((-1,) if z else ()) + t.path_shape)
            if not z:
                wt = wt.reshape(t.path_shape)
            off += n
        if m1 * (2 * l1 + 1) == 0 or m2 * (2 * l2 + 1) == 0 or mo * (2 * lo + 1) == 0:
            continue
        a = x1[:, s1[t.i_in1]].reshape(Z, m1, 2 * l1 + 1)
        b = x2[:, s2[t.i_in2]].reshape(Z, m2, 2 * l2 + 1)
        C = wigner_3j(l1, l2, lo).astype(dtype)
        mode = t.mode
        if mode in ("uuw", "uuu"):
            xx = np.einsum("zui,zuj->zuij", a, b)
        else:
            xx = np.einsum("zui,zvj->zuvij", a, b)
        if mode in ("uvu<v", "u<vw"):
            iu = np.triu_indices(m1, 1)  # _codegen.py:291-295
            xx = xx[:, iu[0], iu[1]]
        if t.has_weight:
            expr = {
                "uvw": f"{z}uvw,ijk,zuvij->zwk",
                "uvu": f"{z}uv,ijk,zuvij->zuk",
                "uvv": f"{z}uv,ijk,zuvij->zvk",
                "uuw": f"{z}uw,ijk,zuij->zwk",
                "uuu": f"{z}u,ijk,zuij->zuk",
                "uvuv": f"{z}uv,ijk,zuvij->zuvk",
                "uvu<v": f"{z}w,ijk,zwij->zwk",
                "u<vw": f"{z}qw,ijk,zqij->zwk",
            }[mode]
            r = np.einsum(expr, wt, C, xx, optimize=True)
        else:
            expr = {
                "uvu": "ijk,zuvij->zuk",
                "uvv": "ijk,zuvij->zvk",
                "uuw": "ijk,zuij->zk",
                "uuu": "ijk,zuij->zuk",
                "uvuv": "ijk,zuvij->zuvk",
                "uvu<v": "ijk,zwij->zwk",
            }[mode]
            r = np.einsum(expr, C, xx)
        out[:, so[t.i_out]] += t.path_weight * r.reshape(Z, -1)  # :312-314, :328-336
    return out


def tp_forward_loops(spec, x1, x2, w=None):
    """Brute-force scalar loops for the ``uvu`` and ``uvw`` modes (tiny inputs only)."""
    x1 = np.asarray(x1, dtype=np.float64)
    x2 = np.asarray(x2, dtype=np.float64)
    Z = x1.shape[0]
    i1, i2, io = spec.irreps_in1, spec.irreps_in2, spec.irreps_out
    s1, s2, so = ir_.slices(i1), ir_.slices(i2), ir_.slices(io)
    out = np.zeros((Z, ir_.dim(io)))
    w = None if w is None else np.asarray(w, dtype=np.float64).reshape(-1, spec.weight_numel)
    off = 0
    for t in spec.instructions:
        (m1, l1, _), (m2, l2, _), (mo, lo, _) = i1[t.i_in1], i2[t.i_in2], io[t.i_out]
        d1, d2, d3 = 2 * l1 + 1, 2 * l2 + 1, 2 * lo + 1
        C = wigner_3j(l1, l2, lo)
        assert t.mode in ("uvu", "uvw") and t.has_weight
        for z in range(Z):
            wz = w[0 if spec.shared_weights else z]
            for u in range(m1):
                for v in range(m2):
                    for k in range(d3):
                        s = 0.0
                        for i in range(d1):
                            for j in range(d2):
                                s += C[i, j, k] * x1[z, s1[t.i_in1].start + u * d1 + i] * x2[z, s2[t.i_in2].start + v * d2 + j]
                        if t.mode == "uvu":
                            out[z, so[t.i_out].start + u * d3 + k] += t.path_weight * wz[off + u * m2 + v] * s
                        else:
                            for ww in range(mo):
                                out[z, so[t.i_out].start + ww * d3 + k] += (
                                    t.path_weight * wz[off + (u * m2 + v) * mo + ww] * s
                                )
        off += int(np.prod(t.path_shape))
    return out
