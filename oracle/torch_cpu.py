"""Timed CPU baseline: torch-CPU restatement of the reference's generated graph.

TEST / BENCHMARK INFRASTRUCTURE ONLY (the ``cpu_baseline`` leg of the benchmark and
parity tests).  It issues the same ATen calls the reference's fx graph does:
one ``torch.einsum`` per instruction with the specialised strings of
e3nn/o3/_tensor_product/_codegen.py:148-187, ``x[edge_src]`` + ``scatter_add_`` as in
e3nn/nn/models/v2106/points_convolution.py:13-17,105-106, and the elementwise
polynomial chain of e3nn/o3/_spherical_harmonics.py:93-112,193-249.
"""
import math
from math import sqrt

import torch

from . import irreps as ir_
from .wigner import wigner_3j


def tp_forward_torch(spec, x1, x2, w):
    """Same contraction order family as the reference graph; x1 [Z,d1], x2 [Z,d2]."""
    Z = x1.shape[0]
    i1, i2, io = spec.irreps_in1, spec.irreps_in2, spec.irreps_out
    s1, s2 = ir_.slices(i1), ir_.slices(i2)
    z = "" if spec.shared_weights else "z"
    if spec.weight_numel:
        w = w.reshape(-1, spec.weight_numel)
    per_out = [[] for _ in io]
    off = 0
    xx_cache = {}
    for t in [t for t in spec.instructions if 0 not in t.path_shape]:
        (m1, l1, _), (m2, l2, _), (mo, lo, _) = i1[t.i_in1], i2[t.i_in2], io[t.i_out]
        a = x1[:, s1[t.i_in1]].reshape(Z, m1, 2 * l1 + 1)
        b = x2[:, s2[t.i_in2]].reshape(Z, m2, 2 * l2 + 1)
        n = 1
        for s in t.path_shape:
            n *= s
        wt = w[:, off : off + n].reshape(((-1,) if z else ()) + tuple(t.path_shape))
        off += n
        tail = {"uvw": "w", "uvu": "u"}[t.mode]
        wi = {"uvw": "uvw", "uvu": "uv"}[t.mode]
        if (l1, l2, lo) == (0, 0, 0):
            r = torch.einsum(f"{z}{wi},zu,zv->z{tail}", wt, a.reshape(Z, m1), b.reshape(Z, m2))
        elif l1 == 0:
            r = torch.einsum(f"{z}{wi},zu,zvj->z{tail}j", wt, a.reshape(Z, m1), b) / sqrt(2 * lo + 1)
        elif l2 == 0:
            r = torch.einsum(f"{z}{wi},zui,zv->z{tail}i", wt, a, b.reshape(Z, m2)) / sqrt(2 * lo + 1)
        elif lo == 0:
            r = torch.einsum(f"{z}{wi},zui,zvi->z{tail}", wt, a, b) / sqrt(2 * l1 + 1)
        else:
            key = (t.i_in1, t.i_in2)
            if key not in xx_cache:
                xx_cache[key] = torch.einsum("zui,zvj->zuvij", a, b)
            C = torch.from_numpy(wigner_3j(l1, l2, lo)).to(x1.dtype)
            r = torch.einsum(f"{z}{wi},ijk,zuvij->z{tail}k", wt, C, xx_cache[key])
        per_out[t.i_out].append(t.path_weight * r.reshape(Z, -1))
    cols = []
    for c, (mul, l, _) in enumerate(io):
        if mul == 0:
            continue
        if per_out[c]:
            acc = per_out[c][0]
            for r in per_out[c][1:]:
                acc = acc + r
        else:
            acc = x1.new_zeros(Z, mul * (2 * l + 1))
        cols.append(acc)
    return torch.cat(cols, dim=1) if len(cols) > 1 else cols[0]


def scatter_torch(src, index, dim_size):
    out = src.new_zeros(dim_size, src.shape[1])
    return out.scatter_add_(0, index.reshape(-1, 1).expand_as(src), src)


def tp_gather_scatter_torch(spec, node_x, edge_attr, weight, edge_src, edge_dst, num_nodes):
    msg = tp_forward_torch(spec, node_x[edge_src], edge_attr, weight)
    return scatter_torch(msg, edge_dst.long(), num_nodes)


def spherical_harmonics_torch(lmax, xyz, normalize=True):
    """lmax <= 3, 'component' normalisation; op-for-op the reference's elementwise chain."""
    if normalize:
        xyz = torch.nn.functional.normalize(xyz, dim=-1)
    x, y, z = xyz[..., 0], xyz[..., 1], xyz[..., 2]
    out = [torch.ones_like(x)]
    if lmax >= 1:
        out += [math.sqrt(3) * x, math.sqrt(3) * y, math.sqrt(3) * z]
    if lmax >= 2:
        a20 = math.sqrt(15) * x * z
        y2 = y.pow(2)
        s = x.pow(2) + z.pow(2)
        a24 = 0.5 * math.sqrt(15) * (z.pow(2) - x.pow(2))
        out += [a20, math.sqrt(15) * x * y, math.sqrt(5) * (y2 - 0.5 * s), math.sqrt(15) * y * z, a24]
    if lmax >= 3:
        c0, c2 = math.sqrt(42) / 6, math.sqrt(168) / 8
        out += [
            c0 * (a20 * z + a24 * x),
            math.sqrt(7) * a20 * y,
            c2 * (4.0 * y2 - s) * x,
            0.5 * math.sqrt(7) * y * (2.0 * y2 - 3.0 * s),
            c2 * z * (4.0 * y2 - s),
            math.sqrt(7) * a24 * y,
            c0 * (a24 * z - a20 * x),
        ]
    return torch.stack(out, dim=-1)
