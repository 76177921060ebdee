"""Oracle: cartesian real spherical harmonics.  TEST INFRASTRUCTURE ONLY.

Follows reference e3nn/o3/_spherical_harmonics.py:93-112 (normalise input, evaluate
the polynomial up to lmax, select the requested l blocks, apply the output
normalisation).  Polynomials: l <= 3 are the closed forms of :194-226; every l is also
available through the recurrence the reference's generator used to print that file
(e3nn/o3/_spherical_harmonics_generator.py:57-65):
    Y^{l+1}_i = c_l * sum_{k,j} w3j(l+1, 1, l)[i, k, j] * x_k * Y^l_j ,
with c_l > 0 fixed by |Y^{l+1}(0,1,0)|^2 = 2l+3 ("component" normalisation).
"""
import math

import numpy as np

from .wigner import wigner_3j


def _closed_form(lmax, x, y, z):
    # reference :194-226, restated
    out = [np.ones_like(x)]
    if lmax >= 1:
        r3 = math.sqrt(3.0)
        out += [r3 * x, r3 * y, r3 * z]
    if lmax >= 2:
        r15, r5 = math.sqrt(15.0), math.sqrt(5.0)
        s = x * x + z * z
        y2 = y * y
        a20 = r15 * x * z
        a24 = 0.5 * r15 * (z * z - x * x)
        out += [a20, r15 * x * y, r5 * (y2 - 0.5 * s), r15 * y * z, a24]
    if lmax >= 3:
        r7 = math.sqrt(7.0)
        c0 = math.sqrt(42.0) / 6.0
        c2 = math.sqrt(168.0) / 8.0
        out += [
            c0 * (a20 * z + a24 * x),
            r7 * a20 * y,
            c2 * (4.0 * y2 - s) * x,
            0.5 * r7 * y * (2.0 * y2 - 3.0 * s),
            c2 * z * (4.0 * y2 - s),
            r7 * a24 * y,
            c0 * (a24 * z - a20 * x),
        ]
    return out


def _recurrence_constants(lmax):
    """c_l for l = 0..lmax-1, evaluated at the pole (0, 1, 0) like the generator."""
    pole = np.array([0.0, 1.0, 0.0])
    y = np.ones(1)
    cs = []
    for l in range(lmax):
        raw = np.einsum("ikj,k,j->i", wigner_3j(l + 1, 1, l), pole, y)
        c = math.sqrt(2 * l + 3) / np.linalg.norm(raw)
        cs.append(c)
        y = c * raw
    return cs


def sh_polynomials(lmax, xyz, use_recurrence=False):
    """[..., (lmax+1)^2] component-normalised polynomials of the (un-normalised) input."""
    xyz = np.asarray(xyz, dtype=np.float64)
    x, y, z = xyz[..., 0], xyz[..., 1], xyz[..., 2]
    if not use_recurrence and lmax <= 3:
        return np.stack(_closed_form(lmax, x, y, z), axis=-1)
    cs = _recurrence_constants(lmax)
    blocks = [np.ones(xyz.shape[:-1] + (1,))]
    for l in range(lmax):
        nxt = cs[l] * np.einsum("ikj,...k,...j->...i", wigner_3j(l + 1, 1, l), xyz, blocks[-1])
        blocks.append(nxt)
    return np.concatenate(blocks, axis=-1)


def spherical_harmonics(ls, xyz, normalize, normalization="integral", use_recurrence=False):
    """ls: int or list of int.  Mirrors reference :115-117 / :93-112."""
    ls = [ls] if isinstance(ls, int) else list(ls)
    xyz = np.asarray(xyz, dtype=np.float64)
    if normalize:
        # torch.nn.functional.normalize: x / max(|x|, 1e-12)  (reference :96)
        n = np.sqrt((xyz * xyz).sum(-1, keepdims=True))
        xyz = xyz / np.maximum(n, 1e-12)
    lmax = max(ls)
    sh = sh_polynomials(lmax, xyz, use_recurrence)
    if ls != list(range(lmax + 1)):
        sh = np.concatenate([sh[..., l * l : (l + 1) * (l + 1)] for l in ls], axis=-1)  # :100-101
    if normalization == "integral":
        sh = sh / math.sqrt(4 * math.pi)  # :103-104
    elif normalization == "norm":
        sh = sh / np.concatenate([math.sqrt(2 * l + 1) * np.ones(2 * l + 1) for l in ls])  # :105-110
    else:
        assert normalization == "component"
    return sh
