"""Oracle: rotation matrices of the irreps, for equivariance tests.  TEST INFRASTRUCTURE ONLY.

The reference builds Wigner D matrices from generators and Euler angles
(e3nn/o3/_wigner.py:62-99, e3nn/o3/_irreps.py:116-200).  Here D^l(R) is obtained from the
defining property the reference tests (tests/o3/cartesian_spherical_harmonics_test.py:51-59):
    Y^l(R x) = D^l(R) Y^l(x)   for all x,
solved in the least-squares sense over a set of sample directions with the oracle's own
spherical harmonics.  Parity: an improper R = -Q acts on an irrep (l, p) as p * D^l(Q).
"""
import numpy as np

from . import irreps as ir_
from .spherical_harmonics import spherical_harmonics


def random_rotation(rng):
    q, r = np.linalg.qr(rng.standard_normal((3, 3)))
    q = q * np.sign(np.diag(r))
    if np.linalg.det(q) < 0:
        q[:, 0] = -q[:, 0]
    return q


def wigner_D(l, R, n_samples=64, seed=0):
    """[2l+1, 2l+1] matrix with Y^l(x @ R.T) = Y^l(x) @ D.T for a proper rotation R."""
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((max(n_samples, 4 * (2 * l + 1)), 3))
    x /= np.linalg.norm(x, axis=1, keepdims=True)
    y = spherical_harmonics(l, x, False, "component", use_recurrence=l > 3)
    yr = spherical_harmonics(l, x @ R.T, False, "component", use_recurrence=l > 3)
    dt, res, rank, _ = np.linalg.lstsq(y, yr, rcond=None)
    assert rank == 2 * l + 1
    return dt.T


def irreps_D(irreps, R, improper=False):
    """Block-diagonal representation matrix of `irreps` (string or list) for rotation R (times inversion)."""
    irreps = ir_.parse(irreps)
    n = ir_.dim(irreps)
    D = np.zeros((n, n))
    i = 0
    cache = {}
    for mul, l, p in irreps:
        if l not in cache:
            cache[l] = wigner_D(l, R)
        d = cache[l] * (p if improper else 1)
        for _ in range(mul):
            D[i : i + 2 * l + 1, i : i + 2 * l + 1] = d
            i += 2 * l + 1
    return D
