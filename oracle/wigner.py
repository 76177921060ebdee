"""Oracle: real-basis Wigner 3j tensors.  TEST INFRASTRUCTURE ONLY.

Follows reference e3nn/o3/_wigner.py:102-164 (wigner_3j -> _so3_clebsch_gordan):
Condon-Shortley SU(2) Clebsch-Gordan coefficients in exact rational arithmetic
(:203-286 uses an equivalent Racah sum), rotated to the real basis with the matrix of
:30-51, real part taken and the whole tensor scaled to Frobenius norm 1 (:159-163).
"""
from fractions import Fraction
from functools import lru_cache
from math import factorial

import numpy as np


def _cg_squared_and_sum(j1, m1, j2, m2, j3, m3):
    """<j1 m1 j2 m2 | j3 m3> = sqrt(pref) * s, both returned exactly (textbook Racah form)."""
    if m3 != m1 + m2 or not (abs(j1 - j2) <= j3 <= j1 + j2):
        return Fraction(0), 0
    f = factorial
    pref = Fraction(
        (2 * j3 + 1) * f(j3 + j1 - j2) * f(j3 - j1 + j2) * f(j1 + j2 - j3), f(j1 + j2 + j3 + 1)
    ) * (f(j3 + m3) * f(j3 - m3) * f(j1 - m1) * f(j1 + m1) * f(j2 - m2) * f(j2 + m2))
    s = Fraction(0)
    for k in range(0, j1 + j2 - j3 + 1):
        args = (k, j1 + j2 - j3 - k, j1 - m1 - k, j2 + m2 - k, j3 - j2 + m1 + k, j3 - j1 - m2 + k)
        if min(args) < 0:
            continue
        d = 1
        for a in args:
            d *= f(a)
        s += Fraction((-1) ** k, d)
    return pref, s


@lru_cache(maxsize=None)
def su2_clebsch_gordan(j1: int, j2: int, j3: int) -> np.ndarray:
    """[2j1+1, 2j2+1, 2j3+1] array indexed by (j1+m1, j2+m2, j3+m3); reference :203-229."""
    out = np.zeros((2 * j1 + 1, 2 * j2 + 1, 2 * j3 + 1))
    for m1 in range(-j1, j1 + 1):
        for m2 in range(-j2, j2 + 1):
            m3 = m1 + m2
            if abs(m3) > j3:
                continue
            pref, s = _cg_squared_and_sum(j1, m1, j2, m2, j3, m3)
            out[j1 + m1, j2 + m2, j3 + m3] = float(pref) ** 0.5 * float(s)
    return out


def real_to_complex(l: int) -> np.ndarray:
    """Unitary taking real-basis components to complex ones; reference :30-41."""
    q = np.zeros((2 * l + 1, 2 * l + 1), dtype=np.complex128)
    r = 2 ** -0.5
    for m in range(1, l + 1):
        q[l - m, l + m] = r
        q[l - m, l - m] = -1j * r
        q[l + m, l + m] = (-1) ** m * r
        q[l + m, l - m] = 1j * (-1) ** m * r
    q[l, l] = 1
    return (-1j) ** l * q


@lru_cache(maxsize=None)
def _wigner_3j_cached(l1: int, l2: int, l3: int) -> np.ndarray:
    q1, q2, q3 = real_to_complex(l1), real_to_complex(l2), real_to_complex(l3)
    c = su2_clebsch_gordan(l1, l2, l3).astype(np.complex128)
    c = np.einsum("ij,kl,mn,ikn->jlm", q1, q2, np.conj(q3.T), c)  # reference :155
    assert np.abs(c.imag).max() < 1e-9
    c = c.real
    return c / np.linalg.norm(c)


def wigner_3j(l1: int, l2: int, l3: int) -> np.ndarray:
    """Real tensor C[2l1+1, 2l2+1, 2l3+1], invariant under D(l1) x D(l2) x D(l3), |C| = 1."""
    assert abs(l2 - l3) <= l1 <= l2 + l3
    return _wigner_3j_cached(l1, l2, l3).copy()
