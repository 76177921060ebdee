"""Oracle: irreps strings -> layout.  TEST INFRASTRUCTURE ONLY.

Restates the part of the reference's ``Irreps`` algebra the hot path depends on
(reference: e3nn/o3/_irreps.py:56-83 parse of one irrep, :358-404 parse of a sum,
:434-448 slices, :229-241 selection rule, :542-568 simplify, :587-614 sort).
An irreps object here is a plain list of ``(mul, l, p)`` integer triples.
"""
from typing import List, Tuple

Irreps = List[Tuple[int, int, int]]


def parse_irrep(s: str) -> Tuple[int, int]:
    # reference _irreps.py:62-73: "<l><e|o|y>", y = parity of spherical harmonics
    s = s.strip()
    l = int(s[:-1])
    if l < 0:
        raise ValueError(s)
    p = {"e": 1, "o": -1, "y": (-1) ** l}[s[-1]]
    return l, p


def parse(irreps) -> Irreps:
    # reference _irreps.py:366-381: "mul x ir + mul x ir + ...", mul defaults to 1
    if not isinstance(irreps, str):
        return [tuple(int(v) for v in t) for t in irreps]
    out = []
    if irreps.strip() == "":
        return out
    for term in irreps.split("+"):
        if "x" in term:
            mul, ir = term.split("x")
            mul = int(mul)
        else:
            mul, ir = 1, term
        l, p = parse_irrep(ir)
        out.append((mul, l, p))
    return out


def dim(irreps: Irreps) -> int:
    # reference _irreps.py:705-707
    return sum(mul * (2 * l + 1) for mul, l, _ in irreps)


def slices(irreps: Irreps):
    # reference _irreps.py:434-448: blocks concatenated in order
    out, i = [], 0
    for mul, l, _ in irreps:
        out.append(slice(i, i + mul * (2 * l + 1)))
        i += mul * (2 * l + 1)
    return out


def product(ir1, ir2):
    # reference _irreps.py:229-241: |l1-l2| <= l <= l1+l2, parity multiplies
    (l1, p1), (l2, p2) = ir1, ir2
    return [(l, p1 * p2) for l in range(abs(l1 - l2), l1 + l2 + 1)]


def simplify(irreps: Irreps) -> Irreps:
    # reference _irreps.py:562-568: merge equal neighbours, drop zero multiplicities
    out = []
    for mul, l, p in irreps:
        if out and out[-1][1:] == (l, p):
            out[-1] = (out[-1][0] + mul, l, p)
        elif mul > 0:
            out.append((mul, l, p))
    return out


def sort(irreps: Irreps):
    """Returns (sorted irreps, p, inv); reference _irreps.py:608-614.

    Sort key is the tuple ((l, p), original index, mul): odd parity (-1) sorts before
    even (+1) at equal l and ties keep their original order.
    """
    keyed = sorted(((l, p), i, mul) for i, (mul, l, p) in enumerate(irreps))
    inv = tuple(i for _, i, _ in keyed)
    p = tuple(inv.index(i) for i in range(len(inv)))  # e3nn/math/perm.py:34-38
    return [(mul, l, pp) for (l, pp), _, mul in keyed], p, inv


def to_str(irreps: Irreps) -> str:
    return "+".join(f"{mul}x{l}{'e' if p == 1 else 'o'}" for mul, l, p in irreps)
