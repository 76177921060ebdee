"""Irreducible representations of O(3) and direct sums of them.

Public behaviour of the reference's ``e3nn.o3.Irrep`` / ``e3nn.o3.Irreps``
(e3nn/o3/_irreps.py:14-264, :301-806) for everything the tensor-product hot path
needs: the string grammar, the feature layout (``dim``, ``slices``), the selection rule
``ir1 * ir2``, ``sort`` / ``simplify`` / ``regroup`` / ``filter`` and ``randn``.  The
rotation-matrix constructors (``D_from_*``) are not part of the hot path and are not provided.

Grammar:  irreps := term ("+" term)* | ""      term := [mul "x"] irrep      irrep := l ("e" | "o" | "y")
where "y" is the parity of the spherical harmonics, (-1)^l.
"""
import itertools
import re
from collections import namedtuple
from typing import List, Union

import torch

_IRREP_NAME = re.compile(r"\s*(\d+)\s*([eoy])\s*")
_TERM = re.compile(r"\s*(?:(\d+)\s*x)?\s*(\d+\s*[eoy])\s*")
_SortResult = namedtuple("sort", ["irreps", "p", "inv"])


def _parse_irrep_name(text: str):
    m = _IRREP_NAME.fullmatch(text)
    if m is None:
        raise ValueError(f'unable to convert string "{text.strip()}" into an Irrep')
    degree = int(m.group(1))
    parity = {"e": 1, "o": -1, "y": -1 if degree % 2 else 1}[m.group(2)]
    return degree, parity


def _not_a_sequence(self, *_args):
    # Irrep and (mul, irrep) pairs are tuples only for hashing, ordering and unpacking
    raise NotImplementedError


class Irrep(tuple):
    """Irreducible representation ``(l, p)``; ``Irrep("1o")``, ``Irrep(2, 1)``, ``Irrep("3y")``.

    Ordered as the pair ``(l, p)``: at equal ``l`` the odd irrep comes first."""

    def __new__(cls, l, p=None):
        if p is None:  # one argument: an Irrep, a (mul, irrep) pair of an Irreps, a name, or an (l, p) pair
            if type(l) is Irrep:
                return l
            if type(l) is _MulIr:
                return l[1]
            l, p = _parse_irrep_name(l) if isinstance(l, str) else tuple(l)
        if isinstance(l, bool) or not isinstance(l, int) or l < 0:
            raise ValueError(f"the degree l must be a non-negative integer, got {l!r}")
        if p != 1 and p != -1:
            raise ValueError(f"the parity p must be 1 or -1, got {p!r}")
        return tuple.__new__(cls, (l, int(p)))

    l = property(lambda self: self[0], doc="degree")  # noqa: E741
    p = property(lambda self: self[1], doc="parity, 1 (even) or -1 (odd)")
    dim = property(lambda self: 2 * self[0] + 1, doc="dimension 2l + 1")

    def is_scalar(self) -> bool:
        return self == (0, 1)

    def __repr__(self) -> str:
        return f"{self[0]}{'o' if self[1] < 0 else 'e'}"

    @classmethod
    def iterator(cls, lmax=None):
        """0e, 0o, 1o, 1e, 2e, 2o, ...: for every l the parity of the spherical harmonics first."""
        degrees = itertools.count() if lmax is None else range(lmax + 1)
        for l in degrees:
            natural = -1 if l % 2 else 1
            yield cls(l, natural)
            yield cls(l, -natural)

    def __mul__(self, other):
        """Irreps of the product: ``|l1 - l2| <= l <= l1 + l2``, parities multiply."""
        other = Irrep(other)
        lo, hi = abs(self[0] - other[0]), self[0] + other[0]
        return (Irrep(l, self[1] * other[1]) for l in range(lo, hi + 1))

    def __rmul__(self, mul):
        assert isinstance(mul, int)
        return Irreps([(mul, self)])

    def __add__(self, other):
        return Irreps([self]) + other

    count = index = __contains__ = __len__ = _not_a_sequence


class _MulIr(tuple):
    """``mul`` copies of one irrep."""

    def __new__(cls, mul, ir=None):
        if ir is None:
            mul, ir = mul
        assert isinstance(mul, int) and isinstance(ir, Irrep)
        return tuple.__new__(cls, (mul, ir))

    mul = property(lambda self: self[0])
    ir = property(lambda self: self[1])
    dim = property(lambda self: self[0] * self[1].dim)

    def __repr__(self) -> str:
        return f"{self[0]}x{self[1]!r}"

    count = index = _not_a_sequence


def _terms_of_string(text: str):
    if not text.strip():
        return []
    terms = []
    for piece in text.split("+"):
        m = _TERM.fullmatch(piece)
        if m is None:
            raise ValueError(f'Unable to convert string "{text}" into an Irreps')
        terms.append(_MulIr(int(m.group(1) or 1), Irrep(m.group(2))))
    return terms


def _term_of_item(item):
    """One element of a list given to ``Irreps``: "1o", Irrep, (mul, irrep-like) or a ``_MulIr``."""
    if isinstance(item, _MulIr):
        return item
    if isinstance(item, (str, Irrep)):
        return _MulIr(1, Irrep(item))
    try:
        mul, ir = item
    except (TypeError, ValueError):
        raise ValueError(f'Unable to interpret "{item}" as an irrep.') from None
    if isinstance(mul, bool) or not isinstance(mul, int) or mul < 0:
        raise ValueError(f'Unable to interpret "{item}" as an irrep.')
    return _MulIr(mul, Irrep(ir))


class Irreps(tuple):
    """Direct sum of irreps, ``Irreps("16x0e + 16x1o")``.

    A feature vector with these irreps stores the blocks in order; a block of
    ``mul x (l, p)`` is a row-major ``[mul, 2l+1]`` array.
    """

    def __new__(cls, irreps=None):
        if isinstance(irreps, Irreps):
            terms = irreps
        elif irreps is None:
            terms = ()
        elif isinstance(irreps, Irrep):
            terms = (_MulIr(1, irreps),)
        elif isinstance(irreps, str):
            terms = _terms_of_string(irreps)
        else:
            terms = [_term_of_item(item) for item in irreps]
        return tuple.__new__(cls, terms)

    @staticmethod
    def spherical_harmonics(lmax: int, p: int = -1) -> "Irreps":
        """``0e + 1o + 2e + ...`` up to ``lmax`` (``p = 1``: all even)."""
        return Irreps([_MulIr(1, Irrep(l, p**l)) for l in range(lmax + 1)])

    # ---- layout -------------------------------------------------------------------------------------------------
    @property
    def dim(self) -> int:
        return sum(term.dim for term in self)

    @property
    def num_irreps(self) -> int:
        return sum(term.mul for term in self)

    @property
    def ls(self) -> List[int]:
        return [term.ir.l for term in self for _ in range(term.mul)]

    @property
    def lmax(self) -> int:
        if not self:
            raise ValueError("an empty Irreps has no lmax")
        return max(term.ir.l for term in self)

    def slices(self):
        """Column range of every block in a feature vector."""
        ends = list(itertools.accumulate(term.dim for term in self))
        return [slice(end - term.dim, end) for term, end in zip(self, ends)]

    def randn(self, *size, normalization="component", requires_grad=False, dtype=None, device=None):
        """Random features; the ``-1`` in ``size`` stands for the irreps axis.  ``"component"``: every component
        N(0, 1); ``"norm"``: every irrep copy uniformly on the unit sphere of its 2l+1 components."""
        axis = size.index(-1)
        before, after = size[:axis], size[axis + 1 :]
        if normalization == "component":
            return torch.randn(*before, self.dim, *after, requires_grad=requires_grad, dtype=dtype, device=device)
        if normalization != "norm":
            raise ValueError(f"normalization must be 'component' or 'norm', got {normalization!r}")
        blocks = []
        for term in self:
            v = torch.randn(*before, term.mul, term.ir.dim, *after, dtype=dtype, device=device)
            v = v / v.norm(dim=axis + 1, keepdim=True)
            blocks.append(v.reshape(*before, term.dim, *after))
        x = torch.cat(blocks, dim=axis) if blocks else torch.zeros(*before, 0, *after, dtype=dtype, device=device)
        return x.requires_grad_(requires_grad)

    # ---- tuple protocol -------------------------------------------------------------------------------------------
    def __getitem__(self, i):
        got = tuple.__getitem__(self, i)
        return Irreps(got) if isinstance(i, slice) else got

    def __contains__(self, ir) -> bool:
        wanted = Irrep(ir)
        return any(term.ir == wanted for term in self)

    def count(self, ir) -> int:
        """Total multiplicity of ``ir``."""
        wanted = Irrep(ir)
        return sum(term.mul for term in self if term.ir == wanted)

    index = _not_a_sequence

    def __add__(self, irreps) -> "Irreps":
        return Irreps(tuple(self) + tuple(Irreps(irreps)))

    def __mul__(self, n) -> "Irreps":
        if isinstance(n, Irreps):
            raise NotImplementedError("Irreps * Irreps is not defined: build an o3.TensorProduct")
        return Irreps(tuple(self) * n)

    __rmul__ = __mul__

    def __repr__(self) -> str:
        return "+".join(map(repr, self))

    # ---- rearrangements -------------------------------------------------------------------------------------------
    def remove_zero_multiplicities(self) -> "Irreps":
        return Irreps([term for term in self if term.mul > 0])

    def simplify(self) -> "Irreps":
        """Merges neighbouring blocks of the same irrep and drops empty ones (the order is kept)."""
        merged = []
        for ir, run in itertools.groupby(self.remove_zero_multiplicities(), key=lambda term: term.ir):
            merged.append((sum(term.mul for term in run), ir))
        return Irreps(merged)

    def sort(self):
        """Stable sort by ``(l, p)``; returns ``(irreps, p, inv)`` with ``sorted[p[i]] = self[i]`` and
        ``sorted[j] = self[inv[j]]``."""
        inv = tuple(sorted(range(len(self)), key=lambda i: (self[i].ir, i, self[i].mul)))
        p = [0] * len(inv)
        for new, old in enumerate(inv):
            p[old] = new
        return _SortResult(Irreps([self[i] for i in inv]), tuple(p), inv)

    def regroup(self) -> "Irreps":
        """Sorted, with equal irreps merged."""
        ordered, _, _ = self.sort()
        return ordered.simplify()

    def filter(self, keep=None, *, drop=None, lmax: int = None) -> "Irreps":
        """Blocks selected by ``keep`` (irreps or a predicate on ``(mul, ir)``), by ``drop`` (the complement) or by
        ``lmax``; at most one of the three."""
        given = [name for name, v in (("keep", keep), ("drop", drop), ("lmax", lmax)) if v is not None]
        if not given:
            return self
        if len(given) > 1:
            raise ValueError("Cannot specify more than one of keep, drop and lmax")
        if lmax is not None:
            return Irreps([term for term in self if term.ir.l <= lmax])
        selector, wanted = (keep, True) if keep is not None else (drop, False)
        if callable(selector):
            return Irreps([term for term in self if bool(selector(term)) is wanted])
        if isinstance(selector, (str, Irrep, _MulIr)):
            selector = [Irrep(selector)] if not isinstance(selector, str) else [term.ir for term in Irreps(selector)]
        chosen = {Irrep(ir) for ir in selector}
        return Irreps([term for term in self if (term.ir in chosen) is wanted])


IrrepsLike = Union[str, Irreps, Irrep, list, tuple]
