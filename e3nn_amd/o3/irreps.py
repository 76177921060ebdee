"""Irreducible representations of O(3) and direct sums of them.

Same public behaviour as the reference's ``e3nn.o3.Irrep`` / ``e3nn.o3.Irreps``
(e3nn/o3/_irreps.py:14-264, :301-806) for everything the tensor-product hot path
needs: parsing, layout (``dim``, ``slices``), the selection rule ``ir1 * ir2``,
``sort`` / ``simplify`` / ``regroup`` / ``filter`` and ``randn``.  The rotation-matrix
constructors (``D_from_*``) are not part of the hot path and are not provided.
"""
import collections
import itertools
from typing import List, Union

import torch


class Irrep(tuple):
    """Irreducible representation ``(l, p)``; ``Irrep("1o")``, ``Irrep(2, 1)``, ``Irrep("3y")``."""

    def __new__(cls, l, p=None):
        if p is None:
            if isinstance(l, Irrep):
                return l
            if isinstance(l, _MulIr):
                return l.ir
            if isinstance(l, str):
                name = l.strip()
                try:
                    deg = int(name[:-1])
                    if deg < 0:
                        raise ValueError
                    p = {"e": 1, "o": -1, "y": (-1) ** deg}[name[-1]]
                    l = deg
                except Exception:
                    raise ValueError(f'unable to convert string "{name}" into an Irrep')
            elif isinstance(l, tuple):
                l, p = l
        if not isinstance(l, int) or l < 0:
            raise ValueError(f"l must be positive integer, got {l}")
        if p not in (-1, 1):
            raise ValueError(f"parity must be on of (-1, 1), got {p}")
        return super().__new__(cls, (l, p))

    @property
    def l(self) -> int:  # noqa: E743
        return self[0]

    @property
    def p(self) -> int:
        return self[1]

    @property
    def dim(self) -> int:
        return 2 * self.l + 1

    def is_scalar(self) -> bool:
        return self.l == 0 and self.p == 1

    def __repr__(self) -> str:
        return f"{self.l}{'e' if self.p == 1 else 'o'}"

    @classmethod
    def iterator(cls, lmax=None):
        for l in itertools.count():
            yield Irrep(l, (-1) ** l)
            yield Irrep(l, -((-1) ** l))
            if l == lmax:
                break

    def __mul__(self, other):
        # selection rule: |l1 - l2| <= l <= l1 + l2, parities multiply
        other = Irrep(other)
        for l in range(abs(self.l - other.l), self.l + other.l + 1):
            yield Irrep(l, self.p * other.p)

    def __rmul__(self, other):
        assert isinstance(other, int)
        return Irreps([(other, self)])

    def __add__(self, other):
        return Irreps(self) + Irreps(other)

    def count(self, _value):
        raise NotImplementedError

    def index(self, _value):
        raise NotImplementedError

    def __contains__(self, _object):
        raise NotImplementedError

    def __len__(self):
        raise NotImplementedError


class _MulIr(tuple):
    def __new__(cls, mul, ir=None):
        if ir is None:
            mul, ir = mul
        assert isinstance(mul, int)
        assert isinstance(ir, Irrep)
        return super().__new__(cls, (mul, ir))

    @property
    def mul(self) -> int:
        return self[0]

    @property
    def ir(self) -> Irrep:
        return self[1]

    @property
    def dim(self) -> int:
        return self.mul * self.ir.dim

    def __repr__(self) -> str:
        return f"{self.mul}x{self.ir}"

    def count(self, _value):
        raise NotImplementedError

    def index(self, _value):
        raise NotImplementedError


class Irreps(tuple):
    """Direct sum of irreps, ``Irreps("16x0e + 16x1o")``.

    A feature vector with these irreps stores the blocks in order; a block of
    ``mul x (l, p)`` is a row-major ``[mul, 2l+1]`` array.
    """

    def __new__(cls, irreps=None):
        if isinstance(irreps, Irreps):
            return super().__new__(cls, irreps)
        out = []
        if isinstance(irreps, Irrep):
            out.append(_MulIr(1, Irrep(irreps)))
        elif isinstance(irreps, str):
            try:
                if irreps.strip() != "":
                    for term in irreps.split("+"):
                        if "x" in term:
                            mul, ir = term.split("x")
                            mul, ir = int(mul), Irrep(ir)
                        else:
                            mul, ir = 1, Irrep(term)
                        assert isinstance(mul, int) and mul >= 0
                        out.append(_MulIr(mul, ir))
            except Exception:
                raise ValueError(f'Unable to convert string "{irreps}" into an Irreps')
        elif irreps is None:
            pass
        else:
            for mul_ir in irreps:
                mul, ir = None, None
                if isinstance(mul_ir, str):
                    mul, ir = 1, Irrep(mul_ir)
                elif isinstance(mul_ir, Irrep):
                    mul, ir = 1, mul_ir
                elif isinstance(mul_ir, _MulIr):
                    mul, ir = mul_ir
                elif len(mul_ir) == 2:
                    mul, ir = mul_ir
                    ir = Irrep(ir)
                if not (isinstance(mul, int) and mul >= 0 and ir is not None):
                    raise ValueError(f'Unable to interpret "{mul_ir}" as an irrep.')
                out.append(_MulIr(mul, ir))
        return super().__new__(cls, out)

    @staticmethod
    def spherical_harmonics(lmax: int, p: int = -1) -> "Irreps":
        return Irreps([(1, (l, p**l)) for l in range(lmax + 1)])

    def slices(self):
        out, i = [], 0
        for mul_ir in self:
            out.append(slice(i, i + mul_ir.dim))
            i += mul_ir.dim
        return out

    def randn(self, *size, normalization="component", requires_grad=False, dtype=None, device=None):
        di = size.index(-1)
        lsize, rsize = size[:di], size[di + 1 :]
        if normalization == "component":
            return torch.randn(*lsize, self.dim, *rsize, requires_grad=requires_grad, dtype=dtype, device=device)
        if normalization == "norm":
            x = torch.zeros(*lsize, self.dim, *rsize, requires_grad=requires_grad, dtype=dtype, device=device)
            with torch.no_grad():
                for s, (mul, ir) in zip(self.slices(), self):
                    r = torch.randn(*lsize, mul, ir.dim, *rsize, dtype=dtype, device=device)
                    r.div_(r.norm(2, dim=di + 1, keepdim=True))
                    x.narrow(di, s.start, mul * ir.dim).copy_(r.reshape(*lsize, -1, *rsize))
            return x
        raise ValueError("Normalization needs to be 'norm' or 'component'")

    def __getitem__(self, i):
        x = super().__getitem__(i)
        return Irreps(x) if isinstance(i, slice) else x

    def __contains__(self, ir) -> bool:
        ir = Irrep(ir)
        return any(ir == irrep for _, irrep in self)

    def count(self, ir) -> int:
        ir = Irrep(ir)
        return sum(mul for mul, irrep in self if ir == irrep)

    def index(self, _object):
        raise NotImplementedError

    def __add__(self, irreps) -> "Irreps":
        return Irreps(super().__add__(Irreps(irreps)))

    def __mul__(self, other) -> "Irreps":
        if isinstance(other, Irreps):
            raise NotImplementedError("Use o3.TensorProduct for this, see the documentation")
        return Irreps(super().__mul__(other))

    def __rmul__(self, other) -> "Irreps":
        return Irreps(super().__rmul__(other))

    def simplify(self) -> "Irreps":
        out = []
        for mul, ir in self:
            if out and out[-1][1] == ir:
                out[-1] = (out[-1][0] + mul, ir)
            elif mul > 0:
                out.append((mul, ir))
        return Irreps(out)

    def remove_zero_multiplicities(self) -> "Irreps":
        return Irreps([(mul, ir) for mul, ir in self if mul > 0])

    def sort(self):
        """Stable sort by ``(l, p)`` (odd before even at equal ``l``); returns ``(irreps, p, inv)``."""
        Ret = collections.namedtuple("sort", ["irreps", "p", "inv"])
        keyed = sorted((ir, i, mul) for i, (mul, ir) in enumerate(self))
        inv = tuple(i for _, i, _ in keyed)
        p = tuple(inv.index(i) for i in range(len(inv)))
        return Ret(Irreps([(mul, ir) for ir, _, mul in keyed]), p, inv)

    def regroup(self) -> "Irreps":
        return self.sort().irreps.simplify()

    def filter(self, keep=None, *, drop=None, lmax: int = None) -> "Irreps":
        if keep is None and drop is None and lmax is None:
            return self
        if sum(v is not None for v in (keep, drop, lmax)) > 1:
            raise ValueError("Cannot specify more than one of keep, drop and lmax")
        if lmax is not None:
            return Irreps([(mul, ir) for mul, ir in self if ir.l <= lmax])
        sel, want = (keep, True) if keep is not None else (drop, False)
        if callable(sel):
            return Irreps([mul_ir for mul_ir in self if bool(sel(mul_ir)) == want])
        if isinstance(sel, str):
            sel = Irreps(sel)
        if isinstance(sel, Irrep):
            sel = [sel]
        if isinstance(sel, _MulIr):
            sel = [sel.ir]
        sel = {Irrep(ir) for ir in sel}
        return Irreps([(mul, ir) for mul, ir in self if (ir in sel) == want])

    @property
    def dim(self) -> int:
        return sum(mul * ir.dim for mul, ir in self)

    @property
    def num_irreps(self) -> int:
        return sum(mul for mul, _ in self)

    @property
    def ls(self) -> List[int]:
        return [l for mul, (l, p) in self for _ in range(mul)]

    @property
    def lmax(self) -> int:
        if len(self) == 0:
            raise ValueError("Cannot get lmax of empty Irreps")
        return max(self.ls)

    def __repr__(self) -> str:
        return "+".join(f"{mul_ir}" for mul_ir in self)


IrrepsLike = Union[str, Irreps, Irrep, list, tuple]
