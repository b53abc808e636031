"""O(3) irreducible-representation bookkeeping (host side, torch free).

Behavioural counterpart of the reference's ``Irrep`` / ``Irreps`` types
(reference: openequivariance/implementations/e3nn_lite.py:53-352), written from
scratch around two frozen value classes.  Only what the tensor-product hot path
needs is provided: parsing, ordering, dimensions, slices, the selection rule
``ir1 * ir2`` and the stable ``sort`` used to lay out channel-wise outputs.
"""
from __future__ import annotations

import re
from typing import Iterable, Iterator, List, NamedTuple, Tuple, Union

_IRREP_RE = re.compile(r"^\s*(\d+)\s*([eoy])\s*$")


class Irrep(tuple):
    """One irrep of O(3): degree ``l >= 0`` and parity ``p`` in {+1, -1}.

    Accepts ``Irrep(l, p)``, ``Irrep("2e")``, ``Irrep((l, p))`` or another Irrep.
    It is a tuple ``(l, p)`` so that it compares, hashes and sorts like the
    reference's type (sorting is by ``l`` first, then by ``p``).
    """

    __slots__ = ()

    def __new__(cls, l, p=None):
        if p is None:
            if isinstance(l, Irrep):
                return l
            if isinstance(l, str):
                m = _IRREP_RE.match(l)
                if m is None:
                    raise ValueError(f'unable to convert string "{l}" into an Irrep')
                deg = int(m.group(1))
                par = {"e": 1, "o": -1, "y": (-1) ** deg}[m.group(2)]
                l, p = deg, par
            elif isinstance(l, tuple) and len(l) == 2:
                l, p = l
            elif hasattr(l, "l") and hasattr(l, "p"):  # e.g. an e3nn Irrep
                l, p = int(l.l), int(l.p)
        if not isinstance(l, int) or isinstance(l, bool) or l < 0:
            raise ValueError(f"l must be a non-negative integer, got {l!r}")
        if p not in (-1, 1):
            raise ValueError(f"parity must be one of (-1, 1), got {p!r}")
        return tuple.__new__(cls, (l, int(p)))

    @property
    def l(self) -> int:
        return tuple.__getitem__(self, 0)

    @property
    def p(self) -> int:
        return tuple.__getitem__(self, 1)

    @property
    def dim(self) -> int:
        return 2 * self.l + 1

    def is_scalar(self) -> bool:
        return self.l == 0 and self.p == 1

    def __repr__(self) -> str:
        return f"{self.l}{'e' if self.p == 1 else 'o'}"

    def __mul__(self, other) -> Iterator["Irrep"]:
        """Selection rule: irreps contained in the product of two irreps."""
        other = Irrep(other)
        par = self.p * other.p
        return (Irrep(l, par) for l in range(abs(self.l - other.l), self.l + other.l + 1))

    def __rmul__(self, mul: int) -> "Irreps":
        if not isinstance(mul, int):
            raise TypeError("only int * Irrep is defined")
        return Irreps([(mul, self)])

    def __add__(self, other) -> "Irreps":
        return Irreps(self) + Irreps(other)

    @classmethod
    def iterator(cls, lmax=None) -> Iterator["Irrep"]:
        l = 0
        while lmax is None or l <= lmax:
            yield Irrep(l, (-1) ** l)
            yield Irrep(l, -((-1) ** l))
            l += 1


class MulIr(tuple):
    """A multiplicity paired with an irrep; behaves as the tuple ``(mul, ir)``."""

    __slots__ = ()

    def __new__(cls, mul, ir=None):
        if ir is None:
            mul, ir = mul
        if not isinstance(mul, int) or mul < 0:
            raise ValueError(f"multiplicity must be a non-negative int, got {mul!r}")
        return tuple.__new__(cls, (mul, Irrep(ir)))

    @property
    def mul(self) -> int:
        return tuple.__getitem__(self, 0)

    @property
    def ir(self) -> Irrep:
        return tuple.__getitem__(self, 1)

    @property
    def dim(self) -> int:
        return self.mul * self.ir.dim

    def __repr__(self) -> str:
        return f"{self.mul}x{self.ir}"


class _SortResult(NamedTuple):
    irreps: "Irreps"
    p: Tuple[int, ...]
    inv: Tuple[int, ...]


class Irreps(tuple):
    """Direct sum of ``mul x irrep`` blocks.

    The memory layout this describes is the one every kernel assumes: blocks are
    concatenated in order, and inside a block element ``(u, m)`` sits at
    ``u * (2l+1) + m`` (multiplicity-major, ``m`` fastest).
    """

    __slots__ = ()

    def __new__(cls, irreps=None):
        if isinstance(irreps, Irreps):
            return tuple.__new__(cls, tuple(irreps))
        blocks: List[MulIr] = []
        if irreps is None:
            pass
        elif isinstance(irreps, Irrep):
            blocks.append(MulIr(1, irreps))
        elif isinstance(irreps, MulIr):
            blocks.append(irreps)
        elif isinstance(irreps, str):
            text = irreps.strip()
            if text:
                for term in text.split("+"):
                    try:
                        if "x" in term:
                            mul_s, ir_s = term.split("x")
                            blocks.append(MulIr(int(mul_s), Irrep(ir_s)))
                        else:
                            blocks.append(MulIr(1, Irrep(term)))
                    except Exception:
                        raise ValueError(f'Unable to convert string "{irreps}" into an Irreps') from None
        else:
            for item in irreps:
                if isinstance(item, MulIr):
                    blocks.append(item)
                elif isinstance(item, (str, Irrep)):
                    blocks.append(MulIr(1, Irrep(item)))
                else:
                    try:
                        mul, ir = item
                        blocks.append(MulIr(int(mul), Irrep(ir)))
                    except Exception:
                        raise ValueError(f'Unable to interpret "{item}" as an irrep.') from None
        return tuple.__new__(cls, blocks)

    @staticmethod
    def spherical_harmonics(lmax: int, p: int = -1) -> "Irreps":
        return Irreps([(1, (l, p ** l)) for l in range(lmax + 1)])

    # ---- sizes / layout -------------------------------------------------
    @property
    def dim(self) -> int:
        return sum(b.dim for b in self)

    @property
    def num_irreps(self) -> int:
        return sum(b.mul for b in self)

    @property
    def ls(self) -> List[int]:
        return [b.ir.l for b in self for _ in range(b.mul)]

    @property
    def lmax(self) -> int:
        if len(self) == 0:
            raise ValueError("Cannot get lmax of empty Irreps")
        return max(self.ls)          # blocks of multiplicity 0 do not count (reference: e3nn_lite.py:346-349)

    def slices(self) -> List[slice]:
        out, start = [], 0
        for b in self:
            out.append(slice(start, start + b.dim))
            start += b.dim
        return out

    def offsets(self) -> List[int]:
        """Column where each block starts."""
        return [s.start for s in self.slices()]

    # ---- algebra ----------------------------------------------------------
    def __getitem__(self, i):
        got = tuple.__getitem__(self, i)
        return Irreps(got) if isinstance(i, slice) else got

    def __contains__(self, ir) -> bool:
        ir = Irrep(ir)
        return any(b.ir == ir for b in self)

    def count(self, ir) -> int:
        ir = Irrep(ir)
        return sum(b.mul for b in self if b.ir == ir)

    def __add__(self, other) -> "Irreps":
        return Irreps(tuple(self) + tuple(Irreps(other)))

    def __mul__(self, n) -> "Irreps":
        if isinstance(n, Irreps):
            raise NotImplementedError("Irreps * Irreps is a tensor product; build a TPProblem instead")
        return Irreps(tuple(self) * n)

    __rmul__ = __mul__

    def simplify(self) -> "Irreps":
        merged: List[Tuple[int, Irrep]] = []
        for b in self:
            if merged and merged[-1][1] == b.ir:
                merged[-1] = (merged[-1][0] + b.mul, b.ir)
            elif b.mul > 0:
                merged.append((b.mul, b.ir))
        return Irreps(merged)

    def remove_zero_multiplicities(self) -> "Irreps":
        return Irreps([b for b in self if b.mul > 0])

    def sort(self) -> _SortResult:
        """Stable sort of the blocks by ``(l, p)``, ties kept in creation order.

        ``inv[new] = old`` and ``p[old] = new`` (reference: e3nn_lite.py:321-328).
        """
        keyed = sorted((b.ir, i, b.mul) for i, b in enumerate(self))
        inv = tuple(i for _, i, _ in keyed)
        p = [0] * len(inv)
        for new, old in enumerate(inv):
            p[old] = new
        return _SortResult(Irreps([(mul, ir) for ir, _, mul in keyed]), tuple(p), inv)

    def regroup(self) -> "Irreps":
        return self.sort().irreps.simplify()

    def __repr__(self) -> str:
        return "+".join(repr(b) for b in self)


IrrepsLike = Union[str, Irreps, Irrep, Iterable]
