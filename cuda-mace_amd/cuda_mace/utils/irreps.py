"""Minimal stand-ins for the e3nn objects whose attributes the op wrappers read.

The reference's wrappers take e3nn `Irreps` and `Instruction` objects from an upstream model and
read a handful of attributes from them (`lmax`, `dim`, `num_irreps`, `simplify()`, indexing into
(mul, irrep) pairs, `path_shape`, `i_in`, `i_out`, `path_weight`).  e3nn is not a dependency here;
these classes provide exactly those attributes so that an upstream-like model object can be built
without it.  Real e3nn objects offer the same attributes and are accepted interchangeably.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Tuple


@dataclass(frozen=True)
class Irrep:
    l: int
    p: int  # parity: +1 (e) or -1 (o)

    @property
    def dim(self) -> int:
        return 2 * self.l + 1

    def __str__(self) -> str:
        return "%d%s" % (self.l, "e" if self.p == 1 else "o")


@dataclass(frozen=True)
class MulIrrep:
    mul: int
    ir: Irrep

    @property
    def dim(self) -> int:
        return self.mul * self.ir.dim

    def __iter__(self):
        yield self.mul
        yield self.ir


class Irreps:
    """Direct sum of `mul x l{e,o}` blocks, e.g. Irreps("128x0e+128x1o+128x2e+128x3o")."""

    def __init__(self, spec):
        items: List[MulIrrep] = []
        if isinstance(spec, Irreps):
            items = list(spec._items)
        elif isinstance(spec, str):
            for tok in spec.replace(" ", "").split("+"):
                if not tok:
                    continue
                mul, ir = tok.split("x") if "x" in tok else ("1", tok)
                items.append(MulIrrep(int(mul), Irrep(int(ir[:-1]), 1 if ir[-1] == "e" else -1)))
        else:
            for it in spec:
                mul, ir = it
                items.append(MulIrrep(int(mul), ir if isinstance(ir, Irrep) else Irrep(int(ir[0]), int(ir[1]))))
        self._items: Tuple[MulIrrep, ...] = tuple(items)

    @staticmethod
    def spherical_harmonics(lmax: int) -> "Irreps":
        return Irreps([(1, Irrep(l, (-1) ** l)) for l in range(lmax + 1)])

    def __iter__(self):
        return iter(self._items)

    def __len__(self):
        return len(self._items)

    def __getitem__(self, i):
        return self._items[i]

    @property
    def dim(self) -> int:
        return sum(x.dim for x in self._items)

    @property
    def num_irreps(self) -> int:
        return sum(x.mul for x in self._items)

    @property
    def lmax(self) -> int:
        return max(x.ir.l for x in self._items)

    def simplify(self) -> "Irreps":
        out: List[MulIrrep] = []
        for x in self._items:
            if out and out[-1].ir == x.ir:
                out[-1] = MulIrrep(out[-1].mul + x.mul, x.ir)
            elif x.mul > 0:
                out.append(x)
        return Irreps(out)

    def __str__(self) -> str:
        return "+".join("%dx%s" % (x.mul, x.ir) for x in self._items)

    __repr__ = __str__


@dataclass(frozen=True)
class Instruction:
    """One block of a per-l linear map: input block i_in -> output block i_out."""

    i_in: int
    i_out: int
    path_shape: Tuple[int, ...]
    path_weight: float
