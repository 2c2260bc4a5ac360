"""O(3) irreducible representations and their direct sums.

Host-side algebra needed to derive a convolution's coefficient table from
irreps strings: parsing, dimensions, block slices, Clebsch-Gordan selection
rules and the canonical (degree, parity) ordering.  Behaviour follows
`src/e3j/spaces/o3.py:110-116,146-165,189-230,249-306` and
`src/e3j/spaces/space.py:107-182`.
"""

from __future__ import annotations

import itertools
import re
from typing import Iterable, Iterator

import numpy as np

_IRREP_RE = re.compile(r"^(\d+)([eo])$")
_MUL_RE = re.compile(r"^(\d+)\s*x\s*(.+)$")


class O3Irrep:
    """One irreducible block: degree `l >= 0` and parity `p` in {+1, -1}."""

    __slots__ = ("l", "p")

    def __init__(self, *args):
        if len(args) == 1:
            (arg,) = args
            if isinstance(arg, O3Irrep):
                self.l, self.p = arg.l, arg.p
            elif isinstance(arg, str):
                match = _IRREP_RE.match(arg.strip())
                if match is None:
                    raise ValueError(f"cannot parse irrep {arg!r}; expected '<l>e' or '<l>o'")
                self.l = int(match.group(1))
                self.p = 1 if match.group(2) == "e" else -1
            elif isinstance(arg, (int, np.integer)):
                self.l, self.p = int(arg), 1
            elif isinstance(arg, tuple) and len(arg) == 2:
                self.l, self.p = int(arg[0]), int(arg[1])
            else:
                raise ValueError(f"cannot build an irrep from {arg!r}")
        elif len(args) == 2:
            self.l, self.p = int(args[0]), int(args[1])
        else:
            raise ValueError("O3Irrep takes (l, p), l, or a string such as '1o'")
        if self.l < 0 or self.p not in (1, -1):
            raise ValueError(f"invalid irrep l={self.l}, p={self.p}")

    @property
    def dim(self) -> int:
        return 2 * self.l + 1

    def __iter__(self):
        yield self.l
        yield self.p

    def __str__(self) -> str:
        return f"{self.l}{'e' if self.p == 1 else 'o'}"

    __repr__ = __str__

    def __eq__(self, other) -> bool:
        return isinstance(other, O3Irrep) and (self.l, self.p) == (other.l, other.p)

    def __hash__(self) -> int:
        return hash((self.l, self.p))

    def _sort_key(self) -> tuple[int, int]:
        # Increasing degree; within a degree the natural parity (-1)^l comes
        # first (`src/e3j/spaces/o3.py:110-116`).
        return (self.l, 0 if self.p == (-1) ** self.l else 1)

    def __lt__(self, other: "O3Irrep") -> bool:
        return self._sort_key() < other._sort_key()

    def __mul__(self, other: "O3Irrep") -> "O3Space":
        """Selection rules of the product of two irreducible blocks."""
        if not isinstance(other, O3Irrep):
            return NotImplemented
        parity = self.p * other.p
        return O3Space(
            [(1, O3Irrep(l, parity)) for l in range(abs(self.l - other.l), self.l + other.l + 1)]
        )

    def __rmul__(self, mul: int) -> "O3Space":
        return O3Space([(int(mul), self)])


class O3Space:
    """Direct sum of `(multiplicity, irrep)` blocks, e.g. `"2x0e + 1o"`."""

    def __init__(self, blocks: "str | O3Space | Iterable"):
        if isinstance(blocks, O3Space):
            self.blocks = list(blocks.blocks)
        elif isinstance(blocks, str):
            self.blocks = self._parse_string(blocks)
        else:
            self.blocks = self._parse_list(blocks)

    @staticmethod
    def _parse_string(text: str) -> list[tuple[int, O3Irrep]]:
        out = []
        for chunk in re.split(r"\s*\+\s*", text.strip()):
            match = _MUL_RE.match(chunk)
            if match:
                out.append((int(match.group(1)), O3Irrep(match.group(2))))
            else:
                out.append((1, O3Irrep(chunk)))
        return out

    @staticmethod
    def _parse_list(blocks) -> list[tuple[int, O3Irrep]]:
        out = []
        for block in blocks:
            if len(block) == 3:
                mul, l, p = block
                irrep = O3Irrep(l, p)
            elif len(block) == 2:
                mul, irrep = block
                irrep = irrep if isinstance(irrep, O3Irrep) else (
                    O3Irrep(*irrep) if isinstance(irrep, tuple) else O3Irrep(irrep))
            else:
                raise ValueError("blocks must be (mul, irrep) or (mul, l, p)")
            if int(mul) <= 0:
                raise ValueError("multiplicities must be positive")
            out.append((int(mul), irrep))
        return out

    # --- container protocol ---------------------------------------------
    def __iter__(self) -> Iterator[tuple[int, O3Irrep]]:
        return iter(self.blocks)

    def __len__(self) -> int:
        return len(self.blocks)

    def __eq__(self, other) -> bool:
        other = other if isinstance(other, O3Space) else O3Space(other)
        return self.blocks == other.blocks

    def __hash__(self) -> int:
        return hash(tuple(self.blocks))

    def __str__(self) -> str:
        return " + ".join(f"{m}x{ir}" for m, ir in self.blocks)

    __repr__ = __str__

    def __rmul__(self, mul: int) -> "O3Space":
        return O3Space([(int(mul) * m, ir) for m, ir in self.blocks])

    # --- sizes ----------------------------------------------------------
    @property
    def dim(self) -> int:
        return sum(m * ir.dim for m, ir in self.blocks)

    @property
    def num_irreps(self) -> int:
        return sum(m for m, _ in self.blocks)

    @property
    def l_max(self) -> int:
        return max(ir.l for _, ir in self.blocks)

    def slices(self) -> list[slice]:
        out, begin = [], 0
        for m, ir in self.blocks:
            out.append(slice(begin, begin + m * ir.dim))
            begin += m * ir.dim
        return out

    # --- ordering -------------------------------------------------------
    def sort(self, return_inverse: bool = False):
        """Stable sort of the blocks by (degree, parity) (`src/e3j/spaces/space.py:141-158`)."""
        order = sorted(range(len(self.blocks)), key=lambda i: (self.blocks[i][1]._sort_key(), i))
        sorted_space = O3Space([self.blocks[i] for i in order])
        if return_inverse:
            return sorted_space, np.asarray(order, dtype=np.int64)
        return sorted_space

    def regroup(self) -> "O3Space":
        """Sort, then merge equal irreps into one block (`src/e3j/spaces/space.py:160-182`)."""
        blocks = self.sort().blocks
        if len(blocks) <= 1:
            return O3Space(self.blocks)
        merged = [list(blocks[0])]
        for mul, ir in blocks[1:]:
            if ir == merged[-1][1]:
                merged[-1][0] += mul
            else:
                merged.append([mul, ir])
        return O3Space([(m, ir) for m, ir in merged])

    # --- products -------------------------------------------------------
    @staticmethod
    def otimes(lhs, rhs, target_filter=None, sort: bool = False) -> "O3Space":
        """Irreducible blocks of `lhs (x) rhs`, optionally filtered (`src/e3j/spaces/o3.py:189-230`).

        Blocks come out in lhs-major, rhs, then increasing output degree order:
        one block per Clebsch-Gordan path.
        """
        lhs, rhs = O3Space(lhs), O3Space(rhs)
        keep = None
        if target_filter is not None:
            target_filter = O3Space(target_filter)
            if any(m != 1 for m, _ in target_filter):
                raise ValueError("Filter `out` should have multiplicities 1")
            keep = {(ir.l, ir.p) for _, ir in target_filter}
        blocks = []
        for (m1, ir1), (m2, ir2) in itertools.product(lhs, rhs):
            for _, ir0 in ir1 * ir2:
                if keep is not None and (ir0.l, ir0.p) not in keep:
                    continue
                blocks.append((m1 * m2, ir0))
        out = O3Space(blocks)
        return out.regroup() if sort else out


def harmonics_space(l_max: int) -> O3Space:
    """`0e + 1o + 2e + ...` up to `l_max`: the irreps of spherical harmonics."""
    return O3Space([(1, O3Irrep(l, (-1) ** l)) for l in range(l_max + 1)])
