"""Symbolic extents: one named runtime ``int`` (``seq_len``) and values affine in it.

The reference traces ``--dynamic seq_len@x:1`` into ``Dim`` expressions, emits ``int seq_len`` as a trailing
kernel parameter, sizes grids with symbolic factors and masks the tiles that hang over
(emmy/compiler/ir/kernel/ir.py:258-276, ir/kernel/render.py:474-477, ir/cuda/ir.py:66-112) and keeps one captured
graph per symbolic key (backend/cuda/program.py:843-907).  Here a symbolic kernel is an ordinary kernel body
lowered at the traced size whose size-dependent fields are marked ``Affine`` (``a * seq_len + b``): the emitters
spell such a field as an expression over the kernel's trailing ``int`` parameter instead of a literal, guard
rows and key blocks at run time, and size the grid with a factor the runtime evaluates per launch.  One code
object then serves every size.
"""

from __future__ import annotations

from dataclasses import dataclass


def param_name(name: str) -> str:
    """The C name of the kernel parameter that carries symbol ``name``.  The symbol's own name is the caller's
    (``s``, ``n``, ``lane`` ...) and may be that of any local of an emitted kernel; the parameter's is reserved."""
    return f"emh_n_{name}"


@dataclass(frozen=True)
class Affine:
    """``a * <name> + b``."""

    name: str
    a: int
    b: int = 0

    def at(self, env: dict) -> int:
        return self.a * int(env[self.name]) + self.b

    def c(self) -> str:
        """C spelling over the kernel's ``int`` parameter of this symbol (:func:`param_name`)."""
        core = param_name(self.name) if self.a == 1 else f"{param_name(self.name)} * {self.a}"
        return f"({core})" if self.b == 0 else f"({core} + {self.b})" if self.b > 0 else f"({core} - {-self.b})"

    def __call__(self, env: dict) -> int:  # usable as a launch-time grid factor
        return self.at(env)


@dataclass(frozen=True)
class CeilDiv:
    """Launch-time grid factor ``ceil(value / div)``."""

    value: Affine
    div: int

    def __call__(self, env: dict) -> int:
        return -(-self.value.at(env) // self.div)


@dataclass(frozen=True)
class XcdRounds:
    """Launch-time grid of a contraction whose row count is symbolic: ``ceil(m / tile_m) * blocks_n`` tile
    blocks of ``per_block`` tiles, dealt over ``xcds`` and rounded up to whole rounds."""

    m: Affine
    tile_m: int
    blocks_n: int
    per_block: int
    xcds: int

    def __call__(self, env: dict) -> int:
        n_blocks = -(-self.m.at(env) // self.tile_m) * self.blocks_n
        return -(-n_blocks // self.xcds) * self.xcds * self.per_block


@dataclass(frozen=True)
class SymSpec:
    """Which fields of a tile body follow the symbolic axis: ``fields`` maps a dotted field path
    (``"rows"``, ``"row_operands.1.mod"``) to its ``Affine``; every other field holds at any size."""

    name: str
    hint: int
    fields: dict

    def get(self, path: str, literal: int):
        """The ``Affine`` of ``path``, or ``literal`` when the field does not depend on the axis."""
        return self.fields.get(path, literal)


def c_value(v) -> str:
    """C spelling of an int or an ``Affine``."""
    return v.c() if isinstance(v, Affine) else str(int(v))


def resolve(v, env: dict) -> int:
    return v.at(env) if isinstance(v, Affine) else int(env[v]) if isinstance(v, str) else int(v)


__all__ = ["param_name", "Affine", "CeilDiv", "XcdRounds", "SymSpec", "c_value", "resolve"]
