"""``Op`` root and the boundary sentinels (emmy/compiler/ir/base.py:32-160)."""

from __future__ import annotations

from dataclasses import dataclass, field


@dataclass
class Op:
    """Base of every operation.  ``source`` is the predecessor op in the
    lowering chain (HipOp → TileOp → frontend ops); ``knobs`` records the
    schedule knobs that produced it.  Both are attribution only."""

    source: object | None = field(default=None, kw_only=True, repr=False, compare=False)
    knobs: dict = field(default_factory=dict, kw_only=True, repr=False, compare=False)

    def pretty_body(self) -> str | None:
        return None


@dataclass
class InputOp(Op):
    """Graph input (no computation)."""


@dataclass
class ConstantOp(Op):
    """Fixed tensor: weights, tables, scalars.  ``value`` is a static scalar;
    ``None`` means the executor supplies the tensor (``input_data`` or the
    traced module's parameter at ``source_path``)."""

    name: str = ""
    value: float | None = None
    source_path: str | None = None
