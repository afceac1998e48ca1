"""Errors raised while lowering a scheduled tile to HIP source."""


class LoweringError(ValueError):
    """The stamped schedule cannot be realised on gfx950 (LDS or register
    budget exceeded, shape not divisible by the tile, …).  Same role as the
    reference's ``LoweringError`` raised by ``KernelOp.validate``
    (emmy/compiler/ir/kernel/ir.py:1650-1705)."""
