"""HipOp — graph-level wrapper around one rendered gfx950 kernel.

The artifact contract of the backend, field for field the reference's
``CudaOp`` (emmy/compiler/ir/cuda/ir.py:43-88) minus the TMA descriptors
(no counterpart on CDNA4): the lowered graph is ``Graph[HipOp + InputOp +
ConstantOp]``; the runtime walks it in topological order and issues one
launch per node, wiring buffer pointers by node id.
"""

from __future__ import annotations

from dataclasses import dataclass

from deplodock_amd.ir.base import Op

# int = static factor; str = symbolic axis name resolved at launch; a callable
# takes the symbolic env and returns an int (e.g. a ceil-div block count).
GridDimSpec = tuple


@dataclass
class HipOp(Op):
    """One kernel invocation.

    ``grid`` / ``block`` hold three per-dim specs whose factors are multiplied
    at launch.  ``arg_order`` lists buffer names (graph node ids) in signature
    order; ``runtime_args`` lists symbolic names passed as trailing ``int``
    parameters.  ``lds_bytes`` is *dynamic* LDS requested at launch (static
    LDS is declared in the source).  ``zero_outputs`` are buffers the runtime
    must clear before the launch (atomic accumulation targets).
    ``algo_bytes`` / ``algo_flops`` are the algorithmic work of one launch,
    used for roofline reporting."""

    kernel_source: str = ""
    kernel_name: str = ""
    arg_order: tuple[str, ...] = ()
    grid: tuple = ((1,), (1,), (1,))
    block: tuple = ((1,), (1,), (1,))
    lds_bytes: int = 0
    zero_outputs: tuple[str, ...] = ()
    comment: str = ""
    runtime_args: tuple[str, ...] = ()
    algo_bytes: int = 0
    algo_flops: int = 0

    def pretty_body(self) -> str:
        return self.kernel_source


def resolve_dim(spec, sym_values: dict[str, int]) -> int:
    """Product of a ``GridDimSpec``'s factors (cuda/ir.py:91-112): ints as is,
    ``str`` looked up in ``sym_values`` (``KeyError`` when unknown), callables
    evaluated on ``sym_values``.  A bare int is accepted as shorthand."""
    if isinstance(spec, int):
        return spec
    total = 1
    for factor in spec:
        if isinstance(factor, int):
            total *= factor
        elif isinstance(factor, str):
            total *= sym_values[factor]
        else:
            total *= int(factor(sym_values))
    return total
