"""The lowering pipeline: frontend graph → tile graph → scheduled → HIP graph.

``HIP_PASSES`` names the stages the way the reference's ``CUDA_PASSES`` does
(emmy/compiler/pipeline/__init__.py:43-47); ``Pipeline.run`` drives them in
order and can dump the graph after each stage (``EMMY_DUMP_DIR``).
"""

from __future__ import annotations

from collections.abc import Callable
from pathlib import Path

from deplodock_amd import config
from deplodock_amd.context import Context
from deplodock_amd.graph import Graph
from deplodock_amd.passes.fuse import fuse
from deplodock_amd.passes.lower import lower
from deplodock_amd.passes.prefetch import add_weight_prefetch
from deplodock_amd.passes.schedule import schedule

HIP_PASSES: tuple[tuple[str, Callable], ...] = (
    ("fuse", lambda g, ctx: fuse(g)),
    ("lowering/tile", schedule),
    ("lowering/hip", lower),
    ("lowering/prefetch", add_weight_prefetch),
)


def format_kernels(graph: Graph) -> str:
    """Every kernel's source, in launch order (what ``emmy compile`` prints)."""
    from deplodock_amd.ir.hip import HipOp

    parts = []
    for nid in graph.topological_order():
        op = graph.nodes[nid].op
        if isinstance(op, HipOp):
            grid = op.grid[0]
            parts.append(f"// ---- {op.kernel_name}  grid={grid} block={op.block[0]} lds={op.lds_bytes}  {op.comment}\n{op.kernel_source}")
    return "\n".join(parts)


class Pipeline:
    def __init__(self, passes=HIP_PASSES, ctx: Context | None = None):
        self.passes = tuple(passes)
        self.ctx = ctx or Context()

    @classmethod
    def build(cls, passes=HIP_PASSES, ctx: Context | None = None) -> Pipeline:
        return cls(passes, ctx)

    def run(self, graph: Graph, dump_dir: Path | None = None) -> Graph:
        dump_dir = dump_dir or config.dump_dir()
        g = graph
        for i, (name, fn) in enumerate(self.passes):
            g = fn(g, self.ctx)
            if dump_dir is not None:
                dump_dir.mkdir(parents=True, exist_ok=True)
                tag = f"{(i + 1) * 10:02d}_{name.replace('/', '_')}"
                (dump_dir / f"{tag}.txt").write_text(g.pretty_print() + "\n")
                if name == "lowering/hip":
                    (dump_dir / f"{tag}_kernels.hip").write_text(format_kernels(g))
        return g
