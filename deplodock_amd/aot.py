"""Ahead-of-time kernel compilation: fill the code-object cache without a GPU.

hipRTC cross-compiles for gfx950 on any host, so the kernels of known workloads
can be built where the tree is built and travel with it (the reference warms
its cubin cache the same way: ``compile_to_cubin`` is GPU-free,
emmy/compiler/backend/cuda/nvcc.py:118-152).
"""

from __future__ import annotations

from deplodock_amd import config
from deplodock_amd.backend.hip import hiprtc, launcher
from deplodock_amd.graph import Graph
from deplodock_amd.ir.hip import HipOp


def compile_graph_kernels(compiled: Graph, *, force: bool = False) -> list[str]:
    """Compile every kernel of a lowered graph into the cache; returns their names.
    ``force`` recompiles even when the cache already holds the code object."""
    names = []
    seen = set()
    for nid in compiled.topological_order():
        op = compiled.nodes[nid].op
        if not isinstance(op, HipOp) or op.kernel_name in seen:
            continue
        seen.add(op.kernel_name)
        if force:
            path = hiprtc.cache_dir() / f"{hiprtc.cache_key(op.kernel_source, op.kernel_name, 'gfx950')}.hsaco"
            blob, _ = launcher.load().compile(op.kernel_source, op.kernel_name, "gfx950", hiprtc.effective_flags())
            path.parent.mkdir(parents=True, exist_ok=True)
            tmp = path.with_suffix(".tmp")
            tmp.write_bytes(blob)
            tmp.replace(path)
        else:
            hiprtc.compile_to_hsaco(op.kernel_source, op.kernel_name)
        names.append(op.kernel_name)
    return names


def cache_location() -> str:
    return str(config.hsaco_cache_dir())
