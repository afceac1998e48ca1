"""gfx950 HIP emitters: one module per kernel family, sharing ``prelude``.

Each emitter takes a scheduled tile body (``deplodock_amd.ir.tile``) and
returns a :class:`deplodock_amd.ir.hip.HipOp`: complete source text, the
argument order and the launch geometry.  Together they replace the
reference's Kernel-IR materialization and CUDA renderer
(emmy/compiler/pipeline/passes/lowering/kernel/*, ir/kernel/render.py:407-515).
"""
