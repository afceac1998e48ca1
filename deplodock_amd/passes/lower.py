"""``Graph[TileOp]`` → ``Graph[HipOp]``: render every scheduled tile to gfx950 source.

Counterpart of the reference's last two pass directories
(emmy/compiler/pipeline/__init__.py:46-47: ``lowering/kernel`` then
``lowering/cuda``; 010_lower_kernelop.py renders a KernelOp to a CudaOp).
Kernel names follow the reference's rule ``k_<label>_<hash[:6]>``
(provenance.py:246-252) with the hash taken over the rendered body.
"""

from __future__ import annotations

import hashlib
import logging
from dataclasses import replace

from deplodock_amd.context import Context
from deplodock_amd.emit.contraction import emit_contraction
from deplodock_amd.emit.copy import emit_index_rows, emit_strided_copy
from deplodock_amd.emit.flash import emit_flash
from deplodock_amd.emit.loopnest import emit_loop_nest
from deplodock_amd.emit.pointwise import emit_map
from deplodock_amd.emit.reduce import emit_row_reduce
from deplodock_amd.emit.reduce_stream import emit_row_reduce_streaming
from deplodock_amd.dtype import F32
from deplodock_amd.emit.errors import LoweringError
from deplodock_amd.emit.splitk import emit_splitk_combine, partial_body, split_planes
from deplodock_amd.graph import Graph, Node, Tensor
from deplodock_amd.ir.hip import HipOp
from deplodock_amd.ir.schedule import ReducePlan
from deplodock_amd.ir.tile import Contraction, Flash, IndexRows, LoopNest, Map, RowReduce, StridedCopy, TileOp

_PLACEHOLDER = "EMH_KERNEL_NAME_"
logger = logging.getLogger(__name__)


def _named(hip: HipOp, op: TileOp) -> HipOp:
    label = op.name.split("__")[0]
    digest = hashlib.sha1(hip.kernel_source.encode()).hexdigest()[:6]
    name = f"{label}_{digest}"
    hip.kernel_source = hip.kernel_source.replace(_PLACEHOLDER, name)
    hip.kernel_name = name
    hip.source = op
    hip.knobs = {**op.knobs, **hip.knobs}
    return hip


def _spills(hip: HipOp, ctx: Context) -> int:
    """Vector registers the compiler spilled building ``hip`` (0 without a launcher library: the compile
    step at load time still refuses a spilling ring).  The code object lands in the cache the loader
    reads, so the check costs no second compile."""
    from deplodock_amd.backend.hip import hiprtc, launcher

    try:
        return hiprtc.spilled_vgprs(hip.kernel_source, hip.kernel_name, arch=ctx.arch)
    except launcher.CompileError:
        raise  # a real compile error (it is a LauncherError too, and must not be taken for a missing library)
    except launcher.LauncherError:
        return 0


def _lower_contraction(op: TileOp, ctx: Context) -> HipOp:
    """Render a contraction whose kernel builds without vector-register spills.  A spilling MFMA kernel is
    slow, and wrong where it waits for part of its outstanding loads by count (spill stores share that
    counter).  The schedule's register estimate cannot see every prologue / epilogue, so the code object
    decides: a spilling kernel is rendered again with register staging, then with the heuristic tile — the
    same degrade path an unrealisable pin takes."""
    from deplodock_amd.passes.schedule import default_contraction_schedule

    body = op.body
    hip = _named(emit_contraction(body, _PLACEHOLDER, ctx), op)
    spilled = _spills(hip, ctx)
    if body.stage is None:
        return hip  # not scheduled (a hand-built body): nothing to degrade to
    if spilled and (body.stage.transport != "sync" or body.stage.reg_depth > 1):
        logger.warning("%s: STAGE=%s spills %d vector registers: plain register staging instead", hip.kernel_name, hip.knobs.get("STAGE"), spilled)
        body.stage = replace(body.stage, transport="sync", depth=2, reg_depth=1)
        hip = _named(emit_contraction(body, _PLACEHOLDER, ctx), op)
        spilled = _spills(hip, ctx)
    if spilled:
        logger.warning("%s: TILE=%s spills %d vector registers: the heuristic tile instead", hip.kernel_name, hip.knobs.get("TILE"), spilled)
        default_contraction_schedule(body, ctx)
        hip = _named(emit_contraction(body, _PLACEHOLDER, ctx), op)
        spilled = _spills(hip, ctx)
    # The heuristic tile itself can spill under a heavy output stage (2048 tokens: the 128x256 tile of the q/k/v
    # projection with head norms and rotary embedding in its epilogue): halve the fragments per wave, rows first (the
    # output stage works on whole column groups), until the kernel builds clean.
    from deplodock_amd.ir.schedule import ScheduleError, TilePlan
    from deplodock_amd.passes.schedule import _check_tile, _default_stage

    for _ in range(4):
        if not spilled:
            break
        plan = body.tile
        fm, fn = plan.regs
        shrunk = None
        for regs in ((fm // 2, fn), (fm, fn // 2)):
            if min(regs) < 1 or regs == (fm, fn):
                continue
            cand = TilePlan(atom=plan.atom, units=plan.units, regs=regs, bk=plan.bk)
            try:
                _check_tile(cand, body, ctx, depth=2)
            except ScheduleError:
                continue
            shrunk = cand
            break
        if shrunk is None:
            break
        logger.warning("%s: TILE=%s spills %d vector registers: %s instead", hip.kernel_name, plan.spell(), spilled, shrunk.spell())
        body.tile = shrunk
        body.stage = _default_stage(shrunk, body, ctx)
        hip = _named(emit_contraction(body, _PLACEHOLDER, ctx), op)
        spilled = _spills(hip, ctx)
    return hip


def _lower_split_contraction(graph: Graph, node: Node, ctx: Context) -> None:
    """``REDUCE=g<n>a|k`` on a contraction: the node becomes the combine kernel and gains a producer, the
    partial kernel, whose output is the fp32 workspace (a scratch tensor of the graph) — the two-node form
    of the reference's split rewrite (emmy/compiler/pipeline/passes/lowering/tile/030_split.py:135-334)."""
    op: TileOp = node.op
    body: Contraction = op.body
    label, _, rest = op.name.partition("__")
    ws_id = f"{node.id}__partial"
    if ws_id in graph.nodes:
        raise LoweringError(f"contraction: workspace id {ws_id!r} is taken")
    part = partial_body(body, ws_id)
    part_op = TileOp(name=f"{label}_partial__{rest}", body=part, knobs=dict(op.knobs))
    part_hip = _named(emit_contraction(part, _PLACEHOLDER, ctx), part_op)
    if _spills(part_hip, ctx):
        raise LoweringError(f"{part_hip.kernel_name}: the partial kernel of the split spills vector registers; pin a smaller tile")
    part_hip.knobs = {**part_hip.knobs, "REDUCE": body.reduce.spell()}
    comb_op = TileOp(name=f"{label}_combine__{rest}", body=body, knobs=dict(op.knobs))
    comb_hip = _named(emit_splitk_combine(body, ws_id, _PLACEHOLDER, ctx), comb_op)
    comb_hip.knobs = {**part_hip.knobs}
    graph.nodes[ws_id] = Node(ws_id, part_hip, [body.a, body.b], Tensor(ws_id, (split_planes(body), body.m, body.n), F32))
    node.op = comb_hip
    node.inputs = [ws_id, *node.inputs]


def _lower_split_row_reduce(graph: Graph, node: Node, ctx: Context) -> None:
    """``REDUCE=g<n>k`` on a row reduction with one value per row (``sum`` / ``mean`` / ``amax`` over the last axis, or
    any single statistic followed by a projection of it): the columns of a row are split into ``n`` contiguous slices.
    Slice j of row r is row ``r * n + j`` of the same buffer seen as ``[rows * n, cols / n]``, so the *partial* kernel is
    the ordinary row kernel over that view with the bare statistic as its output (an fp32 ``[rows, n]`` workspace), and
    the *combine* kernel is the ordinary row kernel over the workspace with the same monoid and the original projection —
    applied once, after the cross-workgroup fold, so it need not distribute over it (the reference's deferred kernel
    finalize, tests/compiler/e2e/test_reduce_coverage.py:280-345)."""
    from deplodock_amd.ir import expr as E
    from deplodock_amd.ir.tile import RowAddr, Stat
    from deplodock_amd.passes.schedule import pick_coop

    op: TileOp = node.op
    body: RowReduce = op.body
    n = body.reduce.cta
    (stat,) = body.stats
    label, _, rest = op.name.partition("__")
    ws_id = f"{node.id}__partial"
    if ws_id in graph.nodes:
        raise LoweringError(f"row reduce: workspace id {ws_id!r} is taken")
    addr = body.x_addr or RowAddr.uniform(body.cols)
    width = body.cols // n
    part = RowReduce(
        rows=body.rows * n, cols=width, x=body.x, x_dtype=body.x_dtype, out=ws_id, out_dtype=F32, stats=(stat,), project=E.Var(stat.name),
        x_addr=RowAddr(offset=addr.offset, div=n, stride_hi=addr.stride_hi, stride_lo=width), scalar_out=True, nontemporal=body.nontemporal,
        reduce=ReducePlan(coop=pick_coop(width, body.x_dtype.nbytes, body.rows * n, ctx, rotate=False, stats=1)),
    )  # fmt: skip
    comb = RowReduce(
        rows=body.rows, cols=n, x=ws_id, x_dtype=F32, out=body.out, out_dtype=body.out_dtype, stats=(Stat(stat.name, stat.monoid, E.Var("x")),), project=body.project,
        out_addr=body.out_addr, scalar_out=True, reduce=ReducePlan(coop=pick_coop(n, 4, body.rows, ctx, rotate=False, stats=1)),
    )  # fmt: skip
    part_hip = _named(emit_row_reduce(part, _PLACEHOLDER, ctx), TileOp(name=f"{label}_partial__{rest}", body=part, knobs=dict(op.knobs)))
    comb_hip = _named(emit_row_reduce(comb, _PLACEHOLDER, ctx), TileOp(name=f"{label}_combine__{rest}", body=comb, knobs=dict(op.knobs)))
    part_hip.knobs = {**part_hip.knobs, "REDUCE": body.reduce.spell()}
    comb_hip.knobs = {**comb_hip.knobs, "REDUCE": body.reduce.spell()}
    graph.nodes[ws_id] = Node(ws_id, part_hip, list(node.inputs), Tensor(ws_id, (body.rows, n), F32))
    node.op = comb_hip
    node.inputs = [ws_id]


def _lower_split_flash(graph: Graph, node: Node, ctx: Context) -> None:
    """``REDUCE=g<n>k`` on attention: the node becomes the combine kernel and gains a producer, the partial kernel, whose
    output is the fp32 workspace ``[slices, batch, heads, queries, head_dim + 4]`` (``head_dim`` unnormalised output
    values, the slice's row maximum and row sum, padding to whole 16-byte rows) — the two-node form of the reference's
    split rewrite (emmy/compiler/pipeline/passes/lowering/tile/030_split.py:217-334)."""
    import dataclasses

    from deplodock_amd.emit.flash import emit_flash_combine, flash_partial_slices

    op: TileOp = node.op
    body: Flash = op.body
    label, _, rest = op.name.partition("__")
    ws_id = f"{node.id}__partial"
    if ws_id in graph.nodes:
        raise LoweringError(f"flash: workspace id {ws_id!r} is taken")
    part = dataclasses.replace(body, partials=ws_id, pair=False)
    part_op = TileOp(name=f"{label}_partial__{rest}", body=part, knobs=dict(op.knobs))
    part_hip = _lower_flash(part_op, ctx)
    slices = flash_partial_slices(part)
    comb_op = TileOp(name=f"{label}_combine__{rest}", body=body, knobs=dict(op.knobs))
    comb_hip = _named(emit_flash_combine(part, ws_id, _PLACEHOLDER, ctx), comb_op)
    comb_hip.knobs = {**part_hip.knobs}
    inputs = [i for i in node.inputs]
    graph.nodes[ws_id] = Node(ws_id, part_hip, inputs, Tensor(ws_id, (slices, body.batch, body.q_heads, body.q_len, body.head_dim + 4), F32))
    node.op = comb_hip
    node.inputs = [ws_id]


def _lower_flash(op: TileOp, ctx: Context) -> HipOp:
    """The attention kernel waits for part of its outstanding direct-to-LDS loads by count, as the contraction's
    rings do, so it must build without vector-register spills too.  A schedule that spills gives up, in turn: the
    pairwise unrolling of its key steps, the mirrored query-block pairing, and finally its shape for the smallest
    one (two row groups x four key-split groups on 32-key blocks)."""
    body = op.body
    hip = _named(emit_flash(body, _PLACEHOLDER, ctx), op)
    from deplodock_amd.emit.flash_f32 import on_f32_atoms

    if on_f32_atoms(body):
        return hip  # one shape, sized to a wave's registers for every head_dim it takes
    if body.private:
        if _spills(hip, ctx):
            raise LoweringError(f"{hip.kernel_name}: the key-split-waves form spills vector registers")
        return hip
    steps = (("pair_steps", False), ("pair", False), ("shape", None))
    for what, value in steps:
        spilled = _spills(hip, ctx)
        if not spilled:
            break
        if what == "shape":
            if (body.waves, body.block_kv, body.kv_split) == (2, 32, 4):
                break
            body.waves, body.block_kv, body.kv_split, body.deep = 2, 32, 4, False
        elif getattr(body, what) == value:
            continue
        else:
            setattr(body, what, value)
        logger.warning("%s: FLASH=%s spills %d vector registers: rendered again without %s", hip.kernel_name, hip.knobs.get("FLASH"), spilled, {"pair_steps": "pairwise key steps", "pair": "query-block pairs", "shape": "its wave shape"}[what])
        try:
            hip = _named(emit_flash(body, _PLACEHOLDER, ctx), op)
        except LoweringError:
            break
    return hip


def lower_tile(op: TileOp, ctx: Context) -> HipOp:
    body = op.body
    if isinstance(body, Contraction):
        return _lower_contraction(op, ctx)
    if isinstance(body, RowReduce):
        hip = (emit_row_reduce_streaming if body.stream else emit_row_reduce)(body, _PLACEHOLDER, ctx)
    elif isinstance(body, Flash):
        hip = _lower_flash(op, ctx)
        return hip
    elif isinstance(body, Map):
        hip = emit_map(body, _PLACEHOLDER, ctx)
    elif isinstance(body, LoopNest):
        hip = emit_loop_nest(body, _PLACEHOLDER, ctx)
    elif isinstance(body, StridedCopy):
        hip = emit_strided_copy(body, _PLACEHOLDER, ctx)
    elif isinstance(body, IndexRows):
        hip = emit_index_rows(body, _PLACEHOLDER, ctx)
    else:
        raise TypeError(f"unknown tile body {type(body).__name__}")
    return _named(hip, op)


def lower(graph: Graph, ctx: Context | None = None) -> Graph:
    """Replace every ``TileOp`` by its ``HipOp`` (in place) and return the graph."""
    ctx = ctx or Context()
    for node in list(graph.nodes.values()):
        if isinstance(node.op, TileOp):
            if isinstance(node.op.body, Contraction) and node.op.body.reduce.cta > 1:
                _lower_split_contraction(graph, node, ctx)
            elif isinstance(node.op.body, Flash) and node.op.body.kv_ctas > 1:
                _lower_split_flash(graph, node, ctx)
            elif isinstance(node.op.body, RowReduce) and node.op.body.reduce.cta > 1:
                _lower_split_row_reduce(graph, node, ctx)
            else:
                node.op = lower_tile(node.op, ctx)
    return graph
