"""Frontend graph → graph of tile kernels (which ops become one kernel).

Decides the kernel boundaries.  The reference reaches the same boundaries by
decomposing frontend ops to primitives and re-fusing loops
(emmy/compiler/pipeline/passes/frontend/decomposition/*, passes/loop/fusion/010_merge_loop_ops.py:48-183,
recognizers passes/lowering/tile/010_recognize.py, _flash.py:478-571, _softmax.py:35-123);
here recognizers match the traced ops directly, walking back from each value
that must exist in memory:

* ``add(residual, linear)``                       → contraction with a residual post-epilogue
* ``silu(linear(x, Wg)) * linear(x, Wu)``          → one gate/up contraction (weights stacked at bind time)
* ``linear``                                      → contraction
* RMSNorm, as one op or as the traced primitive chain
  ``w * bf16(f32(x) * rsqrt(mean(f32(x)^2) + eps))`` → row reduce
* rotary embedding ``t*cos + cat(-t_hi, t_lo)*sin`` → fused into the norm that feeds it, or a row map
* ``softmax``                                     → row reduce with the (max, sum-exp) carrier
* ``scaled_dot_product_attention``                → flash kernel addressing q/k/v/out through strides
* anything else element-wise                       → pointwise map

Layout ops never become kernels (``passes.views``).  The over-fusion the
reference reports for whole-model traces (four mega-kernels holding 97 % of the
forward, plans/qwen3-embedding-06b-tune-findings.md:42-57) is avoided by
construction: a reduction never absorbs a following contraction.
"""

from __future__ import annotations

import math
from dataclasses import dataclass, field

from deplodock_amd.dtype import BF16, F16, F32, DType
from deplodock_amd.graph import Graph, Node, Tensor
from deplodock_amd.ir import expr as E
from deplodock_amd.ir import frontend as F
from deplodock_amd.ir.base import ConstantOp, InputOp
from deplodock_amd.ir.tile import Contraction, Flash, Map, MapOperand, RotateHalf, RowAddr, RowEpilogue, RowOperand, RowPrologue, RowReduce, Stat, TileOp
from deplodock_amd.passes.views import LAYOUT_OPS, NotViewable, View, apply_layout, contiguous_strides, resolve_view


class FusionError(NotImplementedError):
    """No kernel recognizer covers a traced op (or its layout needs a copy this build lacks)."""


def _round(dtype: DType, e: E.Expr) -> E.Expr:
    """Round to ``dtype`` storage and widen again (identity for fp32)."""
    return e if dtype is F32 else E.Round(dtype.name, e)


@dataclass
class StackedConstant:
    """A constant the runtime assembles at bind time by stacking other constants
    along dim 0 (the reference folds such layout work into ``ConstantOp.load_ops``,
    emmy/compiler/ir/base.py:118-160)."""

    parts: tuple[str, ...]
    k_scale: str | None = None  # a length-k constant multiplied into every row (a norm weight folded into the projection)
    transpose: bool = False  # the last two axes swapped afterwards (a ``[K, N]`` weight of ``x @ w`` stored as the ``[N, K]`` rows a contraction reads)
    pad_rows_to: int = 0  # zero rows appended up to this many (an output width that is not whole runs of four columns: a 151 669-word vocabulary)


@dataclass
class _Ctx:
    g: Graph
    out: Graph
    done: dict[str, str] = field(default_factory=dict)  # frontend node id -> lowered buffer id
    names: dict[str, int] = field(default_factory=dict)
    # frontend node id -> (offset, shape, strides) of its value inside ``done[id]``
    # when it is a window of a wider buffer (column slice of a merged projection)
    windows: dict[str, tuple[int, tuple[int, ...], tuple[int, ...]]] = field(default_factory=dict)
    dense: dict[str, View] = field(default_factory=dict)  # layout node id -> its value after a dense copy made it expressible

    def kname(self, label: str) -> str:
        """Kernel label; the lowering appends a hash of the rendered body, so
        identical kernels (e.g. the k and v projections) share one name."""
        return f"k_{label}"

    def single_use(self, nid: str) -> bool:
        return len(self.g.consumers(nid)) == 1 and nid not in self.g.outputs

    def producer(self, nid: str) -> Node:
        return self.g.nodes[nid]


def _is(node: Node, cls, **attrs) -> bool:
    return isinstance(node.op, cls) and all(getattr(node.op, k) == v for k, v in attrs.items())


def _peel_layout(g: Graph, nid: str) -> str:
    """Follow layout ops back to the node that owns the memory."""
    while isinstance(g.nodes[nid].op, LAYOUT_OPS):
        nid = g.nodes[nid].inputs[0]
    return nid


# ---------------------------------------------------------------------------
# Recognizers (each returns True when it emitted a kernel for ``nid``)
# ---------------------------------------------------------------------------


def _need(c: _Ctx, nid: str) -> View:
    """Make sure the value of frontend node ``nid`` exists in memory; return how
    to address it.  Honours a producer that stored its result in another memory
    order than its logical shape (rope, sdpa): the layout chain between that
    producer and ``nid`` is replayed on top of the stored layout."""
    g = c.g
    chain = []
    cur = nid
    while isinstance(g.nodes[cur].op, LAYOUT_OPS):
        chain.append(cur)
        cur = g.nodes[cur].inputs[0]
    _materialize(c, cur)
    base = c.done[cur]
    hint = c.out.nodes[base].hints.get("logical_view")
    if cur in c.windows:
        offset, shape, strides = c.windows[cur]
        v = View(base, offset, shape, strides, g.nodes[cur].output.dtype)
    elif hint is not None:
        shape, strides = hint
        v = View(base, 0, tuple(shape), tuple(strides), g.nodes[cur].output.dtype)
    else:
        shape = tuple(int(d) for d in g.nodes[cur].output.shape)
        v = View(base, 0, shape, contiguous_strides(shape), g.nodes[cur].output.dtype)
    for lid in reversed(chain):
        if lid in c.dense:
            v = c.dense[lid]
            continue
        try:
            v = apply_layout(v, g.nodes[lid].op, tuple(int(d) for d in g.nodes[lid].output.shape), lid)
        except NotViewable:
            # e.g. ``x.transpose(1, 2).reshape(...)``: no strides express it, so the view so far is written out
            # densely by a copy nest (what torch's reshape does) and the layout op applies to the copy
            if not all(isinstance(d, int) for d in (*v.shape, *v.strides, v.offset)):
                raise
            dense = _copy_of_view(c, v, tuple(range(len(v.shape))), f"{lid}__dense")
            v = c.dense[lid] = apply_layout(dense, g.nodes[lid].op, tuple(int(d) for d in g.nodes[lid].output.shape), lid)
    return v


def _materialize(c: _Ctx, nid: str) -> None:
    if nid in c.done:
        return
    node = c.g.nodes[nid]
    if isinstance(node.op, (InputOp, ConstantOp)):
        t = node.output
        if isinstance(node.op, InputOp):
            c.out.add_input(nid, t.shape, t.dtype)
        else:
            c.out.add_constant(nid, t.shape, t.dtype, value=node.op.value, source_path=node.op.source_path)
        c.done[nid] = nid
        return
    for rec in (_rec_same_type_cast, _rec_loop_nest, _rec_batched_linear, _rec_matmul_residual, _rec_matmul_gated, _rec_matmul, _rec_linear_residual, _rec_gate_up, _rec_gate_up_f32, _rec_linear_siblings, _rec_linear, _rec_rope_pair, _rec_rope, _rec_rms_chain, _rec_rms_op, _rec_layer_norm, _rec_softmax, _rec_sdpa, _rec_row_fused, _rec_row_sum, _rec_gather, _rec_cat, _rec_pointwise):
        if rec(c, nid):
            return
    raise FusionError(f"no kernel recognizer for {type(node.op).__name__} at node {nid!r}")


def _rec_same_type_cast(c: _Ctx, nid: str) -> bool:
    """``x.to(dtype)`` where ``x`` already has that type (an fp32 model's ``hidden_states.to(torch.float32)``): no
    kernel, the node is another name for its operand's memory."""
    node = c.g.nodes[nid]
    if not isinstance(node.op, F.CastOp) or c.g.nodes[node.inputs[0]].output.dtype != node.output.dtype:
        return False
    v = _need(c, node.inputs[0])
    c.done[nid] = v.base
    c.windows[nid] = (v.offset, tuple(v.shape), tuple(v.strides))
    return True


def _rec_loop_nest(c: _Ctx, nid: str) -> bool:
    """A Loop-IR kernel of the reference: its operands are materialised as plain row-major tensors of their
    recorded shapes and the statements go to the loop-nest emitter as they stand."""
    node = c.g.nodes[nid]
    if not isinstance(node.op, F.LoopNestOp):
        return False
    from deplodock_amd.ir.tile import LoopNest

    from deplodock_amd.ir import loopnest as L

    operands: dict = {}
    inputs: list[str] = []
    strided: dict[str, View] = {}
    for load_name, src in zip(node.op.loads, node.inputs):
        shape = tuple(int(d) for d in c.g.nodes[src].output.shape)
        v = _need_logical(c, src)
        if (v.offset == 0 and v.shape == shape and v.is_contiguous()) or _same_memory(v, shape):
            operands[load_name] = (v.base, shape, c.g.nodes[src].output.dtype)
        else:
            # a strided view: the buffer is indexed flat and every Load of it computes offset + sum(index * stride)
            if tuple(int(d) for d in v.shape) != shape:
                raise FusionError(f"loop nest {nid!r}: operand {src!r} is a view of shape {v.shape}, recorded as {shape}")
            operands[load_name] = (v.base, (int(c.out.nodes[v.base].output.numel),), c.g.nodes[src].output.dtype)
            strided[load_name] = v
        inputs.append(v.base)

    def flat(stmts: tuple) -> tuple:
        res = []
        for s in stmts:
            if isinstance(s, L.Loop):
                s = L.Loop(s.axis, s.extent, flat(s.body))
            elif isinstance(s, L.Load) and s.input in strided:
                v = strided[s.input]
                if len(s.index) != len(v.strides):
                    raise FusionError(f"loop nest {nid!r}: load of {s.input!r} has {len(s.index)} indices for a rank-{len(v.strides)} operand")
                at: object = L.Lit(int(v.offset))
                for e, st in zip(s.index, v.strides):
                    if st and not (isinstance(e, L.Lit) and e.value == 0):
                        at = L.Bin("+", at, L.Bin("*", e, L.Lit(int(st))))
                s = L.Load(s.name, s.input, (at,))
            res.append(s)
        return tuple(res)

    t = node.output
    body = LoopNest(stmts=flat(node.op.stmts) if strided else node.op.stmts, operands=operands, scalars=dict(node.op.scalars or {}), out=nid, out_name=node.op.out_name or nid,
                    out_shape=tuple(int(d) for d in t.shape), out_dtype=t.dtype)  # fmt: skip
    label = node.op.label or "".join(ch if ch.isalnum() else "_" for ch in nid)[-40:].lstrip("_")
    _emit(c, nid, body, label, inputs)
    return True


def _emit(c: _Ctx, nid: str, body, label: str, inputs: list[str], shape=None, dtype=None) -> None:
    node = c.g.nodes[nid]
    t = Tensor(nid, shape if shape is not None else node.output.shape, dtype or node.output.dtype)
    c.out.add_node(TileOp(name=c.kname(label), body=body), list(dict.fromkeys(inputs)), t, nid)
    c.done[nid] = nid


def _matrix(view: View, what: str) -> tuple[int, int, int]:
    """``view`` as a row-major matrix ``[rows, cols]``: returns ``(rows, cols, ld)``."""
    if view.strides[-1] != 1 and view.shape[-1] != 1:
        raise FusionError(f"{what}: innermost dimension must be contiguous")
    lead = view.collapse_leading(1)
    if lead is None:
        raise FusionError(f"{what}: leading dimensions do not collapse to one stride")
    rows, ld = lead
    return rows, view.shape[-1], (ld if rows > 1 else view.shape[-1])


def _a_operand(c: _Ctx, x_id: str, absorbers: set[str], fold: bool = False) -> tuple[View, RowPrologue | None, list[str], str | None]:
    """The ``a`` operand of a contraction: ``(view, prologue, extra input buffers, weight to fold)``.

    When ``x_id`` is a row RMSNorm of 16-bit rows that nothing but the
    contractions in ``absorbers`` reads, the norm is not materialised: the view
    is the norm's *input* and the prologue carries its statistic and projection
    (with the producer's rounding points), so ``norm -> linear`` is one launch.

    With ``fold`` the caller's ``b`` operand is a constant it assembles itself: the
    normalisation is then deferred (``RowPrologue.scale``) and the fourth value names
    the norm weight (a constant vector, or ``None``) the caller multiplies into the
    columns of ``b``."""
    g = c.g
    node = g.nodes[x_id]
    if x_id not in c.done and x_id not in g.outputs and not (set(g.consumers(x_id)) - absorbers):
        m = None
        if isinstance(node.op, F.RmsNormOp):
            m = _RmsMatch(x=node.inputs[0], weight=node.inputs[1] if node.op.has_weight else None, eps=node.op.eps, inner=F32, cols=int(node.output.shape[-1]))
        elif len(node.output.shape) >= 2:
            m = _match_rms_chain(c, x_id)
        if m is not None and node.output.dtype.nbytes == 2 and m.cols % 32 == 0:  # (whole MFMA steps: a short last slab is not transformed)
            try:
                body, inputs, xv = _rms_body(c, x_id, m, node.output.dtype)
            except FusionError:
                body = None
            if body is not None and isinstance(node.op, F.RmsNormOp) and m.weight is not None:
                body.project = E.Var("x") * E.Un("rsqrt", E.Var("ss") / float(m.cols) + m.eps) * E.Var("w")
            if body is not None and xv.dtype == node.output.dtype and body.x_addr.div == 1 and body.x_addr.stride_hi % 8 == 0 and body.x_addr.offset % 8 == 0:
                wbuf = body.operand_buffers.get("w")
                wdt = body.col_operands[0][1] if body.col_operands else None
                if wbuf is None or wdt.nbytes == 2:
                    view = View(xv.base, body.x_addr.offset, (body.rows, m.cols), (body.x_addr.stride_hi, 1), xv.dtype)
                    w_node = g.nodes[_peel_layout(g, m.weight)] if m.weight is not None else None
                    if fold and (w_node is None or (isinstance(w_node.op, ConstantOp) and w_node.id == m.weight)):
                        scale = E.Un("rsqrt", E.Var("ss") / float(m.cols) + m.eps)
                        return view, RowPrologue(stat_pre=body.stats[0].pre, project=body.project, scale=scale), [], m.weight
                    return view, RowPrologue(stat_pre=body.stats[0].pre, project=body.project, weight=wbuf, weight_dtype=wdt), ([wbuf] if wbuf else []), None
    return _need(c, x_id), None, [], None


def _transposed_parameter(c: _Ctx, w: View) -> View:
    """``w`` as ``[N, K]`` rows when it is the transposed view of a dense ``[K, N]`` parameter: the transposition is
    done once, when the program is bound (a constant assembled from the parameter), instead of by a copy per run."""
    base = c.out.nodes.get(w.base)
    if len(w.shape) != 2 or w.strides[-1] == 1 or base is None or not isinstance(base.op, ConstantOp) or base.op.value is not None:
        return w
    n, k = int(w.shape[0]), int(w.shape[1])
    if w.offset != 0 or tuple(w.strides) != (1, n) or tuple(int(d) for d in base.output.shape) != (k, n):
        return w
    tid = f"{w.base}__t"
    if tid not in c.out.nodes:
        c.out.add_constant(tid, (n, k), w.dtype)
        c.out.nodes[tid].hints["stacked"] = StackedConstant((w.base,), transpose=True)
    return View(tid, 0, (n, k), (k, 1), w.dtype)


def _linear_parts(c: _Ctx, nid: str):
    node = c.g.nodes[nid]
    x, pro, extra, _ = _a_operand(c, node.inputs[0], {nid})
    w = _transposed_parameter(c, _need(c, node.inputs[1]))
    m, k, lda = _matrix(x, "linear input")
    n, k2, ldb = _matrix(w, "linear weight")
    if k != k2:
        raise FusionError("linear: inner dimensions differ")
    return x, w, m, n, k, lda, ldb, pro, extra


def _bias_of(c: _Ctx, nid: str, n: int) -> dict:
    """Contraction keyword arguments that add the linear's bias to the fp32
    accumulator before the single rounding to the output type."""
    node = c.g.nodes[nid]
    if not node.op.has_bias:
        return {}
    b = _need(c, node.inputs[2])
    if b.numel != n or not b.is_contiguous() or b.offset % 4 or n % 4:
        raise FusionError("linear: the bias must be a dense length-n vector (n a multiple of 4)")
    return {"bias": b.base, "bias_dtype": b.dtype, "epilogue": E.Var("acc") + E.Var("bias")}


def _rec_linear(c: _Ctx, nid: str) -> bool:
    node = c.g.nodes[nid]
    if not isinstance(node.op, F.LinearOp):
        return False
    x, w, m, n, k, lda, ldb, pro, extra = _linear_parts(c, nid)
    if n % 4 and not node.op.has_bias:
        # The contraction stores runs of four columns: the weight gets zero rows up to the next multiple of four (a
        # parameter: once, at bind time; else by the copy kernel) and the result is a window of the wider buffer.
        n_pad = -(-n // 4) * 4
        base = c.out.nodes.get(w.base)
        if isinstance(base.op, ConstantOp) and base.op.value is None and w.offset == 0 and tuple(w.strides) == (k, 1):
            pid = f"{w.base}__rows{n_pad}"
            if pid not in c.out.nodes:
                c.out.add_constant(pid, (n_pad, k), w.dtype)
                c.out.nodes[pid].hints["stacked"] = StackedConstant((w.base,), pad_rows_to=n_pad)
            w = View(pid, 0, (n_pad, k), (k, 1), w.dtype)
        else:
            w = _copy_of_view(c, w, (0, 1), f"{nid}__w", pad_rows_to=n_pad)
        lead = tuple(int(d) for d in node.output.shape[:-1])
        body = Contraction(m=m, n=n_pad, k=k, a=x.base, b=w.base, out=nid, in_dtype=x.dtype, out_dtype=node.output.dtype, lda=lda, ldb=k, a_offset=x.offset, b_offset=0, a_prologue=pro)
        _emit(c, nid, body, "rms_norm_linear" if pro else "linear", [x.base, w.base, *extra], shape=(*lead, n_pad))
        c.windows[nid] = (0, (*lead, n), contiguous_strides((*lead, n_pad)))
        return True
    bias = _bias_of(c, nid, n)
    body = Contraction(m=m, n=n, k=k, a=x.base, b=w.base, out=nid, in_dtype=x.dtype, out_dtype=node.output.dtype, lda=lda, ldb=ldb, a_offset=x.offset, b_offset=w.offset, a_prologue=pro, **bias)
    _emit(c, nid, body, "rms_norm_linear" if pro else "linear", [x.base, w.base, *extra, *([bias["bias"]] if bias else [])])
    return True


def _rec_batched_linear(c: _Ctx, nid: str) -> bool:
    """``[P, M, K] x [P | 1, N, K] -> [P, M, N]``: one launch, product ``p`` on workgroup row ``p``."""
    node = c.g.nodes[nid]
    if not isinstance(node.op, F.BatchedLinearOp):
        return False
    x, w = _need(c, node.inputs[0]), _need(c, node.inputs[1])
    if len(x.shape) != 3 or len(w.shape) != 3 or x.shape[2] != w.shape[2] or w.shape[0] not in (1, x.shape[0]):
        raise FusionError(f"batched linear {nid!r}: operands {x.shape} x {w.shape} are not [P, M, K] x [P | 1, N, K]")
    _emit_batched_contraction(c, nid, x, w, "batched_linear")
    return True


def _copy_of_view(c: _Ctx, v: View, order: tuple[int, ...], new_id: str, pad_last_to: int | None = None, pad_rows_to: int | None = None) -> View:
    """A dense row-major copy of ``v`` with its axes in ``order``, made by a copy kernel of its own (``new_id``): what
    a contraction needs when an operand's reduction axis is not the contiguous one, or its leading axes are not one
    uniformly strided run.  The last axis (``pad_last_to``) and the one before it (``pad_rows_to``) can be extended
    with zeros."""
    from deplodock_amd.ir.tile import StridedCopy

    axes = [[int(v.shape[i]), int(v.shape[i]), int(v.strides[i])] for i in order]
    if pad_last_to is not None and pad_last_to > axes[-1][0]:
        axes[-1][0] = int(pad_last_to)
    if pad_rows_to is not None and len(axes) > 1 and pad_rows_to > axes[-2][0]:
        axes[-2][0] = int(pad_rows_to)
    shape = tuple(a[0] for a in axes)
    body = StridedCopy(src=v.base, out=new_id, dtype=v.dtype, src_offset=int(v.offset), src_numel=int(c.out.nodes[v.base].output.numel), axes=tuple(tuple(a) for a in axes))
    c.out.add_node(TileOp(name=c.kname("gather"), body=body), [v.base], Tensor(new_id, shape, v.dtype), new_id)
    return View(new_id, 0, shape, contiguous_strides(shape), v.dtype)


def _emit_batched_contraction(c: _Ctx, nid: str, a: View, b: View, label: str, residual: View | None = None, post: E.Expr | None = None) -> None:
    """``a [..., M, K] x b [... | 1..., N, K] -> [..., M, N]`` as one launch with a workgroup row per product.  The
    kernel reads whole 16-byte chunks along ``K`` and stores runs of four columns: an operand that is not laid out
    for that (reduction axis not contiguous, leading axes not one uniformly strided run, misaligned) is copied
    first; a ragged ``K`` is padded with zeros in both operands; a ragged ``N`` is padded in ``b`` and the result
    is a window of a wider buffer."""
    node = c.g.nodes[nid]
    m, k, n = int(a.shape[-2]), int(a.shape[-1]), int(b.shape[-2])
    lead = tuple(int(d) for d in a.shape[:-2])
    p = 1
    for d in lead:
        p *= d
    shared = all(int(d) == 1 for d in b.shape[:-2])
    if not shared and tuple(int(d) for d in b.shape[:-2]) != lead:
        raise FusionError(f"{label} {nid!r}: leading axes {a.shape[:-2]} and {b.shape[:-2]} differ")
    if a.dtype != b.dtype:
        raise FusionError(f"{label} {nid!r}: operand types differ")
    kp, n_pad = -(-k // 8) * 8, -(-n // 4) * 4
    nb = a.dtype.nbytes

    def unfit(v: View, rows: int) -> bool:
        return v.strides[-1] != 1 and k > 1 or v.collapse_leading(2) is None or (v.offset * nb) % 16 != 0 or (rows > 1 and (v.strides[-2] * nb) % 16 != 0)

    if kp != k or unfit(a, m):
        a = _copy_of_view(c, a, tuple(range(len(a.shape))), f"{nid}__a", pad_last_to=kp)
    if kp != k or n_pad != n or unfit(b, n):
        b = _copy_of_view(c, b, tuple(range(len(b.shape))), f"{nid}__b", pad_last_to=kp, pad_rows_to=n_pad)
    pa, sa = a.collapse_leading(2)
    pb, sb = b.collapse_leading(2)
    if (pa > 1 and (sa * nb) % 16) or (pb > 1 and (sb * nb) % 16):
        raise FusionError(f"{label} {nid!r}: batch strides break 16-byte alignment")
    body = Contraction(
        m=m, n=n_pad, k=kp, a=a.base, b=b.base, out=nid, in_dtype=a.dtype, out_dtype=node.output.dtype, lda=int(a.strides[-2]) if m > 1 else kp, ldb=int(b.strides[-2]) if n_pad > 1 else kp,
        a_offset=a.offset, b_offset=b.offset, batch=p, a_batch=int(sa) if p > 1 else 0, b_batch=0 if shared or p == 1 else int(sb), out_batch=m * n_pad,
        # ``residual``: a tensor of the result's shape read in the output stage as ``res``; ``post`` says what it does there (default: added)
        **({"post": post if post is not None else E.Var("y") + E.Var("res"), "epilogue_operands": (("res", node.output.dtype),)} if residual is not None else {}),
    )  # fmt: skip
    if residual is not None:
        if p != 1 or n_pad != n:
            raise FusionError(f"{label} {nid!r}: a residual rides on a single unpadded product")
        body.operand_buffers = {"res": residual.base}
    _emit(c, nid, body, label, [a.base, b.base, *([residual.base] if residual is not None else [])], shape=(*lead, m, n_pad))
    if n_pad != n:
        c.windows[nid] = (0, (*lead, m, n), contiguous_strides((*lead, m, n_pad)))


def _rec_matmul_residual(c: _Ctx, nid: str) -> bool:
    """``a @ w + residual`` with a single product (the reference's ``matmul_add`` perf cases, tests/perf/cases.py:193-210:
    o_proj / down_proj + residual as one launch): the residual is added to the accumulator in the contraction's output
    stage, as ``_rec_linear_residual`` does for ``F.linear``."""
    node = c.g.nodes[nid]
    if not (_is(node, F.ElementwiseOp, fn="add") and len(node.inputs) == 2):
        return False
    for mi, ri in ((0, 1), (1, 0)):
        mm_id, res_id = node.inputs[mi], node.inputs[ri]
        mm = c.g.nodes[mm_id]
        if not (isinstance(mm.op, F.MatmulOp) and c.single_use(mm_id)) or mm_id in c.done or mm_id in c.g.outputs:
            continue
        ta, tb = c.g.nodes[mm.inputs[0]].output, c.g.nodes[mm.inputs[1]].output
        if len(tb.shape) != 2 or len(ta.shape) < 2 or not all(isinstance(d, int) for d in (*ta.shape, *tb.shape)):
            continue
        if math.prod(int(d) for d in ta.shape[:-2]) != 1 or int(tb.shape[1]) % 4 or int(tb.shape[0]) % 8:
            continue
        rt_ = c.g.nodes[res_id].output
        if tuple(rt_.shape) != tuple(node.output.shape) or tuple(mm.output.shape) != tuple(node.output.shape) or rt_.dtype != node.output.dtype or mm.output.dtype != node.output.dtype:
            continue
        res = _need(c, res_id)
        if not res.is_contiguous() or res.offset:
            continue
        a, b = _need(c, mm.inputs[0]), _need(c, mm.inputs[1])
        bt = _transposed_parameter(c, View(b.base, b.offset, (b.shape[1], b.shape[0]), (b.strides[1], b.strides[0]), b.dtype))
        if len(a.shape) > 2:
            bt = View(bt.base, bt.offset, (*(1,) * (len(a.shape) - 2), *bt.shape), (*(0,) * (len(a.shape) - 2), *bt.strides), bt.dtype)
        _emit_batched_contraction(c, nid, a, bt, "matmul_add", residual=res)
        return True
    return False


def _rec_matmul_gated(c: _Ctx, nid: str) -> bool:
    """``act(x @ wg) * (x @ wu)`` with run-time weights (the reference's ``gated_mlp`` perf cases,
    tests/perf/cases.py:213-232): the gate product is a contraction of its own and the activation (rounded where the
    module rounds it) and the product with it ride in the output stage of the up contraction — two launches instead of
    two contractions and a map.  (``F.linear`` over constant 16-bit weights takes the paired tile of ``_rec_gate_up``.)"""
    node = c.g.nodes[nid]
    if not (_is(node, F.ElementwiseOp, fn="mul") and len(node.inputs) == 2):
        return False
    od = node.output.dtype
    for si, ui in ((0, 1), (1, 0)):
        act, up = c.g.nodes[node.inputs[si]], c.g.nodes[node.inputs[ui]]
        if not (isinstance(act.op, F.ElementwiseOp) and act.op.fn in ("silu", "gelu_tanh", "gelu") and len(act.inputs) == 1 and c.single_use(act.id) and act.id not in c.g.outputs):
            continue
        gate = c.g.nodes[act.inputs[0]]
        if not (isinstance(gate.op, F.MatmulOp) and isinstance(up.op, F.MatmulOp) and c.single_use(gate.id) and c.single_use(up.id)) or up.id in c.done or up.id in c.g.outputs or gate.id in c.g.outputs:
            continue
        ta, tb = c.g.nodes[up.inputs[0]].output, c.g.nodes[up.inputs[1]].output
        if len(tb.shape) != 2 or len(ta.shape) < 2 or not all(isinstance(d, int) for d in (*ta.shape, *tb.shape)):
            continue
        if math.prod(int(d) for d in ta.shape[:-2]) != 1 or int(tb.shape[1]) % 4 or int(tb.shape[0]) % 8:
            continue
        if tuple(gate.output.shape) != tuple(node.output.shape) or tuple(up.output.shape) != tuple(node.output.shape) or gate.output.dtype != od or up.output.dtype != od or act.output.dtype != od:
            continue
        g_view = _need(c, gate.id)
        if not g_view.is_contiguous() or g_view.offset:
            continue
        a, b = _need(c, up.inputs[0]), _need(c, up.inputs[1])
        bt = _transposed_parameter(c, View(b.base, b.offset, (b.shape[1], b.shape[0]), (b.strides[1], b.strides[0]), b.dtype))
        if len(a.shape) > 2:
            bt = View(bt.base, bt.offset, (*(1,) * (len(a.shape) - 2), *bt.shape), (*(0,) * (len(a.shape) - 2), *bt.strides), bt.dtype)
        _emit_batched_contraction(c, nid, a, bt, f"matmul_{act.op.fn}_mul", residual=g_view, post=_round(od, E.Un(act.op.fn, E.Var("res"))) * E.Var("y"))
        return True
    return False


def _rec_matmul(c: _Ctx, nid: str) -> bool:
    """``[..., M, K] @ [..., K, N]``: one (batched) contraction.  The contraction reads both operands along their
    reduction axis, so ``b`` is taken as ``[N, K]`` rows: a ``k.transpose(-1, -2)`` already is that in memory; a
    plain ``[K, N]`` operand (``p @ v``) is transposed by a copy nest first."""
    node = c.g.nodes[nid]
    if not isinstance(node.op, F.MatmulOp):
        return False
    a, b = _need(c, node.inputs[0]), _need(c, node.inputs[1])
    if len(a.shape) < 2 or len(b.shape) < 2 or a.shape[-1] != b.shape[-2]:
        raise FusionError(f"matmul {nid!r}: operands {a.shape} @ {b.shape}")
    rb = len(b.shape)
    order_b = (*range(rb - 2), rb - 1, rb - 2)  # [..., N, K]
    bt = View(b.base, b.offset, tuple(b.shape[i] for i in order_b), tuple(b.strides[i] for i in order_b), b.dtype)
    if rb == 2:
        bt = _transposed_parameter(c, bt)  # a parameter stored [K, N] (GPT-2's Conv1D): transposed once, when the program is bound
    if rb == 2 and len(a.shape) > 2:
        bt = View(bt.base, bt.offset, (*(1,) * (len(a.shape) - 2), *bt.shape), (*(0,) * (len(a.shape) - 2), *bt.strides), bt.dtype)
    _emit_batched_contraction(c, nid, a, bt, "matmul")
    return True


def _plain_projection(c: _Ctx, nid: str) -> bool:
    """A bias-free linear over a constant weight whose result only feeds layout ops
    (so no other recognizer wants to absorb it) and is not a graph output."""
    g = c.g
    node = g.nodes[nid]
    if not isinstance(node.op, F.LinearOp) or nid in g.outputs or nid in c.done:
        return False
    if node.op.has_bias and not (isinstance(g.nodes[node.inputs[2]].op, ConstantOp) and len(g.nodes[node.inputs[2]].output.shape) == 1 and g.nodes[node.inputs[2]].op.value is None):
        return False  # (a bias that is a plain parameter vector can be stacked like the weights)
    if not isinstance(g.nodes[node.inputs[1]].op, ConstantOp) or len(g.nodes[node.inputs[1]].output.shape) != 2:
        return False
    cons = g.consumers(nid)
    return bool(cons) and all(isinstance(g.nodes[x].op, LAYOUT_OPS) for x in cons)


def _rec_linear_siblings(c: _Ctx, nid: str) -> bool:
    """Projections of one activation (q/k/v) as a single contraction over the
    stacked weights; each projection becomes a column window of the wide result."""
    g = c.g
    if not _plain_projection(c, nid):
        return False
    node = g.nodes[nid]
    x_id = node.inputs[0]
    w0 = g.nodes[node.inputs[1]].output
    group = [
        sid
        for sid in g.topological_order()
        if _plain_projection(c, sid)
        and g.nodes[sid].inputs[0] == x_id
        and g.nodes[sid].output.dtype == node.output.dtype
        and g.nodes[g.nodes[sid].inputs[1]].output.dtype == w0.dtype
        and g.nodes[g.nodes[sid].inputs[1]].output.shape[1] == w0.shape[1]
        and g.nodes[sid].output.shape[:-1] == node.output.shape[:-1]
        and g.nodes[sid].op.has_bias == node.op.has_bias  # all biased (Qwen-2's q / k / v) or none
    ]
    if len(group) < 2:
        return False
    weights = [g.nodes[sid].inputs[1] for sid in group]
    widths = [int(g.nodes[w].output.shape[0]) for w in weights]
    if any(n % 8 for n in widths):
        return False  # column windows must stay 16-byte aligned for the consumers' vector loads
    x, pro, extra, fold_w = _a_operand(c, x_id, set(group), fold=True)
    m, k, lda = _matrix(x, "linear input")
    if k != int(w0.shape[1]):
        raise FusionError("linear: inner dimensions differ")
    n_total = sum(widths)
    stacked = "__".join(weights) + (f"__k*{fold_w}" if fold_w else "")
    if stacked not in c.out.nodes:
        c.out.add_constant(stacked, (n_total, k), w0.dtype)
        c.out.nodes[stacked].hints["stacked"] = StackedConstant(tuple(weights), k_scale=fold_w)
    fid = "__".join(group)
    od = node.output.dtype
    bias_kw: dict = {}
    bias_in: list[str] = []
    if node.op.has_bias:
        biases = [g.nodes[sid].inputs[2] for sid in group]
        bdt = g.nodes[biases[0]].output.dtype
        if any(g.nodes[b].output.dtype != bdt or int(g.nodes[b].output.shape[0]) != n for b, n in zip(biases, widths)):
            return False
        for b in biases:
            _materialize(c, b)
        sb = "__".join(biases)
        if sb not in c.out.nodes:
            c.out.add_constant(sb, (n_total,), bdt)
            c.out.nodes[sb].hints["stacked"] = StackedConstant(tuple(biases))
        bias_kw = {"bias": sb, "bias_dtype": bdt, "epilogue": E.Var("acc") + E.Var("bias")}
        bias_in = [sb]
    body = Contraction(m=m, n=n_total, k=k, a=x.base, b=stacked, out=fid, in_dtype=x.dtype, out_dtype=od, lda=lda, a_offset=x.offset, a_prologue=pro, **bias_kw)
    c.out.add_node(TileOp(name=c.kname("rms_norm_linear" if pro else "linear"), body=body), list(dict.fromkeys([x.base, stacked, *extra, *bias_in])), Tensor(fid, (m, n_total), od), fid)
    col = 0
    for sid, n in zip(group, widths):
        shape = tuple(int(d) for d in g.nodes[sid].output.shape)
        lead = contiguous_strides(shape[:-1] + (1,))[:-1]
        c.done[sid] = fid
        c.windows[sid] = (col, shape, tuple(s * n_total for s in lead) + (1,))
        col += n
    return True


def _rec_linear_residual(c: _Ctx, nid: str) -> bool:
    node = c.g.nodes[nid]
    if not (_is(node, F.ElementwiseOp, fn="add") and len(node.inputs) == 2):
        return False
    for li, ri in ((0, 1), (1, 0)):
        lin_id, res_id = node.inputs[li], node.inputs[ri]
        # a reshape of the projection's rows between it and the add (``y.view(batch, seq, n) + residual``) changes nothing in memory
        while isinstance(c.g.nodes[lin_id].op, F.ViewOp) and c.single_use(lin_id) and lin_id not in c.done and c.g.nodes[lin_id].output.shape[-1] == c.g.nodes[c.g.nodes[lin_id].inputs[0]].output.shape[-1]:
            lin_id = c.g.nodes[lin_id].inputs[0]
        lin = c.g.nodes[lin_id]
        if not (isinstance(lin.op, F.LinearOp) and c.single_use(lin_id)) or lin_id in c.done:
            continue
        if c.g.nodes[res_id].output.shape != node.output.shape or c.g.nodes[res_id].output.dtype != node.output.dtype:
            continue
        res = _need(c, res_id)
        if not res.is_contiguous() or res.offset:
            continue
        x, w, m, n, k, lda, ldb, pro, extra = _linear_parts(c, lin_id)
        od = node.output.dtype
        body = Contraction(
            m=m, n=n, k=k, a=x.base, b=w.base, out=nid, in_dtype=x.dtype, out_dtype=od, lda=lda, ldb=ldb, a_offset=x.offset, b_offset=w.offset,
            post=E.Var("y") + E.Var("res"), epilogue_operands=(("res", od),), a_prologue=pro, **(bias := _bias_of(c, lin_id, n)),
        )  # fmt: skip
        body.operand_buffers = {"res": res.base}
        _emit(c, nid, body, "rms_norm_linear_add" if pro else "linear_add", [x.base, w.base, *extra, *([bias["bias"]] if bias else []), res.base])
        return True
    return False


def _rec_gate_up_f32(c: _Ctx, nid: str) -> bool:
    """``act(gate(x)) * up(x)`` on fp32 operands: the paired tile of ``_rec_gate_up`` is written for 16-bit operands, so
    the gate projection stays a contraction of its own and its activation and the product ride in the output stage of
    the up projection (two launches instead of two contractions and a map)."""
    node = c.g.nodes[nid]
    if not (_is(node, F.ElementwiseOp, fn="mul") and len(node.inputs) == 2) or node.output.dtype is not F32:
        return False
    for si, ui in ((0, 1), (1, 0)):
        act, up = c.g.nodes[node.inputs[si]], c.g.nodes[node.inputs[ui]]
        if not (isinstance(act.op, F.ElementwiseOp) and act.op.fn in ("silu", "gelu_tanh", "gelu") and len(act.inputs) == 1 and c.single_use(act.id) and act.id not in c.g.outputs):
            continue
        gate = c.g.nodes[act.inputs[0]]
        if not (isinstance(gate.op, F.LinearOp) and isinstance(up.op, F.LinearOp) and c.single_use(gate.id) and c.single_use(up.id)) or up.id in c.done or up.id in c.g.outputs or gate.id in c.g.outputs:
            continue
        if tuple(gate.output.shape) != tuple(node.output.shape) or tuple(up.output.shape) != tuple(node.output.shape) or gate.output.dtype is not F32 or up.output.dtype is not F32:
            continue
        g_view = _need(c, gate.id)
        if not g_view.is_contiguous() or g_view.offset:
            continue
        x, w, m, n, k, lda, ldb, pro, extra = _linear_parts(c, up.id)
        body = Contraction(
            m=m, n=n, k=k, a=x.base, b=w.base, out=nid, in_dtype=x.dtype, out_dtype=F32, lda=lda, ldb=ldb, a_offset=x.offset, b_offset=w.offset,
            post=E.Un(act.op.fn, E.Var("res")) * E.Var("y"), epilogue_operands=(("res", F32),), a_prologue=pro, **(bias := _bias_of(c, up.id, n)),
        )  # fmt: skip
        body.operand_buffers = {"res": g_view.base}
        _emit(c, nid, body, f"linear_{act.op.fn}_mul", [x.base, w.base, *extra, *([bias["bias"]] if bias else []), g_view.base])
        return True
    return False


def _rec_gate_up(c: _Ctx, nid: str) -> bool:
    node = c.g.nodes[nid]
    if not (_is(node, F.ElementwiseOp, fn="mul") and len(node.inputs) == 2) or node.output.dtype.nbytes != 2:
        return False  # (the paired tile is written for 16-bit operands: fp32 takes ``_rec_gate_up_f32``)
    for si, ui in ((0, 1), (1, 0)):
        silu = c.g.nodes[node.inputs[si]]
        up = c.g.nodes[node.inputs[ui]]
        if not (isinstance(silu.op, F.ElementwiseOp) and silu.op.fn in ("silu", "gelu_tanh", "gelu") and len(silu.inputs) == 1 and c.single_use(silu.id) and isinstance(up.op, F.LinearOp) and c.single_use(up.id)):
            continue  # (SwiGLU, or GeGLU in either GELU form: the activation is a name in the tile's epilogue)
        gate = c.g.nodes[silu.inputs[0]]
        if not (isinstance(gate.op, F.LinearOp) and c.single_use(gate.id)) or gate.op.has_bias or up.op.has_bias:
            continue
        if gate.inputs[0] != up.inputs[0]:
            continue
        wg, wu = c.g.nodes[gate.inputs[1]], c.g.nodes[up.inputs[1]]
        if not (isinstance(wg.op, ConstantOp) and isinstance(wu.op, ConstantOp)) or wg.output.shape != wu.output.shape:
            continue
        x, pro, extra, fold_w = _a_operand(c, gate.inputs[0], {gate.id, up.id}, fold=True)
        m, k, lda = _matrix(x, "gate/up input")
        n = int(wg.output.shape[0])
        stacked = f"{wg.id}__{wu.id}" + (f"__k*{fold_w}" if fold_w else "")
        if stacked not in c.out.nodes:
            c.out.add_constant(stacked, (2 * n, k), wg.output.dtype)
            c.out.nodes[stacked].hints["stacked"] = StackedConstant((wg.id, wu.id), k_scale=fold_w)
        od = node.output.dtype
        epi = _round(od, E.Un(silu.op.fn, _round(od, E.Var("acc")))) * _round(od, E.Var("acc2"))
        body = Contraction(m=m, n=n, k=k, a=x.base, b=stacked, out=nid, in_dtype=x.dtype, out_dtype=od, lda=lda, a_offset=x.offset, epilogue=epi, gate_pair=True, a_prologue=pro)
        _emit(c, nid, body, ("rms_norm_" if pro else "") + f"linear_{silu.op.fn}_mul", [x.base, stacked, *extra])
        return True
    return False


@dataclass
class _RmsMatch:
    x: str  # frontend node holding the row values (before any f32 cast)
    weight: str | None
    eps: float
    inner: DType  # dtype the normalised value is rounded to before the weight multiply
    cols: int


def _match_rms_chain(c: _Ctx, nid: str) -> _RmsMatch | None:
    """``w * cast(f32(x) * rsqrt(mean(f32(x)^2, -1, keepdim) + eps))`` as traced from HF-style RMSNorm."""
    g = c.g
    node = g.nodes[nid]
    weight = None
    cur = node
    if _is(cur, F.ElementwiseOp, fn="mul") and len(cur.inputs) == 2:
        a, b = (g.nodes[i] for i in cur.inputs)
        cand = [(a, b), (b, a)]
        for wnode, other in cand:
            if len(wnode.output.shape) == 1 and wnode.output.shape[0] == cur.output.shape[-1] and isinstance(g.nodes[_peel_layout(g, wnode.id)].op, (ConstantOp, InputOp)):
                weight, cur = wnode.id, other
                break
    inner = cur.output.dtype
    if isinstance(cur.op, F.CastOp):
        cur = g.nodes[cur.inputs[0]]
    if not (_is(cur, F.ElementwiseOp, fn="mul") and len(cur.inputs) == 2):
        return None
    a, b = (g.nodes[i] for i in cur.inputs)
    for xs, rs in ((a, b), (b, a)):
        if not _is(rs, F.ElementwiseOp, fn="rsqrt"):
            continue
        add = g.nodes[rs.inputs[0]]
        if not (_is(add, F.ElementwiseOp, fn="add") and add.op.scalar is not None):
            continue
        mean = g.nodes[add.inputs[0]]
        rank = len(g.nodes[mean.inputs[0]].output.shape) if mean.inputs else 0
        if not (isinstance(mean.op, F.MeanOp) and mean.op.keepdim and mean.op.axis == rank - 1):
            continue
        pw = g.nodes[mean.inputs[0]]
        if not (_is(pw, F.ElementwiseOp, fn="pow") and pw.op.scalar == 2.0):
            continue
        if pw.inputs[0] != xs.id:
            continue
        src = xs
        if isinstance(src.op, F.CastOp):
            src = g.nodes[src.inputs[0]]
        return _RmsMatch(x=src.id, weight=weight, eps=float(add.op.scalar), inner=inner, cols=int(node.output.shape[-1]))
    return None


def _rms_body(c: _Ctx, nid: str, m: _RmsMatch, out_dtype: DType):
    xv = _need(c, m.x)
    if xv.strides[-1] != 1:
        raise FusionError("rms_norm: the normalised axis must be contiguous")
    rows, x_addr = _row_addr(xv)
    x = E.Var("x")
    norm = x * E.Un("rsqrt", E.Var("ss") / float(m.cols) + m.eps)
    col_ops: tuple = ()
    inputs = [xv.base]
    if m.weight is not None:
        wv = _need(c, m.weight)
        if not wv.is_contiguous() or wv.offset:
            raise FusionError("rms_norm: weight must be a plain vector")
        project = E.Var("w") * _round(m.inner, norm)
        col_ops = (("w", wv.dtype),)
        inputs.append(wv.base)
    else:
        project = norm
    body = RowReduce(rows=rows, cols=m.cols, x=xv.base, x_dtype=xv.dtype, out=nid, out_dtype=out_dtype, stats=(Stat("ss", "sum", x * x),), project=project, col_operands=col_ops, x_addr=x_addr)
    body.operand_buffers = {"w": inputs[1]} if m.weight is not None else {}
    return body, inputs, xv


def _row_addr(v: View) -> tuple[int, RowAddr]:
    """Rows of ``v`` (all dims but the last) as a ``RowAddr``; one- or two-level."""
    lead = v.collapse_leading(1)
    if lead is not None:
        rows, stride = lead
        return rows, RowAddr.uniform(stride if rows > 1 else v.shape[-1], v.offset)
    dims = [(n, s) for n, s in zip(v.shape[:-1], v.strides[:-1]) if n != 1]
    # split into (outer run, inner run), each uniformly strided
    for cut in range(1, len(dims)):
        hi, lo = dims[:cut], dims[cut:]

        def run(ds):
            count, stride = ds[-1]
            for n, s in reversed(ds[:-1]):
                if s != stride * count:
                    return None
                count *= n
            return count, stride

        rh, rl = run(hi), run(lo)
        if rh and rl:
            return rh[0] * rl[0], RowAddr(offset=v.offset, div=rl[0], stride_hi=rh[1], stride_lo=rl[1])
    raise FusionError("row kernel: rows are not addressable with two strides")


def _rec_rms_chain(c: _Ctx, nid: str) -> bool:
    m = _match_rms_chain(c, nid)
    if m is None:
        return False
    node = c.g.nodes[nid]
    body, inputs, _ = _rms_body(c, nid, m, node.output.dtype)
    _emit(c, nid, body, "rms_norm_reduce", inputs)
    return True


def _rec_rms_op(c: _Ctx, nid: str) -> bool:
    node = c.g.nodes[nid]
    if not isinstance(node.op, F.RmsNormOp):
        return False
    m = _RmsMatch(x=node.inputs[0], weight=node.inputs[1] if node.op.has_weight else None, eps=node.op.eps, inner=F32, cols=int(node.output.shape[-1]))
    # nn.RMSNorm computes in the input dtype's fp32 upcast and rounds once at the end.
    body, inputs, _ = _rms_body(c, nid, m, node.output.dtype)
    if m.weight is not None:
        x = E.Var("x")
        body.project = x * E.Un("rsqrt", E.Var("ss") / float(m.cols) + m.eps) * E.Var("w")
    _emit(c, nid, body, "rms_norm_reduce", inputs)
    return True


def _rec_softmax(c: _Ctx, nid: str) -> bool:
    node = c.g.nodes[nid]
    if not isinstance(node.op, F.SoftmaxOp):
        return False
    xv, moved = _axis_last(c, nid, node.inputs[0], node.op.axis)
    rows, x_addr = _row_addr(xv)
    x = E.Var("x")
    stats = (Stat("m", "max", x), Stat("d", "sum", E.Un("exp", x - E.Var("m")), keep=True))
    body = RowReduce(rows=rows, cols=int(xv.shape[-1]), x=xv.base, x_dtype=xv.dtype, out=nid, out_dtype=node.output.dtype, stats=stats, project=x * E.Un("rcp", E.Var("d")), x_addr=x_addr)
    _emit(c, nid, body, "softmax_reduce", [xv.base], shape=tuple(xv.shape) if moved else None)
    if moved:
        # the result lies with the reduced axis last; readers address it in the traced order through these strides
        logical = tuple(int(d) for d in node.output.shape)
        dense = contiguous_strides(tuple(xv.shape))
        axis = node.op.axis
        strides = [0] * len(logical)
        others = [i for i in range(len(logical)) if i != axis]
        for pos, i in enumerate(others):
            strides[i] = dense[pos]
        strides[axis] = 1
        c.out.nodes[nid].hints["logical_view"] = (logical, tuple(strides))
    return True


def _axis_last(c: _Ctx, nid: str, src: str, axis: int) -> tuple[View, bool]:
    """``src`` addressed with ``axis`` as its last, contiguous axis: as it lies when that is the case already, else
    through a dense copy with the axis moved last.  Returns ``(view, moved)``."""
    xv = _need(c, src)
    rank = len(xv.shape)
    if axis == rank - 1 and (xv.strides[-1] == 1 or xv.shape[-1] == 1):
        return xv, False
    order = (*(i for i in range(rank) if i != axis), axis)
    if not all(isinstance(d, int) for d in (*xv.shape, *xv.strides, xv.offset)):
        raise FusionError("a reduction over a non-innermost axis needs static shapes")
    return _copy_of_view(c, xv, order, f"{nid}__axis_last"), axis != rank - 1


def _rec_row_sum(c: _Ctx, nid: str) -> bool:
    """``sum`` / ``mean`` over the innermost axis as a row reduction with one value per row."""
    node = c.g.nodes[nid]
    if not isinstance(node.op, (F.MeanOp, F.SumOp, F.AmaxOp)):
        return False
    # any other axis is moved last by a dense copy; what is left of the shape keeps its order, so the result needs no view
    xv, _ = _axis_last(c, nid, node.inputs[0], node.op.axis)
    rows, x_addr = _row_addr(xv)
    cols = int(xv.shape[-1])
    project = E.Var("s") / float(cols) if isinstance(node.op, F.MeanOp) else E.Var("s")
    monoid, label = ("max", "amax_reduce") if isinstance(node.op, F.AmaxOp) else ("sum", "mean_reduce" if isinstance(node.op, F.MeanOp) else "sum_reduce")
    body = RowReduce(rows=rows, cols=cols, x=xv.base, x_dtype=xv.dtype, out=nid, out_dtype=node.output.dtype, stats=(Stat("s", monoid, E.Var("x")),), project=project, x_addr=x_addr, scalar_out=True)
    _emit(c, nid, body, label, [xv.base])
    return True


def _dense(c: _Ctx, v: View, new_id: str) -> View:
    """``v`` itself when it enumerates its memory in row-major order, else a dense copy."""
    if v.strides == contiguous_strides(v.shape):
        return v
    return _copy_of_view(c, v, tuple(range(len(v.shape))), new_id)


def _rec_gather(c: _Ctx, nid: str) -> bool:
    """Embedding lookup / ``index_select``: one kernel that copies the picked slices."""
    from deplodock_amd.ir.tile import IndexRows

    node = c.g.nodes[nid]
    if not isinstance(node.op, F.GatherOp):
        return False
    xv = _dense(c, _need(c, node.inputs[0]), f"{nid}__table")
    iv = _dense(c, _need(c, node.inputs[1]), f"{nid}__index")
    axis = node.op.axis
    shape = tuple(int(d) for d in xv.shape)
    outer = math.prod(shape[:axis])
    inner = math.prod(shape[axis + 1 :])
    count = int(iv.numel)
    if xv.offset or iv.offset:
        raise FusionError(f"gather {nid!r}: operands must start at their buffers' first element")
    body = IndexRows(src=xv.base, idx=iv.base, out=nid, dtype=xv.dtype, idx_dtype=iv.dtype, outer=outer, n=shape[axis], inner=inner, count=count)
    _emit(c, nid, body, "index_rows", [xv.base, iv.base])
    return True


def _rec_cat(c: _Ctx, nid: str) -> bool:
    """``cat`` along one axis as a loop nest over the result: every point loads (index clamped into range) from each
    piece and keeps the one its position falls in — the reference lowers ``cat`` to the same index-mapped select
    (decomposition/150_cat.py)."""
    from deplodock_amd.ir import loopnest as L
    from deplodock_amd.ir.tile import LoopNest

    node = c.g.nodes[nid]
    if not isinstance(node.op, F.CatOp):
        return False
    out_shape = tuple(int(d) for d in node.output.shape)
    dim = node.op.dim
    # empty pieces (a key / value cache that holds nothing yet) contribute nothing
    pieces = [src for src in node.inputs if all(int(d) > 0 for d in c.g.nodes[src].output.shape)]
    if len(pieces) == 1:
        v = _need(c, pieces[0])
        c.done[nid] = v.base
        c.windows[nid] = (v.offset, tuple(v.shape), tuple(v.strides))
        return True
    axes = [L.Var(f"c{i}") for i in range(len(out_shape))]
    stmts: list = []
    branches: list = []
    operands: dict = {}
    inputs: list[str] = []
    lo = 0
    for k, src in enumerate(pieces):
        v = _need(c, src)
        if not all(isinstance(d, int) for d in (*v.shape, *v.strides, v.offset)):
            raise FusionError("cat: static shapes only")
        n = int(v.shape[dim])
        hi = lo + n
        inside = L.Bin("&&", L.Bin(">=", axes[dim], L.Lit(lo)), L.Bin("<", axes[dim], L.Lit(hi)))
        at: object = L.Lit(int(v.offset))
        for i, st in enumerate(v.strides):
            if not st:
                continue
            e = L.Ternary(inside, L.Bin("-", axes[dim], L.Lit(lo)), L.Lit(0)) if i == dim else axes[i]
            at = L.Bin("+", at, L.Bin("*", e, L.Lit(int(st))))
        operands[f"s{k}"] = (v.base, (int(c.out.nodes[v.base].output.numel),), v.dtype)
        inputs.append(v.base)
        stmts.append(L.Load(f"t{k}", f"s{k}", (at,)))
        branches.append((f"t{k}", L.Bin("<", axes[dim], L.Lit(hi)) if k < len(pieces) - 1 else L.Lit(1)))
        lo = hi
    if lo != out_shape[dim]:
        raise FusionError(f"cat {nid!r}: the pieces add up to {lo}, the result has {out_shape[dim]}")
    body: tuple = (*stmts, L.Select("u", tuple(branches)), L.Write(nid, tuple(axes), "u"))
    for i in reversed(range(len(out_shape))):
        body = (L.Loop(f"c{i}", out_shape[i], body),)
    nest = LoopNest(stmts=body, operands=operands, scalars={}, out=nid, out_name=nid, out_shape=out_shape, out_dtype=node.output.dtype)
    _emit(c, nid, nest, "cat", inputs)
    return True


def _rec_layer_norm(c: _Ctx, nid: str) -> bool:
    """LayerNorm over the last axis as one register-resident row kernel: the mean, then the centred sum of squares
    (a second statistic over the resident row, which is what keeps the variance free of cancellation), then the
    projection; computed in fp32 and rounded once, as ``nn.LayerNorm`` does."""
    node = c.g.nodes[nid]
    if not isinstance(node.op, F.LayerNormOp):
        return False
    xv = _need(c, node.inputs[0])
    if xv.strides[-1] != 1:
        xv = _copy_of_view(c, xv, tuple(range(len(xv.shape))), f"{nid}__rows")
    rows, x_addr = _row_addr(xv)
    cols = int(xv.shape[-1])
    x = E.Var("x")
    mean = E.Var("s1") / float(cols)
    stats = (Stat("s1", "sum", x), Stat("s2", "sum", (x - mean) * (x - mean)))
    project = (x - mean) * E.Un("rsqrt", E.Var("s2") / float(cols) + node.op.eps)
    col_ops, buffers, inputs = [], {}, [xv.base]
    for name, src, on in (("w", 1, node.op.has_weight), ("b", 2, node.op.has_bias)):
        if not on:
            continue
        pv = _need(c, node.inputs[src])
        if not pv.is_contiguous() or pv.offset or pv.numel != cols:
            raise FusionError(f"layer_norm: the {'weight' if name == 'w' else 'bias'} must be a plain vector of the normalised width")
        col_ops.append((name, pv.dtype))
        buffers[name] = pv.base
        inputs.append(pv.base)
        project = project * E.Var("w") if name == "w" else project + E.Var("b")
    body = RowReduce(rows=rows, cols=cols, x=xv.base, x_dtype=xv.dtype, out=nid, out_dtype=node.output.dtype, stats=stats, project=project, col_operands=tuple(col_ops), x_addr=x_addr)
    body.operand_buffers = buffers
    _emit(c, nid, body, "layer_norm_reduce", inputs)
    return True


def _match_rope(c: _Ctx, nid: str):
    """``t*cos + cat(neg(t[..., h:]), t[..., :h]) * sin`` → ``(t, cos, sin)`` node ids."""
    g = c.g
    node = g.nodes[nid]
    if not (_is(node, F.ElementwiseOp, fn="add") and len(node.inputs) == 2):
        return None
    for ai, bi in ((0, 1), (1, 0)):
        ma, mb = g.nodes[node.inputs[ai]], g.nodes[node.inputs[bi]]
        if not (_is(ma, F.ElementwiseOp, fn="mul") and _is(mb, F.ElementwiseOp, fn="mul") and len(ma.inputs) == 2 and len(mb.inputs) == 2):
            continue
        for ci, si in ((0, 1), (1, 0)):
            cat = g.nodes[mb.inputs[ci]]
            sin = mb.inputs[si]
            if not (isinstance(cat.op, F.CatOp) and len(cat.inputs) == 2 and cat.op.dim == len(cat.output.shape) - 1):
                continue
            neg, lo = g.nodes[cat.inputs[0]], g.nodes[cat.inputs[1]]
            if not (_is(neg, F.ElementwiseOp, fn="neg") and isinstance(lo.op, F.SliceOp)):
                continue
            hi = g.nodes[neg.inputs[0]]
            if not isinstance(hi.op, F.SliceOp):
                continue
            t = lo.inputs[0]
            d = int(g.nodes[t].output.shape[-1])
            last = len(g.nodes[t].output.shape) - 1
            if hi.inputs[0] != t or lo.op.dim != last or hi.op.dim != last:
                continue
            if (lo.op.start, lo.op.end, hi.op.start, hi.op.end) != (0, d // 2, d // 2, d):
                continue
            for ti, co in ((0, 1), (1, 0)):
                if ma.inputs[ti] == t:
                    return t, ma.inputs[co], sin
    return None


@dataclass
class _RopePlan:
    """What ``_rec_rope`` needs to know about one rotary-embedding expression."""

    t_id: str
    cos_id: str
    sin_id: str
    d: int
    od: DType
    t_view_shape: tuple[int, ...]
    order: list[int]  # dims of the rotated tensor (minus the last) in memory order
    mem_shape: tuple[int, ...]
    rows: int
    div: int  # cos/sin table row of memory row r is (r // div) % mod
    mod: int
    rms: _RmsMatch | None  # the norm feeding the rotation when it can be fused in
    pad: int = 0  # leading unit dims the traced result has more than the rotated tensor (``t_view_shape`` includes them, ``order`` does not)


def _plan_rope(c: _Ctx, nid: str) -> _RopePlan | None:
    hit = _match_rope(c, nid)
    if hit is None:
        return None
    t_id, cos_id, sin_id = hit
    g = c.g
    node = g.nodes[nid]
    d = int(node.output.shape[-1])
    src_id = _peel_layout(g, t_id)
    src = g.nodes[src_id]
    if isinstance(src.op, F.RmsNormOp):
        rms = _RmsMatch(x=src.inputs[0], weight=src.inputs[1] if src.op.has_weight else None, eps=src.op.eps, inner=F32, cols=int(src.output.shape[-1]))
    else:
        rms = _match_rms_chain(c, src_id)
    fuse_norm = rms is not None and rms.cols == d and all(cons in _rope_internal(g, t_id, nid) or isinstance(g.nodes[cons].op, LAYOUT_OPS) for cons in g.consumers(src_id))
    # Address rows of the *output* in the memory order of the rotated operand
    # (so the kernel is a row map whatever transposes the trace applied).
    tv = resolve_view(g, t_id)
    if tv.strides[-1] != 1:
        raise FusionError("rope: the rotated axis must be contiguous")
    order = sorted(range(len(tv.shape) - 1), key=lambda i: -tv.strides[i] if tv.shape[i] > 1 else 0)
    order = [i for i in order if tv.shape[i] > 1]
    mem_shape = tuple(tv.shape[i] for i in order)
    rows = 1
    for n in mem_shape:
        rows *= n
    # position axis = the axis of t that cos varies over; tables are [.., positions, d]
    cos_shape = tuple(int(v) for v in g.nodes[cos_id].output.shape)
    pos_axes = [i for i in range(len(cos_shape) - 1) if cos_shape[i] > 1]
    if len(pos_axes) > 1 or cos_shape[-1] != d:
        raise FusionError("rope: cos/sin must vary over one position axis")
    # The tables broadcast against the rotated tensor from the right, and the result takes the longer rank
    # (a trace may carry a table with more leading unit dims than the tensor it rotates).
    pad = max(0, len(node.output.shape) - len(tv.shape))
    if pos_axes:
        pa = pos_axes[0] - (len(cos_shape) - len(tv.shape))
        if pa not in order:
            raise FusionError("rope: unsupported cos/sin layout")
        k = order.index(pa)
        div = 1
        for n in mem_shape[k + 1 :]:
            div *= n
        mod = mem_shape[k]
    else:
        div, mod = 1, 1
    t_shape = (1,) * pad + tuple(int(v) for v in g.nodes[t_id].output.shape)
    return _RopePlan(t_id, cos_id, sin_id, d, node.output.dtype, t_shape, order, mem_shape, rows, div, mod, rms if fuse_norm else None, pad)


def _rope_tables(c: _Ctx, p: _RopePlan, div: int) -> tuple[tuple[RowOperand, RowOperand], View, View]:
    cos_v, sin_v = _need(c, p.cos_id), _need(c, p.sin_id)
    if not (cos_v.strides[-1] == 1 and sin_v.strides[-1] == 1):
        raise FusionError("rope: cos/sin must be contiguous along the rotated axis")
    if p.mod > 1:
        pa = [i for i in range(len(cos_v.shape) - 1) if cos_v.shape[i] > 1][0]
        if cos_v.strides[pa] != p.d or sin_v.strides[pa] != p.d:
            raise FusionError("rope: unsupported cos/sin layout")
    ops = (RowOperand("cos", cos_v.dtype, div=div, mod=p.mod, offset=cos_v.offset), RowOperand("sin", sin_v.dtype, div=div, mod=p.mod, offset=sin_v.offset))
    return ops, cos_v, sin_v


def _rope_expr(od: DType) -> E.Expr:
    return _round(od, _round(od, E.Var("y") * E.Var("cos")) + _round(od, E.Var("yr") * E.Var("sin")))


def _logical_strides(p: _RopePlan, mem_strides: tuple[int, ...]) -> tuple[int, ...]:
    """Strides of the traced (logical) shape over a buffer whose rows follow
    ``p.order``; ``mem_strides`` are the strides of those memory-order dims."""
    out = [0] * len(p.t_view_shape)
    for pos, i in enumerate(p.order):
        out[i + p.pad] = mem_strides[pos]
    out[-1] = 1
    return tuple(out)


#: tokens up to which the q / k head norm + rotary embedding stays a launch of its own behind the few-row projection
#: (the decoder block as one graph, two launches against the fused one: 24 tokens 25.3 / 26.0 us, 32 tokens 26.1 / 26.7;
#: 64 tokens 30.0 / 28.8)
_ROW_EPILOGUE_MIN_TOKENS = 32


def _rec_rope_pair(c: _Ctx, nid: str) -> bool:
    """Query and key head-norm + rotary embedding as one launch.  Applies when
    both read adjacent head ranges of one merged projection buffer
    (``[tokens, (q heads + k heads + ...) * d]``): the heads of both are walked
    as rows of one kernel, the two norm weights are stacked per head, and each
    result is a window of the ``[tokens, q heads + k heads, d]`` output."""
    g = c.g
    p = _plan_rope(c, nid)
    if p is None or p.rms is None or p.rms.weight is None:
        return False
    # one token: the token dim is a unit dim the plan drops; the heads alone are the rows
    single = len(p.mem_shape) == 1 and p.mod == 1
    if not single and (len(p.mem_shape) != 2 or p.mod != p.mem_shape[0]):
        return False
    partner = None
    for oid in g.topological_order():
        if oid == nid or oid in c.done or not _is(g.nodes[oid], F.ElementwiseOp, fn="add"):
            continue
        q = _plan_rope(c, oid)
        if q is None or q.rms is None or q.rms.weight is None:
            continue
        if (q.cos_id, q.sin_id, q.d, q.od, q.mod, q.order, q.rms.eps, q.rms.inner) == (p.cos_id, p.sin_id, p.d, p.od, p.mod, p.order, p.rms.eps, p.rms.inner) and len(q.mem_shape) == len(p.mem_shape):
            partner = (oid, q)
            break
    if partner is None:
        return False
    oid, q = partner
    xa, xb = _need(c, p.rms.x), _need(c, q.rms.x)
    if xa.base != xb.base or xa.dtype != xb.dtype:
        return False
    plans = [(nid, p, xa), (oid, q, xb)]
    plans.sort(key=lambda t: t[2].offset)
    (id0, p0, x0), (id1, p1, x1) = plans
    try:
        (rows0, a0), (rows1, a1) = _row_addr(x0), _row_addr(x1)
    except FusionError:
        return False
    h0, h1 = p0.mem_shape[-1], p1.mem_shape[-1]
    d = p.d
    if single:
        # [heads, d] windows of one row of the merged projection: rows d apart, the key heads right behind the query heads
        if not (a0.div == 1 and a1.div == 1 and rows0 == h0 and rows1 == h1 and (h0 == 1 or a0.stride_hi == d) and (h1 == 1 or a1.stride_hi == d) and a1.offset == a0.offset + h0 * d):
            return False
        prod = c.out.nodes.get(x0.base)
        pitch = (h0 + h1) * d
        if prod is not None and isinstance(prod.op, TileOp) and isinstance(prod.op.body, Contraction):
            pitch = prod.op.body.ldo or prod.op.body.n
        a0 = RowAddr(offset=a0.offset, div=h0 + h1, stride_hi=pitch, stride_lo=d)
    elif not (a0.div == h0 and a1.div == h1 and a0.stride_lo == d and a1.stride_lo == d and a0.stride_hi == a1.stride_hi and a1.offset == a0.offset + h0 * d and (h0 + h1) * d <= a0.stride_hi):
        return False
    # the two weights are only read through their stacked copy: they get no buffers of their own
    w0, w1 = g.nodes[p0.rms.weight], g.nodes[p1.rms.weight]
    if not (isinstance(w0.op, ConstantOp) and isinstance(w1.op, ConstantOp) and w0.output.dtype == w1.output.dtype and tuple(w0.output.shape) == tuple(w1.output.shape) == (d,)):
        return False
    heads = h0 + h1
    tokens = 1 if single else p0.mem_shape[0]
    stacked = f"{p0.rms.weight}__x{h0}__{p1.rms.weight}__x{h1}"
    if stacked not in c.out.nodes:
        c.out.add_constant(stacked, (heads * d,), w0.output.dtype)
        c.out.nodes[stacked].hints["stacked"] = StackedConstant((p0.rms.weight,) * h0 + (p1.rms.weight,) * h1)
    od = p.od
    x = E.Var("x")
    norm = x * E.Un("rsqrt", E.Var("ss") / float(d) + p.rms.eps)
    tables, cos_v, sin_v = _rope_tables(c, p, div=heads)
    fid = f"{id0}__{id1}"
    body = RowReduce(
        rows=tokens * heads, cols=d, x=x0.base, x_dtype=x0.dtype, out=fid, out_dtype=od, stats=(Stat("ss", "sum", x * x),),
        project=_round(od, E.Var("w") * _round(p.rms.inner, norm)), x_addr=RowAddr(offset=a0.offset, div=heads, stride_hi=a0.stride_hi, stride_lo=d),
        row_operands=(RowOperand("w", w0.output.dtype, div=1, mod=heads, offset=0), *tables),
    )  # fmt: skip
    body.rotate = RotateHalf(_rope_expr(od))
    body.operand_buffers = {"w": stacked, "cos": cos_v.base, "sin": sin_v.base}
    mem = (lambda hi: (d,)) if single else (lambda hi: (hi, d))  # strides of the plan's memory-order dims (heads [, tokens])
    raw_only_feeds_rope = all(_feeds_only(g, _peel_layout(g, rp.t_id), _rope_internal(g, rp.t_id, rid)) for rid, rp in ((id0, p0), (id1, p1)))
    # With a few tokens the projection is one pass over its weights in the few-row form, which has no output tile to
    # run a row kernel on: a second small launch costs less than giving that form up (us in the decoder block, fused
    # against few-row projection + this kernel: 16 tokens 7.3 against 3.0 + 1.9).
    if tokens > _ROW_EPILOGUE_MIN_TOKENS and raw_only_feeds_rope and _absorb_row_kernel(c, body, x0, a0, tokens, heads):
        # the projection that produced the heads rotates them on its way out: the results are windows of its buffer
        for rid, rp, first in ((id0, p0, 0), (id1, p1, h0)):
            c.done[rid] = x0.base
            c.windows[rid] = (a0.offset + first * d, rp.t_view_shape, _logical_strides(rp, mem(a0.stride_hi)))
        return True
    c.out.add_node(TileOp(name=c.kname("rms_norm_rope"), body=body), list(dict.fromkeys([x0.base, stacked, cos_v.base, sin_v.base])), Tensor(fid, (tokens, heads, d), od), fid)
    for rid, rp, first in ((id0, p0, 0), (id1, p1, h0)):
        c.done[rid] = fid
        c.windows[rid] = (first * d, rp.t_view_shape, _logical_strides(rp, mem(heads * d)))
    return True


def _feeds_only(g: Graph, src_id: str, allowed: set[str]) -> bool:
    """Does every path from ``src_id`` lead, through layout ops only, into ``allowed``?"""
    if src_id in g.outputs:
        return False
    for cons in g.consumers(src_id):
        if cons in allowed:
            continue
        if not isinstance(g.nodes[cons].op, LAYOUT_OPS) or not _feeds_only(g, cons, allowed):
            return False
    return True


def _absorb_row_kernel(c: _Ctx, body: RowReduce, x: View, addr: RowAddr, tokens: int, groups: int) -> bool:
    """Fold ``body`` (a row kernel over ``groups`` column groups per token, in place
    on the leading columns of ``x``'s buffer) into the contraction that writes that
    buffer.  Applies to a plain contraction whose result rows are the tokens."""
    prod = c.out.nodes.get(x.base)
    if prod is None or not isinstance(prod.op, TileOp) or not isinstance(prod.op.body, Contraction):
        return False
    con = prod.op.body
    d = body.cols
    if con.post is not None or con.gate_pair or con.row_epilogue is not None or con.reduce.cta != 1 or con.in_dtype.nbytes != 2:
        return False
    if not (con.out == x.base and con.m == tokens and addr.stride_hi == (con.ldo or con.n) and addr.offset == con.out_offset and groups * d <= con.n):
        return False
    if not (con.out_dtype == body.x_dtype == body.out_dtype and all(ro.dtype == con.out_dtype for ro in body.row_operands)):
        return False
    if d % 16 or d & (d - 1) or body.col_operands:
        return False
    con.row_epilogue = RowEpilogue(cols=d, col_end=groups * d, stats=body.stats, project=body.project, rotate=body.rotate, row_operands=body.row_operands, operand_buffers=dict(body.operand_buffers))
    for ro in body.row_operands:
        buf = body.operand_buffers.get(ro.name, ro.name)
        if buf not in prod.inputs:
            prod.inputs.append(buf)
    prod.op.name = prod.op.name.replace("linear", "linear_rope" if body.rotate is not None else "linear_rownorm", 1)
    return True


def _rec_rope(c: _Ctx, nid: str) -> bool:
    p = _plan_rope(c, nid)
    if p is None:
        return False
    g = c.g
    od, d = p.od, p.d
    row_ops, cos_v, sin_v = _rope_tables(c, p, div=p.div)
    # Output buffer: rows in t's memory order; the logical result is a view of it.
    out_mem_shape = (*p.mem_shape, d)
    if p.rms is not None:
        body, inputs, xv = _rms_body(c, nid, p.rms, od)
        if (body.rows, body.cols) != (p.rows, d):
            raise FusionError("rope: norm rows do not match the rotated tensor")
        body.project = _round(od, body.project)  # the norm's result is a tensor of the output dtype: keep its rounding point
    else:
        tv = resolve_view(g, p.t_id)
        xv = _need(c, p.t_id)
        # rows walk the rotated tensor in the planned order, addressed through the strides it really has
        # (a window of a merged projection buffer is wider-strided than the traced tensor)
        rows2, x_addr = _row_addr(View(xv.base, xv.offset, tuple(xv.shape[i] for i in p.order) + (d,), tuple(xv.strides[i] for i in p.order) + (1,), xv.dtype))
        body = RowReduce(rows=rows2, cols=d, x=xv.base, x_dtype=xv.dtype, out=nid, out_dtype=od, stats=(), project=E.Var("x"), x_addr=x_addr)
        body.operand_buffers = {}
        inputs = [xv.base]
    body.row_operands = row_ops
    body.rotate = RotateHalf(_rope_expr(od))
    body.operand_buffers.update({"cos": cos_v.base, "sin": sin_v.base})
    inputs += [cos_v.base, sin_v.base]
    _emit(c, nid, body, "rms_norm_rope" if p.rms is not None else "rope", inputs, shape=out_mem_shape)
    # Record how the logical (traced) shape maps onto the memory-order buffer.
    c.out.nodes[nid].hints["logical_view"] = (p.t_view_shape, _logical_strides(p, contiguous_strides(out_mem_shape)[:-1]))
    return True


def _rope_internal(g: Graph, t_id: str, add_id: str) -> set[str]:
    """Node ids that belong to the rope expression rooted at ``add_id`` (for single-use checks)."""
    seen: set[str] = set()
    stack = [add_id]
    while stack:
        n = stack.pop()
        if n in seen or n == t_id:
            continue
        seen.add(n)
        stack.extend(g.nodes[n].inputs)
    seen.add(t_id)
    return seen


def _undo_repeat_kv(g: Graph, nid: str) -> tuple[str, int]:
    """``(source, group)`` when ``nid`` is a KV tensor whose heads were repeated for grouped attention the
    materialising way — ``x[:, :, None].expand(B, Hkv, group, S, D).reshape(B, Hkv * group, S, D)`` — so that
    repeated head ``h`` reads source head ``h // group``: exactly what the kernel's grouped addressing does, with
    no copy.  ``(nid, 1)`` otherwise."""
    view, exp = g.nodes[nid], None
    if isinstance(view.op, F.ContiguousOp):
        view = g.nodes[view.inputs[0]]
    if isinstance(view.op, F.ViewOp):
        exp = g.nodes[view.inputs[0]]
    if exp is None or not isinstance(exp.op, F.ExpandOp) or not _is(g.nodes[exp.inputs[0]], F.UnsqueezeOp, dim=2):
        return nid, 1
    src = g.nodes[exp.inputs[0]].inputs[0]
    s_shape, e_shape, o_shape = (tuple(int(d) for d in g.nodes[n].output.shape) for n in (src, exp.id, view.id))
    if len(s_shape) != 4 or e_shape != (*s_shape[:2], e_shape[2], *s_shape[2:]) or o_shape != (s_shape[0], s_shape[1] * e_shape[2], *s_shape[2:]):
        return nid, 1
    return src, e_shape[2]


def _rec_sdpa(c: _Ctx, nid: str) -> bool:
    node = c.g.nodes[nid]
    if not isinstance(node.op, F.SdpaOp):
        return False
    (k_id, k_rep), (v_id, v_rep) = _undo_repeat_kv(c.g, node.inputs[1]), _undo_repeat_kv(c.g, node.inputs[2])
    if k_rep != v_rep:
        k_id, v_id, k_rep = node.inputs[1], node.inputs[2], 1
    q, k, v = (_need_logical(c, i) for i in (node.inputs[0], k_id, v_id))
    if min(len(q.shape), len(k.shape), len(v.shape)) < 3:
        raise FusionError("sdpa: expected [batch..., heads, seq, head_dim] operands")

    def batched(t: View) -> tuple[int, tuple[int, int, int]]:
        """``(batch count, (batch, head, seq) strides)`` of an operand whose dims before the last three are
        batch dims (the reference pads k / v with leading unit dims up to q's rank, frontend/ir.py:252-259)."""
        lead = [(n, st) for n, st in zip(t.shape[:-3], t.strides[:-3]) if n != 1]
        count, stride = 1, 0
        for n, st in reversed(lead):
            if count > 1 and st != stride * count:
                raise FusionError("sdpa: batch dims must collapse into one uniformly strided axis")
            stride = st if count == 1 else stride
            count *= n
        return count, (stride, t.strides[-3], t.strides[-2])

    (B, q_str), (Bk, k_str), (Bv, v_str) = batched(q), batched(k), batched(v)
    if Bk != B or Bv != B:
        raise FusionError("sdpa: q, k and v must agree on the batch size")
    Hq, Sq, D = q.shape[-3:]
    Hkv, Skv = k.shape[-3], k.shape[-2]
    if Hq != Hkv and not (node.op.enable_gqa or k_rep > 1):
        raise FusionError("sdpa: grouped heads need enable_gqa=True")
    for t in (q, k, v):
        if t.strides[-1] != 1:
            raise FusionError("sdpa: head_dim must be contiguous")
    # If the only consumer swaps heads and sequence (to [B, S, H, D], then flattens), write that layout directly.
    lead = len(node.output.shape) - 3
    logical = tuple(int(d_) for d_ in node.output.shape)
    out_id, o_shape, o_strides = nid, (B, Hq, Sq, D), (Hq * Sq * D, Sq * D, D)
    cons = c.g.consumers(nid)
    transposed = len(cons) == 1 and nid not in c.g.outputs and _is(c.g.nodes[cons[0]], F.TransposeOp, dim0=lead, dim1=lead + 1)
    if transposed:
        o_shape, o_strides = (B, Sq, Hq, D), (Sq * Hq * D, D, Hq * D)
    scale = node.op.scale if node.op.scale is not None else 1.0 / math.sqrt(D)
    mask_kw: dict = {}
    inputs = [q.base, k.base, v.base]
    if node.op.has_mask:
        mv = _need_logical(c, node.inputs[3])
        shp, st = (1,) * (4 - len(mv.shape)) + tuple(mv.shape), (0,) * (4 - len(mv.shape)) + tuple(mv.strides)
        if len(shp) != 4 or shp[-1] != Skv or shp[-2] not in (1, Sq) or shp[0] not in (1, B) or shp[1] not in (1, Hq) or (shp[-1] > 1 and st[-1] != 1):
            raise FusionError(f"sdpa: the mask must broadcast to [batch, heads, queries, keys] with contiguous keys, got {tuple(mv.shape)}")
        mask_kw = dict(mask=mv.base, mask_dtype=mv.dtype, mask_offset=mv.offset, mask_strides=tuple(0 if n == 1 else s_ for n, s_ in zip(shp[:3], st[:3])))
        inputs.append(mv.base)
    from deplodock_amd.passes.decompose_attention import flash_head_dim

    width = D if q.dtype == F32 else (flash_head_dim(D) or D)  # (the fp32 kernel pads its tiles itself)
    body = Flash(
        batch=B, q_heads=Hq, kv_heads=Hkv, q_len=Sq, kv_len=Skv, head_dim=width, head_dim_real=D if width != D else None,
        q=q.base, k=k.base, v=v.base, out=out_id, dtype=q.dtype,
        scale=float(scale), causal=node.op.is_causal, q_strides=q_str, k_strides=k_str, v_strides=v_str, o_strides=o_strides,
        q_offset=q.offset, k_offset=k.offset, v_offset=v.offset, **mask_kw,
    )  # fmt: skip
    _emit(c, nid, body, "sdpa_reduce", inputs, shape=o_shape)
    if transposed or len(logical) != 4:
        # how the traced shape (with its batch dims as traced) maps onto the buffer (not a comparison of the shapes:
        # they read the same when there are as many tokens as heads)
        lead_strides = contiguous_strides(logical[:lead] + (1,))[:-1]
        c.out.nodes[nid].hints["logical_view"] = (logical, (*(ls * o_strides[0] for ls in lead_strides), o_strides[1], o_strides[2], 1))
    return True


def _need_logical(c: _Ctx, nid: str) -> View:
    return _need(c, nid)


_POINTWISE_FN = {"add": "add", "sub": "sub", "mul": "mul", "div": "div", "maximum": "max", "minimum": "min"}
_POINTWISE_UN = {"neg": "neg", "rsqrt": "rsqrt", "sqrt": "sqrt", "exp": "exp", "silu": "silu", "sigmoid": "sigmoid", "tanh": "tanh", "abs": "abs", "reciprocal": "rcp",
                 "relu": "relu", "erf": "erf", "gelu": "gelu", "gelu_tanh": "gelu_tanh"}  # fmt: skip


def _pointwise_node_expr(op, args: list[E.Expr]) -> E.Expr | None:
    """The expression of one element-wise / cast / copy op over its argument expressions."""
    if isinstance(op, (F.CastOp, F.ContiguousOp)):
        return args[0]
    if not isinstance(op, F.ElementwiseOp):
        return None
    if op.fn in _POINTWISE_UN and len(args) == 1:
        return E.Un(_POINTWISE_UN[op.fn], args[0])
    if op.fn == "pow" and op.scalar == 2.0:
        return args[0] * args[0]
    if op.fn == "pow" and op.scalar is not None and not op.scalar_first and float(op.scalar) in (1.0, 3.0, 4.0):
        out = args[0]  # small whole powers as products (the reference's decomposition/030_pow.py does the same)
        for _ in range(int(op.scalar) - 1):
            out = out * args[0]
        return out
    if op.fn == "pow" and len(args) == 1 and op.scalar is not None:
        return E.Bin("pow", E.Const(op.scalar), args[0]) if op.scalar_first else E.Bin("pow", args[0], E.Const(op.scalar))
    if op.fn in _POINTWISE_FN:
        if op.scalar is not None:
            a, b = (E.Const(op.scalar), args[0]) if op.scalar_first else (args[0], E.Const(op.scalar))
        elif len(args) == 2:
            a, b = args
        else:
            return None
        return E.Bin(_POINTWISE_FN[op.fn], a, b)
    raise FusionError(f"element-wise op {op.fn!r} is not supported")


_MAX_FUSED_POINTWISE = 24  # ops folded into one map kernel


def _rec_row_fused(c: _Ctx, nid: str) -> bool:
    """An element-wise tree whose leaves include ``keepdim`` reductions over the last axis of element-wise functions
    of the *same* rows (a normalisation spelled out: Gemma's ``x * rsqrt(mean(x^2) + eps) * (1 + w)``, a hand-written
    layer norm, ``x - x.amax(-1, keepdim=True)``) as one register-resident row kernel: each reduction is a row
    statistic, the rest is the projection.  Casts are folded wherever they are read (recomputed, never stored);
    anything the row kernel has no operand form for leaves the match to the one-op-per-kernel fallbacks."""
    g = c.g
    node = g.nodes[nid]
    if not isinstance(node.op, (F.CastOp, F.ContiguousOp, F.ElementwiseOp)) or nid in c.done:
        return False
    shape = tuple(node.output.shape)
    if len(shape) < 1 or not all(isinstance(d, int) for d in shape) or shape[-1] < 2:
        return False
    stat_shape = (*shape[:-1], 1)
    cols = int(shape[-1])
    leaves: dict[str, E.Var] = {}
    stats: list[Stat] = []
    stat_of: dict[str, E.Expr] = {}
    folded = [0]

    class _Decline(Exception):
        pass

    def is_stat(cur: str) -> bool:
        n = g.nodes[cur]
        return isinstance(n.op, (F.MeanOp, F.SumOp, F.AmaxOp)) and cur not in c.done and n.op.keepdim and tuple(n.output.shape) == stat_shape and n.op.axis == len(shape) - 1 \
            and tuple(g.nodes[n.inputs[0]].output.shape) == shape and c.single_use(cur)  # fmt: skip

    def broadcast_of_stat(cur: str) -> bool:
        """``stat.expand_as(x)``: a per-row value spelled at the rows' full shape."""
        n = g.nodes[cur]
        return isinstance(n.op, F.ExpandOp) and cur not in c.done and tuple(n.output.shape) == shape and tuple(g.nodes[n.inputs[0]].output.shape) == stat_shape

    def foldable(cur: str, root: bool, strict: bool) -> bool:
        n = g.nodes[cur]
        if broadcast_of_stat(cur):
            return True
        if not isinstance(n.op, (F.CastOp, F.ContiguousOp, F.ElementwiseOp)) or cur in c.done or tuple(n.output.shape) not in (shape, stat_shape):
            return False
        if strict and sum(tuple(g.nodes[i].output.shape) == shape for i in n.inputs) > 1:
            return False  # under a statistic the row has one source: an op that joins two tensors (a residual add) is that source, stored by its own kernel
        return root or isinstance(n.op, (F.CastOp, F.ContiguousOp)) or c.single_use(cur)

    def build(cur: str, root: bool, strict: bool) -> E.Expr:
        n = g.nodes[cur]
        if cur in stat_of:
            return stat_of[cur]
        if cur in leaves:
            return leaves[cur]  # once a tensor is read from memory it is read from memory everywhere
        if is_stat(cur):
            pre = build(n.inputs[0], False, True)
            name = f"s{len(stats)}"
            stats.append(Stat(name, "max" if isinstance(n.op, F.AmaxOp) else "sum", pre))
            stat_of[cur] = _round(n.output.dtype, E.Var(name) / float(cols) if isinstance(n.op, F.MeanOp) else E.Var(name))
            return stat_of[cur]
        if not foldable(cur, root, strict) or folded[0] >= _MAX_FUSED_POINTWISE:
            leaves[cur] = E.Var(f"a{len(leaves)}")
            return leaves[cur]
        if broadcast_of_stat(cur):
            return build(n.inputs[0], False, strict)
        folded[0] += 1
        args = [build(i, False, strict) for i in n.inputs]
        e = _pointwise_node_expr(n.op, args)
        if e is None:
            raise _Decline
        return _round(n.output.dtype, e)

    def statistics_first(cur: str, root: bool, seen: set) -> None:
        """The reductions the tree reaches, innermost first: their operand decides what the resident row is."""
        if cur in seen:
            return
        seen.add(cur)
        if is_stat(cur):
            statistics_first(g.nodes[cur].inputs[0], False, seen)
            build(cur, False, True)
        elif foldable(cur, root, False):
            for i in g.nodes[cur].inputs:
                statistics_first(i, False, seen)

    try:
        statistics_first(nid, True, set())
        if not stats:
            return False
        project = build(nid, True, False)
    except (_Decline, FusionError):
        return False
    if not stats:
        return False
    # operands: the resident row (the one tensor the statistics read), further tensors of the rows' shape (a residual),
    # vectors along the row
    in_stats = set().union(*(E.variables(st.pre) for st in stats))
    x_leaf, col_ops, row_ops, buffers, inputs = None, [], [], {}, []
    rename: dict[str, E.Expr] = {}
    for leaf_id, var in leaves.items():
        t = g.nodes[leaf_id].output
        lshape = tuple(t.shape)
        if lshape == shape and var.name in in_stats:
            if x_leaf is not None:
                return False
            x_leaf = leaf_id
            rename[var.name] = E.Var("x")
        elif lshape == shape:
            v = _need(c, leaf_id)
            if v.strides != contiguous_strides(v.shape):
                return False
            name = f"r{len(row_ops)}"
            row_ops.append((name, v))
            rename[var.name] = E.Var(name)
        elif len(lshape) >= 1 and lshape[-1] == cols and all(d == 1 for d in lshape[:-1]):
            v = _need(c, leaf_id)
            if v.strides[-1] != 1 or v.offset:
                return False
            name = f"w{len(col_ops)}"
            col_ops.append((name, v.dtype))
            buffers[name] = v.base
            inputs.append(v.base)
            rename[var.name] = E.Var(name)
        elif isinstance(g.nodes[leaf_id].op, ConstantOp) and g.nodes[leaf_id].op.value is not None and t.numel == 1:
            rename[var.name] = E.Const(float(g.nodes[leaf_id].op.value))
        else:
            return False
    if x_leaf is None:
        return False
    xv = _need(c, x_leaf)
    if xv.strides[-1] != 1:
        return False
    try:
        rows, x_addr = _row_addr(xv)
    except FusionError:
        return False
    sub = lambda e: E.substitute(e, rename)  # noqa: E731
    for name, v in row_ops:
        buffers[name] = v.base
        inputs.append(v.base)
    body = RowReduce(rows=rows, cols=cols, x=xv.base, x_dtype=xv.dtype, out=nid, out_dtype=node.output.dtype,
                     stats=tuple(Stat(st.name, st.monoid, sub(st.pre)) for st in stats), project=sub(project), col_operands=tuple(col_ops),
                     row_operands=tuple(RowOperand(name, v.dtype, div=1, mod=rows, offset=int(v.offset)) for name, v in row_ops), x_addr=x_addr)  # fmt: skip
    body.operand_buffers = buffers
    _emit(c, nid, body, "row_fused_reduce", [xv.base, *inputs])
    return True


def _rec_pointwise(c: _Ctx, nid: str) -> bool:
    """Fallback: a tree of element-wise ops / casts as one flat map.  Producers
    that are element-wise themselves, have this one reader and the same shape
    are folded in with their own rounding point, so ``exp(neg(x)) * y`` is one
    kernel; other inputs become operands (same shape, a vector along the last
    axis, one value per row, or a scalar)."""
    g = c.g
    node = g.nodes[nid]
    if not isinstance(node.op, (F.CastOp, F.ContiguousOp, F.ElementwiseOp)):
        return False
    od = node.output.dtype
    shape = tuple(int(d) for d in node.output.shape)
    leaves: dict[str, E.Var] = {}  # frontend node id -> operand variable
    folded = [0]

    def build(cur: str, root: bool) -> E.Expr:
        n = g.nodes[cur]
        same_shape = tuple(int(d) for d in n.output.shape) == shape
        foldable = isinstance(n.op, (F.CastOp, F.ContiguousOp, F.ElementwiseOp)) and same_shape and cur not in c.done and (root or (c.single_use(cur) and folded[0] < _MAX_FUSED_POINTWISE))
        if not foldable:
            if cur not in leaves:
                leaves[cur] = E.Var(f"a{len(leaves)}")
            return leaves[cur]
        folded[0] += 1
        args = [build(i, False) for i in n.inputs]
        e = _pointwise_node_expr(n.op, args)
        if e is None:
            raise FusionError(f"no kernel recognizer for {type(n.op).__name__} at node {cur!r}")
        return _round(n.output.dtype, e)

    expr = build(nid, True)
    inner = shape[-1] if shape else 1
    operands, buffers, offsets = [], {}, {}
    for leaf_id, var in leaves.items():
        v = _need_logical(c, leaf_id)
        if any(st == 0 and n > 1 for n, st in zip(v.shape, v.strides)):  # an expanded operand is its unit-size source, broadcast
            v = View(v.base, v.offset, tuple(1 if st == 0 else n for n, st in zip(v.shape, v.strides)), v.strides, v.dtype)
        lead_ones = len(v.shape) >= 1 and all(d == 1 for d in v.shape[:-1])
        if v.shape == shape and v.is_contiguous():
            kind = "flat"
        elif v.numel == 1:
            kind = "scalar"
        elif lead_ones and v.shape[-1] == inner and v.strides[-1] == 1:
            kind = "col"
        elif len(v.shape) == len(shape) and v.shape[:-1] == shape[:-1] and v.shape[-1] == 1 and View(v.base, v.offset, v.shape[:-1], v.strides[:-1], v.dtype).is_contiguous():
            kind = "row"
        else:
            # general broadcasting (e.g. a [1, 1, S, S] mask into [B, H, S, S]), or a strided operand: the operand is
            # first written out densely in the result's shape by a copy nest (repeated axes read with stride 0)
            pad = len(shape) - len(v.shape)
            if pad < 0 or any(n not in (1, full) for n, full in zip(v.shape, shape[pad:])):
                raise FusionError(f"pointwise operand {leaf_id!r} of {nid!r} does not broadcast (shape {v.shape} into {shape})")
            wide = View(v.base, v.offset, shape, (0,) * pad + tuple(0 if n == 1 and full != 1 else st for n, st, full in zip(v.shape, v.strides, shape[pad:])), v.dtype)
            v = _copy_of_view(c, wide, tuple(range(len(shape))), f"{nid}__b{len(operands)}")
            kind = "flat"
        operands.append(MapOperand(var.name, v.dtype, kind))
        buffers[var.name] = v.base
        offsets[var.name] = v.offset
    numel = 1
    for d in shape:
        numel *= d
    body = Map(numel=numel, operands=tuple(operands), expr=expr, out=nid, out_dtype=od, inner=inner)
    body.operand_buffers = buffers
    body.operand_offsets = offsets
    label = "pointwise_" + (type(node.op).__name__.lower().removesuffix("op") if folded[0] == 1 else f"fused{folded[0]}")
    _emit(c, nid, body, label, list(buffers.values()))
    return True


# ---------------------------------------------------------------------------
# Driver
# ---------------------------------------------------------------------------


def fuse(g: Graph) -> Graph:
    """Lower a frontend ``Graph`` to ``Graph[TileOp + InputOp + ConstantOp]``."""
    from deplodock_amd.passes.decompose_attention import AttentionShapeError, decompose_attention
    from deplodock_amd.passes.raise_attention import raise_attention
    from deplodock_amd.passes.raise_loops import raise_loop_nests

    try:
        g = decompose_attention(g, _undo_repeat_kv)  # attention the flash kernel does not take (fp32, other head dims) becomes two loop nests
    except AttentionShapeError as exc:
        raise FusionError(str(exc)) from exc
    g = raise_loop_nests(g)  # Loop-IR kernels that are a contraction / a row normalisation become frontend ops first
    g = raise_attention(g)  # softmax(q @ k^T * scale [+ mask]) @ v spelled with matmuls becomes the fused op
    out = Graph()
    out.constant_values = dict(getattr(g, "constant_values", {}))
    c = _Ctx(g=g, out=out)
    # Inputs first, in their traced order, so positional binding stays stable.
    for nid in g.inputs:
        _materialize(c, nid)
    final_outputs = []
    for oid in g.outputs:
        v = _need_logical(c, oid)
        shape = tuple(int(d) for d in g.nodes[oid].output.shape)
        if not (v.offset == 0 and v.shape == shape and v.is_contiguous()) and not _same_memory(v, shape):
            v = _copy_of_view(c, v, tuple(range(len(v.shape))), f"{oid}__out")  # a strided view as a graph output: written out densely
        final_outputs.append(v.base)
        if v.base != oid:
            out.nodes[v.base].hints.setdefault("output_alias", []).append((oid, shape))
    out.outputs = final_outputs
    return out


def _same_memory(v: View, shape: tuple[int, ...]) -> bool:
    """True when ``v`` enumerates its buffer in plain row-major order (e.g. a reshape of a contiguous buffer)."""
    return v.offset == 0 and v.strides == contiguous_strides(v.shape)


__all__ = ["fuse", "FusionError", "StackedConstant", "BF16", "F16"]
