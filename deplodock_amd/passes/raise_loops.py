"""Loop-IR kernels that are a tiled kernel in disguise are raised back to frontend ops.

A kernel of the reference's corpus is a fused loop nest (post-fusion, pre-tiling: the stage its own tile planner
starts from, emmy/compiler/pipeline/passes/lowering/tile/).  Two shapes of nest have a tiled kernel here, and
rendering them loop for loop would leave the matrix cores idle:

* **a contraction with an element-wise output stage** — ``for m: for n: {pre; for k: acc += a[m,k] * b[n,k]; post;
  write}`` — becomes ``LinearOp`` (``x @ W.T``, emmy/compiler/ir/frontend/ir.py:212-217; the reference decomposes
  it into exactly this multiply + sum nest, decomposition/_helpers.py:87-110) followed by the ``ElementwiseOp``
  nodes of its ``pre`` / ``post`` statements; the fusion pass then folds a residual add into the contraction's
  output stage as it does for a traced module;
* **a row RMS normalisation** — ``for r: {for c: acc += x*x; s = rsqrt(acc / count + eps); for c: write x*s*w}`` —
  becomes ``RmsNormOp`` (frontend/ir.py:309-312; decomposition/080_rms_norm.py:25-57 + 090_mean.py:27-44).

An operand of such a contraction that is read through a permuted or folded index (the o-projection reads the attention
output ``[H, S, D]`` as ``[S, H*D]``) is first copied to a plain matrix by a small loop nest of its own.

* **the general form** (``_try_batched_contraction``) — a batch of outer loops, operands that are *computed* in the
  reduction loop (a rotary embedding folded into the reads of q and k; softmax probabilities from two folds that
  precede the loop), any output stage — becomes operand nests + one ``BatchedLinearOp`` + an output-stage nest.

Anything else stays a ``LoopNestOp`` and goes to the loop-nest emitter.  ``EMMY_NEST=loops``
keeps every nest there (A/B, and the emitter's own tests).
"""

from __future__ import annotations

from deplodock_amd import config
from deplodock_amd.graph import Graph, Node, Tensor
from deplodock_amd.ir import frontend as F
from deplodock_amd.ir import loopnest as L

_UNARY = {"negative": "neg", "reciprocal": "reciprocal", "rsqrt": "rsqrt", "sqrt": "sqrt", "exp": "exp", "tanh": "tanh", "sigmoid": "sigmoid", "silu": "silu", "abs": "abs"}
_BINARY = {"add": "add", "subtract": "sub", "multiply": "mul", "divide": "div", "maximum": "maximum", "minimum": "minimum"}


class _NoMatch(Exception):
    pass


def _simple_index(index: tuple, shape: tuple[int, ...], extents: dict[str, int]) -> list[str]:
    """The loop axes a ``Load`` / ``Write`` index walks, in order, when every entry is a bare axis over its whole
    dimension or a literal 0 on a dimension of extent 1."""
    if len(index) != len(shape):
        raise _NoMatch
    axes = []
    for e, dim in zip(index, shape):
        if isinstance(e, L.Lit) and e.value == 0 and dim == 1:
            continue
        if isinstance(e, L.Var) and extents.get(e.name) == dim and e.name not in axes:
            axes.append(e.name)
            continue
        raise _NoMatch
    return axes


class _Builder:
    """New frontend nodes standing in for one ``LoopNestOp`` node."""

    def __init__(self, g: Graph, node: Node):
        self.g, self.node, self.new = g, node, []
        self.dtype = node.output.dtype
        self.n = 0

    def add(self, op, inputs: list[str], shape: tuple[int, ...], final: bool = False) -> str:
        nid = self.node.id if final else f"{self.node.id}__r{self.n}"
        self.n += 1
        self.new.append(Node(nid, op, list(inputs), Tensor(nid, tuple(shape), self.dtype)))
        return nid

    def shape_of(self, nid: str) -> tuple[int, ...]:
        for n in self.new:
            if n.id == nid:
                return tuple(n.output.shape)
        return tuple(int(d) for d in self.g.nodes[nid].output.shape)

    def view(self, nid: str, shape: tuple[int, ...], final: bool = False) -> str:
        if self.shape_of(nid) == tuple(shape) and not final:
            return nid
        return self.add(F.ViewOp(shape=tuple(shape)), [nid], shape, final)

    def gather(self, load: L.Load, rows: L.Loop, cols: L.Loop) -> str:
        """A plain row-major ``[rows, cols]`` copy of what ``load`` reads (its index any expression over the two
        axes): a small loop nest of its own, so the contraction sees an ordinary matrix."""
        nid = f"{self.node.id}__r{self.n}"
        src = _source(self.node, load)
        stmts = (L.Loop(rows.axis, rows.extent, (L.Loop(cols.axis, cols.extent, (L.Load("t", load.input, load.index), L.Write(nid, (L.Var(rows.axis), L.Var(cols.axis)), "t"))),)),)
        return self.add(F.LoopNestOp(stmts=stmts, loads=(load.input,), scalars={}, out_name=nid, label="gather"), [src], (rows.extent, cols.extent))

    def finish(self, res: str, out_shape: tuple[int, ...]) -> None:
        """Make the new node ``res`` the stand-in for the raised node: under its id, in its recorded shape."""
        if self.shape_of(res) != tuple(out_shape):
            self.view(res, out_shape, final=True)
            return
        for n in self.new:
            n.inputs = [self.node.id if i == res else i for i in n.inputs]
            if n.id == res:
                n.id = n.output.name = self.node.id
        self.new.sort(key=lambda n: n.id == self.node.id)  # the stand-in last (stable: producers keep their order)


def _source(node: Node, load: L.Load) -> str:
    """The graph tensor a ``Load`` reads."""
    try:
        return node.inputs[node.op.loads.index(load.input)]
    except ValueError as exc:
        raise _NoMatch from exc


def _elementwise(b: _Builder, stmts: list, env: dict, mn: tuple[str, str], extents: dict[str, int], full: tuple[int, ...], loops=None) -> None:
    """Bind the value of every statement of an output stage in ``env``: a tensor node (broadcastable against
    ``full``, the contraction's result shape) or a python float."""
    node = b.node
    m_ax, n_ax = mn
    for s in stmts:
        if isinstance(s, L.Load):
            if s.input in (node.op.scalars or {}):
                env[s.name] = float(node.op.scalars[s.input])
                continue
            src = _source(node, s)
            try:
                axes = _simple_index(s.index, b.shape_of(src), extents)
            except _NoMatch:
                if set().union(*(L.expr_vars(e) for e in s.index)) != {m_ax, n_ax} or loops is None:
                    raise
                env[s.name] = b.view(b.gather(s, *loops), full)
                continue
            if axes == [m_ax, n_ax]:
                env[s.name] = b.view(src, full)
            elif axes == [n_ax]:
                env[s.name] = b.view(src, (extents[n_ax],))
            elif axes == [m_ax]:
                env[s.name] = b.view(src, full[:-1] + (1,))
            elif axes == [] and b.shape_of(src) and all(d == 1 for d in b.shape_of(src)):
                env[s.name] = b.view(src, (1,))
            else:
                raise _NoMatch
        elif isinstance(s, L.Assign):
            args = [env[a] for a in s.args if a in env]
            if len(args) != len(s.args):
                raise _NoMatch
            tensors = [a for a in args if isinstance(a, str)]
            if not tensors:
                raise _NoMatch  # constant folding of scalars is not worth a case
            if s.op in _UNARY:
                env[s.name] = b.add(F.ElementwiseOp(fn=_UNARY[s.op]), tensors, _bshape(b, tensors, full))
            elif s.op in _BINARY:
                if len(tensors) == 2:
                    env[s.name] = b.add(F.ElementwiseOp(fn=_BINARY[s.op]), tensors, _bshape(b, tensors, full))
                else:
                    scalar = next(a for a in args if not isinstance(a, str))
                    env[s.name] = b.add(F.ElementwiseOp(fn=_BINARY[s.op], scalar=scalar, scalar_first=not isinstance(args[0], str)), tensors, _bshape(b, tensors, full))
            else:
                raise _NoMatch
        else:
            raise _NoMatch


def _bshape(b: _Builder, tensors: list[str], full: tuple[int, ...]) -> tuple[int, ...]:
    """Broadcast shape of ``tensors`` (each ``full``, a trailing vector, a column or a single value)."""
    import numpy as np

    return tuple(int(d) for d in np.broadcast_shapes(*(b.shape_of(t) for t in tensors)))


def _try_contraction(g: Graph, node: Node) -> list[Node] | None:
    op: F.LoopNestOp = node.op
    stmts = list(op.stmts)
    head = [s for s in stmts if not isinstance(s, L.Loop)]
    loops = [s for s in stmts if isinstance(s, L.Loop)]
    try:
        if len(loops) != 1 or stmts[-1] is not loops[0] or not all(isinstance(s, L.Load) for s in head):
            raise _NoMatch
        lm = loops[0]
        if len(lm.body) != 1 or not isinstance(lm.body[0], L.Loop):
            raise _NoMatch
        ln = lm.body[0]
        inner = [s for s in ln.body if isinstance(s, L.Loop)]
        if len(inner) != 1 or not isinstance(ln.body[-1], L.Write):
            raise _NoMatch
        lk = inner[0]
        at = ln.body.index(lk)
        pre, post, write = list(ln.body[:at]), list(ln.body[at + 1 : -1]), ln.body[-1]
        extents = {lm.axis: lm.extent, ln.axis: ln.extent, lk.axis: lk.extent}
        if len(extents) != 3:
            raise _NoMatch
        # the fold: acc += a * b over k, nothing else in the loop
        kb = list(lk.body)
        if len(kb) != 4 or not (isinstance(kb[-1], L.Accum) and kb[-1].op == "add" and isinstance(kb[-2], L.Assign) and kb[-2].op == "multiply" and kb[-1].value == kb[-2].name):
            raise _NoMatch
        loads = {s.name: s for s in kb[:2] if isinstance(s, L.Load)}
        if len(loads) != 2 or set(kb[-2].args) != set(loads):
            raise _NoMatch
        b = _Builder(g, node)
        x = w = None
        for ld in loads.values():
            if ld.input in (op.scalars or {}):
                raise _NoMatch
            src = _source(node, ld)
            if g.nodes[src].output.dtype != b.dtype:
                raise _NoMatch
            try:
                axes = _simple_index(ld.index, b.shape_of(src), extents)
            except _NoMatch:
                axes = None
            used = set().union(*(L.expr_vars(e) for e in ld.index))
            if axes == [lm.axis, lk.axis]:
                x = src
            elif axes == [ln.axis, lk.axis]:
                w = src
            elif used == {lm.axis, lk.axis} and x is None:
                x = b.gather(ld, lm, lk)  # read through a permuted / folded index: made a plain matrix first
            elif used == {ln.axis, lk.axis} and w is None:
                w = b.gather(ld, ln, lk)
            else:
                raise _NoMatch
        if x is None or w is None:
            raise _NoMatch
        if b.shape_of(w) != (ln.extent, lk.extent):
            w = b.view(w, (ln.extent, lk.extent))  # unit dimensions around [N, K]
        full = tuple(b.shape_of(x)[:-1]) + (ln.extent,)  # x is [1.., M, K] (checked above): the product is [1.., M, N]
        out_shape = tuple(int(d) for d in node.output.shape)
        if _simple_index(write.index, out_shape, extents) != [lm.axis, ln.axis]:
            raise _NoMatch
        env: dict = {}
        _elementwise(b, head, env, (lm.axis, ln.axis), extents, full, (lm, ln))
        _elementwise(b, pre, env, (lm.axis, ln.axis), extents, full, (lm, ln))
        env[kb[-1].name] = b.add(F.LinearOp(has_bias=False), [x, w], full)
        _elementwise(b, post, env, (lm.axis, ln.axis), extents, full, (lm, ln))
        res = env.get(write.value)
        if not isinstance(res, str) or b.shape_of(res) != full or not any(n.id == res for n in b.new):
            raise _NoMatch
        b.finish(res, out_shape)
        return b.new
    except (_NoMatch, KeyError, IndexError):
        return None


def _uses(stmt) -> tuple[str, ...]:
    if isinstance(stmt, L.Assign):
        return stmt.args
    if isinstance(stmt, (L.Accum, L.Write)):
        return (stmt.value,)
    if isinstance(stmt, L.Select):
        return tuple(v for v, _ in stmt.branches)
    return ()


def _index_vars(stmt) -> set[str]:
    exprs = stmt.index if isinstance(stmt, (L.Load, L.Write)) else tuple(p for _, p in stmt.branches) if isinstance(stmt, L.Select) else ()
    return set().union(*(L.expr_vars(e) for e in exprs)) if exprs else set()


def _defined(body) -> set[str]:
    """Names a statement list binds in its own scope (a loop contributes what it folds)."""
    out: set[str] = set()
    for s in body:
        if isinstance(s, L.Loop):
            out |= {t.name for t in s.body if isinstance(t, L.Accum)}
        elif not isinstance(s, L.Write):
            out.add(s.name)
    return out


def _all_uses(body) -> set[str]:
    out: set[str] = set()
    for s in L.walk(body):
        out |= set(_uses(s))
    return out


def _nest_node(b: _Builder, stmts: tuple, shape: tuple[int, ...], label: str, extra: dict[str, str] | None = None) -> str:
    """A ``LoopNestOp`` node over ``stmts`` (whose ``Write`` names the new node); its operands are the tensors of the
    raised node that the statements load, plus ``extra`` (load name -> new node id)."""
    node = b.node
    nid = f"{node.id}__r{b.n}"
    stmts = _retarget(stmts, nid)
    names = list(dict.fromkeys(s.input for s in L.walk(stmts) if isinstance(s, L.Load)))
    scalars = {k: v for k, v in (node.op.scalars or {}).items() if k in names}
    loads, inputs = [], []
    for name in names:
        if name in scalars:
            continue
        if extra and name in extra:
            loads.append(name)
            inputs.append(extra[name])
        elif name in node.op.loads:
            loads.append(name)
            inputs.append(node.inputs[node.op.loads.index(name)])
        else:
            raise _NoMatch
    return b.add(F.LoopNestOp(stmts=stmts, loads=tuple(loads), scalars=scalars, out_name=nid, label=label), inputs, shape)


def _retarget(stmts: tuple, out: str) -> tuple:
    """``stmts`` with every ``Write`` pointed at ``out``."""
    res = []
    for s in stmts:
        if isinstance(s, L.Loop):
            res.append(L.Loop(s.axis, s.extent, _retarget(s.body, out)))
        elif isinstance(s, L.Write):
            res.append(L.Write(out, s.index, s.value))
        else:
            res.append(s)
    return tuple(res)


def _wrap(loops: list[L.Loop], body: tuple) -> tuple:
    for lp in reversed(loops):
        body = (L.Loop(lp.axis, lp.extent, tuple(body)),)
    return tuple(body)


def _try_batched_contraction(g: Graph, node: Node) -> list[Node] | None:
    """The general form: outer loops that only wrap (a batch), then ``for m: {prefix; for n: {pre; for k: {...;
    acc += u * v}; post; write}}`` where ``u`` is computed from values that do not vary with ``n`` and ``v`` from
    values that do not vary with ``m``.  ``u`` and ``v`` are written out as ``[P, M, K]`` and ``[P | 1, N, K]`` by loop
    nests of their own (with ``prefix`` — e.g. the two folds of a softmax — in the first), the products are one
    batched contraction, and ``pre`` / ``post`` run in a third nest over its result."""
    op: F.LoopNestOp = node.op
    try:
        stmts = list(op.stmts)
        head = [s for s in stmts if not isinstance(s, L.Loop)]
        if not stmts or not isinstance(stmts[-1], L.Loop) or len(head) != len(stmts) - 1 or not all(isinstance(s, L.Load) and not s.index or isinstance(s, L.Load) and not _index_vars(s) for s in head):
            raise _NoMatch
        batch: list[L.Loop] = []
        cur = stmts[-1]
        while len(cur.body) == 1 and isinstance(cur.body[0], L.Loop):
            batch.append(cur)
            cur = cur.body[0]
        if cur.body and isinstance(cur.body[-1], L.Write) and batch:
            lm, prefix, ln = batch.pop(), [], cur  # ``for m: for n: {...; write}``: nothing between the two loops
        else:
            lm = cur
            if not lm.body or not isinstance(lm.body[-1], L.Loop) or any(isinstance(s, L.Write) for s in lm.body[:-1]):
                raise _NoMatch
            prefix, ln = list(lm.body[:-1]), lm.body[-1]
        inner = [s for s in ln.body if isinstance(s, L.Loop)]
        if len(inner) != 1 or not isinstance(ln.body[-1], L.Write) or any(isinstance(s, L.Write) for s in ln.body[:-1]):
            raise _NoMatch
        lk = inner[0]
        at = ln.body.index(lk)
        pre, post, write = list(ln.body[:at]), list(ln.body[at + 1 : -1]), ln.body[-1]
        kb = list(lk.body)
        if len(kb) < 3 or any(isinstance(s, (L.Loop, L.Write)) for s in kb) or sum(isinstance(s, L.Accum) for s in kb) != 1:
            raise _NoMatch
        acc, prod = kb[-1], kb[-2]
        if not (isinstance(acc, L.Accum) and acc.op == "add" and isinstance(prod, L.Assign) and prod.op == "multiply" and acc.value == prod.name):
            raise _NoMatch
        axes = [lp.axis for lp in batch] + [lm.axis, ln.axis, lk.axis]
        if len(set(axes)) != len(axes):
            raise _NoMatch
        bvars = {lp.axis for lp in batch}
        # what every value of the k loop varies with
        deps: dict[str, set[str]] = {s.name: set() for s in head}
        for name in _defined(prefix):
            deps[name] = bvars | {lm.axis}
        for name in _defined(pre):
            deps[name] = bvars | {lm.axis, ln.axis}
        body_k = kb[:-2]
        for s in body_k:
            d = _index_vars(s)
            for u in _uses(s):
                if u not in deps:
                    raise _NoMatch
                d |= deps[u]
            deps[s.name] = d
        u_name, v_name = prod.args
        if ln.axis in deps[u_name] or lm.axis in deps[v_name]:
            u_name, v_name = v_name, u_name
        if ln.axis in deps[u_name] or lm.axis in deps[v_name]:
            raise _NoMatch

        def side(target: str) -> list:
            need, keep = {target}, []
            for s in reversed(body_k):
                if s.name in need:
                    keep.append(s)
                    need |= set(_uses(s))
            return list(reversed(keep))

        a_stmts, b_stmts = side(u_name), side(v_name)
        if any(ln.axis in deps[s.name] for s in a_stmts) or any(lm.axis in deps[s.name] for s in b_stmts):
            raise _NoMatch
        b = _Builder(g, node)
        pshape = tuple(lp.extent for lp in batch)
        p = 1
        for d in pshape:
            p *= d
        bidx = tuple(L.Var(lp.axis) for lp in batch)
        extents = {lp.axis: lp.extent for lp in (*batch, lm, ln, lk)}

        def in_place(side_stmts: list, axes: list[str]) -> str | None:
            """The graph tensor itself when the side is one plain load walking ``axes`` in order: no copy needed."""
            if len(side_stmts) != 1 or not isinstance(side_stmts[0], L.Load) or side_stmts[0].input in (op.scalars or {}):
                return None
            try:
                src = _source(node, side_stmts[0])
                return src if _simple_index(side_stmts[0].index, b.shape_of(src), extents) == axes else None
            except _NoMatch:
                return None

        baxes = [lp.axis for lp in batch]
        a_id = in_place(a_stmts, [*baxes, lm.axis, lk.axis]) if not prefix else None
        if a_id is None:
            a_head = [s for s in head if s.name in _all_uses(a_stmts) | _all_uses(prefix)]
            a_body = _wrap(batch + [lm], (*prefix, L.Loop(lk.axis, lk.extent, (*a_stmts, L.Write("", (*bidx, L.Var(lm.axis), L.Var(lk.axis)), u_name)))))
            a_id = _nest_node(b, (*a_head, *a_body), (*pshape, lm.extent, lk.extent), "operand_a")
        b_batched = any(deps[s.name] & bvars for s in b_stmts)
        b_id = in_place(b_stmts, [*(baxes if b_batched else []), ln.axis, lk.axis])
        if b_id is None:
            b_loops = (batch if b_batched else []) + [ln]
            b_head = [s for s in head if s.name in _all_uses(b_stmts)]
            b_body = _wrap(b_loops, (L.Loop(lk.axis, lk.extent, (*b_stmts, L.Write("", (*(bidx if b_batched else ()), L.Var(ln.axis), L.Var(lk.axis)), v_name))),))
            b_id = _nest_node(b, (*b_head, *b_body), (*(pshape if b_batched else ()), ln.extent, lk.extent), "operand_b")
        x3 = b.view(a_id, (p, lm.extent, lk.extent))
        w3 = b.view(b_id, (p if b_batched else 1, ln.extent, lk.extent))
        t3 = b.add(F.BatchedLinearOp(), [x3, w3], (p, lm.extent, ln.extent))
        t = b.view(t3, (*pshape, lm.extent, ln.extent))
        # the output stage: pre / post over the products, as a nest of its own
        out_shape = tuple(int(d) for d in node.output.shape)
        stage = [*pre, *post]
        if not stage and write.value == acc.name:
            try:
                if _simple_index(write.index, out_shape, {**{lp.axis: lp.extent for lp in batch}, lm.axis: lm.extent, ln.axis: ln.extent}) == [*(lp.axis for lp in batch), lm.axis, ln.axis]:
                    b.finish(t3, out_shape)
                    return b.new
            except _NoMatch:
                pass
        used = _all_uses(stage) | {write.value}
        e_prefix = prefix if used & _defined(prefix) else []
        e_head = [s for s in head if s.name in used | _all_uses(e_prefix)]
        load_t = L.Load(acc.name, t, (*bidx, L.Var(lm.axis), L.Var(ln.axis)))
        e_body = _wrap(batch + [lm], (*e_prefix, L.Loop(ln.axis, ln.extent, (*pre, load_t, *post, write))))
        res = _nest_node(b, (*e_head, *e_body), out_shape, "output_stage", extra={t: t})
        b.finish(res, out_shape)
        return b.new
    except (_NoMatch, KeyError, IndexError, ValueError):
        return None


def _try_rms_norm(g: Graph, node: Node) -> list[Node] | None:
    op: F.LoopNestOp = node.op
    scalars = op.scalars or {}
    try:
        stmts = list(op.stmts)
        head = {s.name: scalars[s.input] for s in stmts[:-1] if isinstance(s, L.Load) and s.input in scalars}
        if len(head) != len(stmts) - 1 or not isinstance(stmts[-1], L.Loop):
            raise _NoMatch
        lr = stmts[-1]
        body = list(lr.body)
        if len(body) != 5 or not (isinstance(body[0], L.Loop) and isinstance(body[4], L.Loop) and all(isinstance(s, L.Assign) for s in body[1:4])):
            raise _NoMatch
        l1, (mean, plus, rs), l2 = body[0], body[1:4], body[4]
        if l1.extent != l2.extent:
            raise _NoMatch
        # sum of squares
        b1 = list(l1.body)
        if len(b1) == 3:  # the row element loaded once and multiplied by itself
            b1 = [b1[0], b1[0], *b1[1:]]
        if len(b1) != 4 or not (isinstance(b1[0], L.Load) and isinstance(b1[1], L.Load) and isinstance(b1[2], L.Assign) and isinstance(b1[3], L.Accum)):
            raise _NoMatch
        if b1[0].input != b1[1].input or b1[0].index != b1[1].index or b1[2].op != "multiply" or len(b1[2].args) != 2 or set(b1[2].args) != {b1[0].name, b1[1].name} or b1[3].op != "add" or b1[3].value != b1[2].name:
            raise _NoMatch
        b = _Builder(g, node)
        x = _source(node, b1[0])
        ext1 = {lr.axis: lr.extent, l1.axis: l1.extent}
        if _simple_index(b1[0].index, b.shape_of(x), ext1) != [lr.axis, l1.axis]:
            raise _NoMatch
        # mean, + eps, rsqrt
        if not (mean.op == "divide" and mean.args[0] == b1[3].name and head.get(mean.args[1]) == float(l1.extent)):
            raise _NoMatch
        eps_name = [a for a in plus.args if a != mean.name]
        if not (plus.op == "add" and mean.name in plus.args and len(eps_name) == 1 and eps_name[0] in head and rs.op == "rsqrt" and rs.args == (plus.name,)):
            raise _NoMatch
        # x * s * w
        b2 = list(l2.body)
        if len(b2) != 5 or not isinstance(b2[-1], L.Write):
            raise _NoMatch
        lds = {s.name: s for s in b2 if isinstance(s, L.Load)}
        muls = [s for s in b2 if isinstance(s, L.Assign)]
        if len(lds) != 2 or len(muls) != 2 or any(m.op != "multiply" for m in muls):
            raise _NoMatch
        ext2 = {lr.axis: lr.extent, l2.axis: l2.extent}
        first, second = muls
        if set(first.args) - {rs.name} == set() or rs.name not in first.args:
            raise _NoMatch
        (xn_name,) = set(first.args) - {rs.name}
        (w_name,) = set(second.args) - {first.name}
        if first.name not in second.args or xn_name not in lds or w_name not in lds or b2[-1].value != second.name:
            raise _NoMatch
        if _source(node, lds[xn_name]) != x or _simple_index(lds[xn_name].index, b.shape_of(x), ext2) != [lr.axis, l2.axis]:
            raise _NoMatch
        w = _source(node, lds[w_name])
        if _simple_index(lds[w_name].index, b.shape_of(w), ext2) != [l2.axis] or b.shape_of(w) != (l2.extent,):
            raise _NoMatch
        out_shape = tuple(int(d) for d in node.output.shape)
        if _simple_index(b2[-1].index, out_shape, ext2) != [lr.axis, l2.axis] or b.shape_of(x) != out_shape:
            raise _NoMatch
        if g.nodes[x].output.dtype != b.dtype or g.nodes[w].output.dtype != b.dtype:
            raise _NoMatch
        b.add(F.RmsNormOp(eps=float(head[eps_name[0]]), has_weight=True), [x, w], out_shape, final=True)
        return b.new
    except (_NoMatch, KeyError, ValueError, IndexError):
        return None


def raise_loop_nests(g: Graph) -> Graph:
    """``g`` with every ``LoopNestOp`` that has a tiled form replaced by frontend nodes (a new graph; ``g`` is left
    as it was)."""
    if not any(isinstance(n.op, F.LoopNestOp) for n in g.nodes.values()) or (config.knob_raw("NEST") or "").strip().lower().split("/")[0] == "loops":
        return g
    out = Graph()
    for attr, value in vars(g).items():
        if attr != "nodes":
            setattr(out, attr, value)
    out.nodes = {}
    for nid, node in g.nodes.items():
        new = None
        if isinstance(node.op, F.LoopNestOp):
            new = _try_contraction(g, node) or _try_rms_norm(g, node) or _try_batched_contraction(g, node)
        if new is None:
            out.nodes[nid] = node
        else:
            for n in new:
                if n.id in out.nodes or (n.id in g.nodes and n.id != nid):
                    raise ValueError(f"raised node id {n.id!r} is taken")
                out.nodes[n.id] = n
    return out


__all__ = ["raise_loop_nests"]
