"""Attention outside the streaming kernels' reach is decomposed into loop nests before fusion.

The flash kernels serve 16-bit operands whose rows are whole 16-byte chunks up to head_dim 256 and, on fp32 atoms, fp32
operands and other 16-bit rows of any head_dim up to 256; what is left is wider head dims, value rows of another length
than the keys', masks without a key axis and mixed operand types.  The reference compiles fp32 only and its
perf cases call ``F.scaled_dot_product_attention(q, k, v, is_causal=True, enable_gqa=...)`` on fp32 tensors
(tests/perf/cases.py:64-69, 174-190); it lowers the fused op by decomposing it into ``q k^T -> * scale -> [+ mask] ->
softmax -> @ v`` (emmy/compiler/pipeline/passes/frontend/decomposition/010_sdpa.py:53-138: grouped KV heads by
``head // group`` indexing, a causal mask as ``+ (-1e9)`` where ``key > query``), which its loop fusion turns into
two kernels: the masked scores, and softmax times ``v``.

Here an ``SdpaOp`` the flash kernel does not take is rewritten into those same two kernels, written as Loop-IR
statements (``LoopNestOp``): the loop-nest raiser then makes each a batched MFMA contraction with loop-nest operand
and output stages, exactly as it does for the reference's own two attention kernels of its on-disk corpus.
"""

from __future__ import annotations

import math

from deplodock_amd.graph import Graph, Node, Tensor
from deplodock_amd.ir import frontend as F
from deplodock_amd.ir import loopnest as L

FLASH_HEAD_DIMS = (64, 128, 256)


def flash_head_dim(d: int) -> int | None:
    """The width the flash kernel runs a 16-bit head_dim ``d`` at: ``d`` itself or the next of its widths up (rows of whole
    16-byte chunks are padded with columns that count as zeros); ``None`` when it takes neither."""
    if d % 8 or d < 8:
        return None
    return next((w for w in FLASH_HEAD_DIMS if w >= d), None)


def f32_head_dim(d) -> bool:
    """Whether the fp32 streaming kernel takes rows of ``d`` values (``emit/flash_f32.py``: up to 256, any alignment)."""
    from deplodock_amd.emit.flash_f32 import f32_supported

    return isinstance(d, int) and f32_supported(d)


#: largest scores tensor ``[batch..., heads, queries, keys]`` the decomposed route writes to device memory
SCORES_LIMIT_BYTES = 8 * 2**30


class AttentionShapeError(ValueError):
    pass


def _static(shape) -> tuple[int, ...]:
    if not all(isinstance(d, int) for d in shape):
        raise AttentionShapeError("attention outside the streaming kernels (16-bit rows that are not whole 16-byte chunks, head dims beyond 256) needs static shapes")
    return tuple(int(d) for d in shape)


def _wrap(axes: list[tuple[str, int]], body: tuple) -> tuple:
    for name, extent in reversed(axes):
        body = (L.Loop(name, extent, tuple(body)),)
    return tuple(body)


def _aligned_index(shape: tuple[int, ...], lead_vars: list[L.Var], lead_shape: tuple[int, ...], tail: tuple, what: str) -> tuple:
    """Index of an operand whose dims before its last ``len(tail)`` line up, from the right, with q's leading dims
    (each equal to q's, or 1 and then read at 0)."""
    nlead = len(shape) - len(tail)
    if nlead > len(lead_vars):
        raise AttentionShapeError(f"sdpa: {what} has more leading dims than q")
    idx = []
    for d, var, full in zip(shape[:nlead], lead_vars[len(lead_vars) - nlead :], lead_shape[len(lead_shape) - nlead :]):
        if d == full:
            idx.append(var if full > 1 else L.Lit(0))
        elif d == 1:
            idx.append(L.Lit(0))
        else:
            raise AttentionShapeError(f"sdpa: {what} dim {d} does not match q's {full}")
    return (*idx, *tail)


def _decompose(g: Graph, node: Node, undo_repeat) -> list[Node]:
    op: F.SdpaOp = node.op
    nid = node.id
    q_id, k_id, v_id = node.inputs[:3]
    (k_src, k_rep), (v_src, v_rep) = undo_repeat(g, k_id), undo_repeat(g, v_id)
    if k_rep == v_rep and k_rep > 1:
        k_id, v_id = k_src, v_src  # the materialised repeat is the ``head // group`` indexing below
    q, k, v = (_static(g.nodes[i].output.shape) for i in (q_id, k_id, v_id))
    if min(len(q), len(k), len(v)) < 3:
        raise AttentionShapeError("sdpa: expected [batch..., heads, seq, head_dim] operands")
    hq, sq, d = q[-3:]
    hkv, skv = k[-3], k[-2]
    dv = v[-1]
    if k[-1] != d or v[-3] != hkv or v[-2] != skv:
        raise AttentionShapeError(f"sdpa: operands {q} / {k} / {v} do not fit together")
    if hq != hkv and not (op.enable_gqa or k_rep > 1):
        raise AttentionShapeError("sdpa: grouped heads need enable_gqa=True")
    if hq % hkv:
        raise AttentionShapeError("sdpa: q heads must be a multiple of kv heads")
    group = hq // hkv
    lead = q[:-3]
    dtype = node.output.dtype
    scale = float(op.scale) if op.scale is not None else 1.0 / math.sqrt(d)

    lead_vars = [L.Var(f"b{i}") for i in range(len(lead))]
    lead_axes = [(var.name, n) for var, n in zip(lead_vars, lead) if n > 1]  # unit dims are read at 0, with no loop
    lead_idx = tuple(var if n > 1 else L.Lit(0) for var, n in zip(lead_vars, lead))
    h, i, j, dd = L.Var("h"), L.Var("i"), L.Var("j"), L.Var("d")
    kv_head = L.Bin("/", h, L.Lit(group)) if group > 1 else h

    # kernel 1: scores[..., h, i, j] = sum_d q[..., h, i, d] * k[..., h / group, j, d] * scale (+ mask)
    scores_id = f"{nid}__scores"
    scores_shape = (*lead, hq, sq, skv)
    # This route materialises the scores (the flash kernel, which streams them, takes 16-bit operands only): bounded, so
    # that a long fp32 sequence is refused with a message instead of asking the allocator for the memory.
    scores_bytes = math.prod(scores_shape) * dtype.nbytes
    if scores_bytes > SCORES_LIMIT_BYTES:
        raise AttentionShapeError(
            f"sdpa: the decomposed route (16-bit rows that are not whole 16-byte chunks, head dims beyond 256) would materialise {scores_bytes / 2**30:.1f} GiB of scores "
            f"{scores_shape}; the limit is {SCORES_LIMIT_BYTES / 2**30:.0f} GiB — pad the head_dim to whole 16-byte chunks (streamed by the flash kernel) or run shorter sequences"
        )
    head = [L.Load("c_scale", "scale", (L.Lit(0),))]
    scalars = {"scale": scale}
    loads, inputs = ["q", "k"], [q_id, k_id]
    post = [L.Assign("scaled", "multiply", ("acc", "c_scale"))]
    value = "scaled"
    if op.has_mask:
        m_id = node.inputs[3]
        m = _static(g.nodes[m_id].output.shape)
        if len(m) < 2 or m[-1] not in (1, skv) or m[-2] not in (1, sq):
            raise AttentionShapeError(f"sdpa: the mask {m} must broadcast to [..., queries, keys]")
        tail = (i if m[-2] > 1 else L.Lit(0), j if m[-1] > 1 else L.Lit(0))
        m_idx = _aligned_index(m, [*lead_vars, h], (*lead, hq), tail, "the mask")
        post = [L.Load("bias", "mask", m_idx), *post, L.Assign("masked", "add", ("scaled", "bias"))]
        loads.append("mask")
        inputs.append(m_id)
        value = "masked"
    elif op.is_causal:
        head += [L.Load("c_zero", "mask_zero", (L.Lit(0),)), L.Load("c_fill", "mask_fill", (L.Lit(0),))]
        scalars.update(mask_zero=0.0, mask_fill=-1e9)
        post = [L.Select("bias", (("c_zero", L.Bin("<=", j, i)), ("c_fill", L.Bin(">", j, i)))), *post, L.Assign("masked", "add", ("scaled", "bias"))]
        value = "masked"
    k_loop = L.Loop("d", d, (
        L.Load("qv", "q", (*lead_idx, h, i, dd)),
        L.Load("kv", "k", _aligned_index(k, lead_vars, lead, (kv_head, j, dd), "k")),
        L.Assign("prod", "multiply", ("qv", "kv")),
        L.Accum("acc", "prod", "add"),
    ))  # fmt: skip
    body1 = _wrap([*lead_axes, ("h", hq), ("i", sq), ("j", skv)], (k_loop, *post, L.Write(scores_id, (*lead_idx, h, i, j), value)))
    n1 = Node(scores_id, F.LoopNestOp(stmts=(*head, *body1), loads=tuple(loads), scalars=scalars, out_name=scores_id, label="sdpa_scores"),
              inputs, Tensor(scores_id, scores_shape, dtype))  # fmt: skip

    # kernel 2: out[..., h, i, e] = sum_j exp(s[j] - max_j s) / sum_j exp(s[j] - max_j s) * v[..., h / group, j, e]
    s_idx = (*lead_idx, h, i, j)
    e = L.Var("e")
    fold_max = L.Loop("j", skv, (L.Load("s0", "scores", s_idx), L.Accum("row_max", "s0", "maximum")))
    fold_sum = L.Loop("j", skv, (L.Load("s1", "scores", s_idx), L.Assign("c1", "subtract", ("s1", "row_max")), L.Assign("e1", "exp", ("c1",)), L.Accum("row_sum", "e1", "add")))
    pv = L.Loop("j", skv, (
        L.Load("s2", "scores", s_idx),
        L.Assign("c2", "subtract", ("s2", "row_max")),
        L.Assign("e2", "exp", ("c2",)),
        L.Load("vv", "v", _aligned_index(v, lead_vars, lead, (kv_head, j, e), "v")),
        L.Assign("p", "divide", ("e2", "row_sum")),
        L.Assign("pv", "multiply", ("p", "vv")),
        L.Accum("o", "pv", "add"),
    ))  # fmt: skip
    body2 = _wrap([*lead_axes, ("h", hq), ("i", sq)], (fold_max, fold_sum, L.Loop("e", dv, (pv, L.Write(nid, (*lead_idx, h, i, e), "o")))))
    n2 = Node(nid, F.LoopNestOp(stmts=body2, loads=("scores", "v"), scalars={}, out_name=nid, label="sdpa_softmax_v"), [scores_id, v_id], node.output)
    return [n1, n2]


def decompose_attention(g: Graph, undo_repeat, streamed=None) -> Graph:
    """``g`` with every ``SdpaOp`` no streaming kernel takes (16-bit rows that are not whole 16-byte chunks, head dims
    beyond 256, value rows of another length than the keys') replaced by the two loop nests of the decomposed form; a new
    graph when anything changed.  ``undo_repeat(g, node id) -> (source id, group)`` sees through a materialised head
    repeat; ``streamed(node) -> bool`` replaces the rule for which ops stay fused."""

    from deplodock_amd import config

    pinned_apart = config.knob_raw("FLASH") == "decompose"  # ``EMMY_FLASH=decompose``: the reference's two-kernel route everywhere

    def flash_takes(node: Node) -> bool:
        if pinned_apart:
            return False
        q, k, v = (g.nodes[i].output for i in node.inputs[:3])
        if q.dtype.name in ("bf16", "f16") and flash_head_dim(int(q.shape[-1])) is not None:
            return True
        # the kernel on fp32 atoms: fp32 operands, or 16-bit rows that are not whole 16-byte chunks — any row length it
        # has registers for, q / k / v rows alike
        if q.dtype.name not in ("f32", "bf16", "f16") or not (k.dtype.name == v.dtype.name == q.dtype.name):
            return False
        if not (f32_head_dim(q.shape[-1]) and k.shape[-1] == v.shape[-1] == q.shape[-1]):
            return False
        if node.op.has_mask:  # the kernel reads a mask with the keys along its last axis; a column mask is left to the decomposed form
            m = g.nodes[node.inputs[3]].output
            if len(m.shape) > 4 or len(m.shape) < 1 or m.shape[-1] != k.shape[-2]:
                return False
        return True

    hits = [nid for nid, n in g.nodes.items() if isinstance(n.op, F.SdpaOp) and not (streamed or flash_takes)(n)]
    if not hits:
        return g
    out = Graph()
    for attr, value in vars(g).items():
        if attr != "nodes":
            setattr(out, attr, value)
    out.nodes = {}
    for nid, node in g.nodes.items():
        if nid not in hits:
            out.nodes[nid] = node
            continue
        for n in _decompose(g, node, undo_repeat):
            if n.id in out.nodes or (n.id in g.nodes and n.id != nid):
                raise ValueError(f"decomposed node id {n.id!r} is taken")
            out.nodes[n.id] = n
    return out


__all__ = ["decompose_attention", "AttentionShapeError"]
