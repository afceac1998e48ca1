"""Attention spelled with matmuls is raised to ``SdpaOp`` before fusion.

A model that does not call the fused op computes ``softmax(q @ k.transpose(-1, -2) * scale [+ mask], -1) @ v``.  The
reference meets the same thing from the other side: it *decomposes* ``SdpaOp`` into exactly these ops
(emmy/compiler/pipeline/passes/frontend/decomposition/010_sdpa.py:28-138) and its tile lowering finds the streaming
form in the decomposed loops (passes/lowering/tile/_flash.py:96-110).  Here the frontend graph is matched instead:
the final ``MatmulOp`` node becomes an ``SdpaOp`` over ``(q, k, v[, mask])`` with the scale made explicit, and the
ordinary attention recogniser emits the flash kernel.

Matched only where the flash kernel applies (16-bit operands, head_dim 64 / 128 / 256, ``k`` transposed as a view
of a ``[..., S, D]`` tensor, every intermediate read once); anything else keeps its matmuls, which lower to batched
contractions and the softmax row kernel.
"""

from __future__ import annotations

from deplodock_amd.graph import Graph, Node
from deplodock_amd.ir import frontend as F


def _single_use(g: Graph, nid: str) -> bool:
    return len(g.consumers(nid)) == 1 and nid not in g.outputs


def _match(g: Graph, node: Node):
    """``(q, k, v, mask | None, scale)`` when ``node`` (a ``MatmulOp``) closes a matmul-spelled attention."""
    p_id, v_id = node.inputs
    p = g.nodes[p_id]
    rank = len(node.output.shape)
    if rank < 3 or not isinstance(p.op, F.SoftmaxOp) or p.op.axis != len(p.output.shape) - 1 or not _single_use(g, p_id):
        return None
    cur = g.nodes[p.inputs[0]]
    mask, scale = None, 1.0
    # softmax input: [+ mask] of [* scale | / scale] of q @ k^T, each read once
    if isinstance(cur.op, F.ElementwiseOp) and cur.op.fn == "add" and cur.op.scalar is None and len(cur.inputs) == 2 and _single_use(g, cur.id):
        sides = [i for i in cur.inputs if isinstance(g.nodes[_skip_scale(g, i)[0]].op, F.MatmulOp)]
        if len(sides) != 1:
            return None
        mask = next(i for i in cur.inputs if i != sides[0])
        cur = g.nodes[sides[0]]
    inner, scale = _skip_scale(g, cur.id)
    s = g.nodes[inner]
    if not isinstance(s.op, F.MatmulOp) or not _single_use(g, s.id) or (inner != cur.id and not _single_use(g, cur.id)):
        return None
    q_id, kt_id = s.inputs
    kt = g.nodes[kt_id]
    kr = len(kt.output.shape)
    if not (isinstance(kt.op, F.TransposeOp) and {kt.op.dim0 % kr, kt.op.dim1 % kr} == {kr - 1, kr - 2}):
        return None
    k_id = kt.inputs[0]
    q, k, v = g.nodes[q_id].output, g.nodes[k_id].output, g.nodes[v_id].output
    if not (len(q.shape) == len(k.shape) == len(v.shape) == rank) or q.dtype.name not in ("bf16", "f16") or not (q.dtype == k.dtype == v.dtype == node.output.dtype):
        return None
    d = int(q.shape[-1])
    from deplodock_amd.passes.decompose_attention import flash_head_dim

    if flash_head_dim(d) is None or int(k.shape[-1]) != d or int(v.shape[-1]) != d or tuple(k.shape[:-1]) != tuple(v.shape[:-1]) or tuple(q.shape[:-2]) != tuple(k.shape[:-2]):
        return None
    if mask is not None:
        m = g.nodes[mask].output
        if m.dtype.name not in ("bf16", "f16", "f32") or len(m.shape) > rank:
            return None
    return q_id, k_id, v_id, mask, scale


def _skip_scale(g: Graph, nid: str) -> tuple[str, float]:
    """``(producer, factor)`` when ``nid`` multiplies or divides its one tensor operand by a python scalar."""
    n = g.nodes[nid]
    if isinstance(n.op, F.ElementwiseOp) and n.op.scalar is not None and len(n.inputs) == 1:
        if n.op.fn == "mul":
            return n.inputs[0], float(n.op.scalar)
        if n.op.fn == "div" and not n.op.scalar_first and n.op.scalar != 0:
            return n.inputs[0], 1.0 / float(n.op.scalar)
    return nid, 1.0


def raise_attention(g: Graph) -> Graph:
    """``g`` with every matmul-spelled attention closed by an ``SdpaOp`` (a new graph when anything matched)."""
    hits = {}
    for nid, node in g.nodes.items():
        if isinstance(node.op, F.MatmulOp):
            m = _match(g, node)
            if m is not None:
                hits[nid] = m
    if not hits:
        return g
    out = Graph()
    for attr, value in vars(g).items():
        if attr != "nodes":
            setattr(out, attr, value)
    out.nodes = {}
    for nid, node in g.nodes.items():
        if nid in hits:
            q, k, v, mask, scale = hits[nid]
            op = F.SdpaOp(is_causal=False, scale=scale, enable_gqa=False, has_mask=mask is not None)
            out.nodes[nid] = Node(nid, op, [q, k, v] + ([mask] if mask is not None else []), node.output, dict(node.hints))
        else:
            out.nodes[nid] = node
    return out  # the bypassed score / softmax nodes stay in the graph unread: fusion only materialises what an output needs


__all__ = ["raise_attention"]
