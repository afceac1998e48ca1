"""Reading the reference's frontend-graph JSON (``Graph.to_dict`` / ``Graph.from_dict``).

The reference serialises every IR stage as ``{"inputs": [...], "outputs": [...], "nodes": {id: {"op":
<class name>, "op_fields": {...}, "inputs": [...], "output": {"name", "shape", "dtype"}}}}``
(emmy/compiler/graph.py:875-960) and keeps traced decoder blocks in that form as fixtures
(tests/compiler/fixtures/tinyllama_layer0.json, qwen25_7b_layer0.json).  This module reads the
*frontend* stage of that format — the ops a trace produces: ``InputOp``, ``ConstantOp``, ``ElementwiseOp``,
``LinearOp``, ``SdpaOp``, ``MeanOp``, ``SumOp``, ``RmsNormOp``, ``SoftmaxOp`` and the layout ops
``ReshapeOp`` / ``TransposeOp`` / ``SliceOp`` / ``CatOp`` / ``UnsqueezeOp`` (emmy/compiler/ir/frontend/ir.py,
emmy/compiler/ir/tensor/ir.py) — into this backend's traced-graph form, so a graph the reference wrote
drives this backend.  Of the later stages the *Loop IR* is read too: a ``LoopOp`` node (a post-fusion, pre-tiling
kernel, the form of the reference's on-disk kernel corpus ``kernels/*.json`` and
``experiments/kernel_dataset/*/*.json``) keeps its statements (``ir/loopnest.py``: parsed, never evaluated) and
lowers to a tiled kernel where it is a contraction or a row normalisation in disguise, else to the loop-nest
emitter.  Tile IR and Kernel IR hold the reference's own lowering for another machine and are refused.

Conventions of the format that are resolved here:

* python scalars of an ATen call are shape-``[1]`` ``ConstantOp`` nodes with a ``value``; where they are
  operands of an element-wise op they become its ``scalar``, where they are arguments of a layout op
  (slice dim / start / end, cat dim, the two dims of a transpose) they are folded into the op;
* ``SliceOp`` in the legacy convention has inputs ``[tensor, dim, start, end]`` (frontend/ir.py:100-136),
  ``CatOp`` ends with its dim constant (:138-166), a two-element ``TransposeOp.axes`` is a swap (:33-61);
* ``MeanOp`` / ``SumOp`` keep the reduced axis when the recorded output shape has it;
* dtypes are spelled ``float32`` / ``f32`` / ``bfloat16`` / ``bf16`` / ``float16`` / ``f16``.
"""

from __future__ import annotations

import json
from pathlib import Path

from deplodock_amd.dtype import BF16, F16, F32, I32, I64, DType
from deplodock_amd.graph import Graph, Node, Tensor
from deplodock_amd.ir import frontend as F
from deplodock_amd.ir.base import ConstantOp, InputOp


class IngestError(ValueError):
    """The JSON is not a frontend-stage graph of the reference, or uses an op this backend does not trace."""


_DTYPES: dict[str, DType] = {"float32": F32, "f32": F32, "bfloat16": BF16, "bf16": BF16, "float16": F16, "f16": F16, "int32": I32, "i32": I32, "int64": I64, "i64": I64}
_ELEMENTWISE = {
    "add": "add", "subtract": "sub", "sub": "sub", "multiply": "mul", "mul": "mul", "divide": "div", "div": "div", "pow": "pow", "maximum": "maximum", "minimum": "minimum",
    "negative": "neg", "neg": "neg", "rsqrt": "rsqrt", "sqrt": "sqrt", "exp": "exp", "silu": "silu", "sigmoid": "sigmoid", "tanh": "tanh", "abs": "abs", "reciprocal": "reciprocal",
}  # fmt: skip
_LATER_STAGES = {"TileOp", "KernelOp", "CudaOp", "ReduceOp", "IndexMapOp"}
_INT_MAX = 2**62


def _dtype(name: str, cast: DType | None = None) -> DType:
    try:
        dt = _DTYPES[name]
    except KeyError as exc:
        raise IngestError(f"unknown dtype {name!r}") from exc
    return cast if cast is not None and dt in (F32, BF16, F16) else dt


def graph_from_reference_dict(data: dict, cast: DType | None = None) -> Graph:
    """The traced-graph form of a reference frontend graph.  Weights (``ConstantOp`` without a value) become
    constants whose values the caller supplies when it runs the graph.  ``cast``: read every floating-point
    tensor as this dtype instead of the recorded one (the reference's fixtures are fp32 traces; the attention
    kernel of this backend takes 16-bit operands), as if the module had been cast before it was traced."""
    if not isinstance(data, dict) or not {"inputs", "outputs", "nodes"} <= set(data) or not isinstance(data["nodes"], dict):
        raise IngestError("not a reference graph: expected {'inputs', 'outputs', 'nodes': {id: ...}}")
    nodes: dict = data["nodes"]
    scalars: dict[str, float] = {}
    for nid, nd in nodes.items():
        if nd["op"] in _LATER_STAGES:
            raise IngestError(f"node {nid!r} is a {nd['op']}: only the frontend (traced) and Loop-IR stages of the reference's JSON are read")
        if nd["op"] == "ConstantOp" and nd.get("op_fields", {}).get("value") is not None and list(nd["output"]["shape"]) in ([1], []):
            scalars[nid] = float(nd["op_fields"]["value"])

    g = Graph()

    def shape_of(nid: str) -> tuple[int, ...]:
        shp = nodes[nid]["output"]["shape"]
        if any(not isinstance(d, int) for d in shp):
            raise IngestError(f"node {nid!r} has a symbolic shape {shp}: trace with concrete sizes")
        return tuple(shp)

    def add(nid: str, op, inputs: list[str]) -> None:
        out = nodes[nid]["output"]
        for i in inputs:
            if i not in g.nodes:
                raise IngestError(f"node {nid!r} reads {i!r}, which is not a tensor of the graph")
        g.nodes[nid] = Node(nid, op, list(inputs), Tensor(nid, shape_of(nid), _dtype(out.get("dtype", "f32"), cast)))

    def order() -> list[str]:
        seen: dict[str, int] = {}
        out: list[str] = []

        def visit(n: str) -> None:
            if seen.get(n) == 2:
                return
            if seen.get(n) == 1:
                raise IngestError(f"cycle through {n!r}")
            if n not in nodes:
                raise IngestError(f"unknown node {n!r}")
            seen[n] = 1
            for i in nodes[n]["inputs"]:
                visit(i)
            seen[n] = 2
            out.append(n)

        for n in nodes:
            visit(n)
        return out

    for nid in order():
        nd = nodes[nid]
        kind, fields, ins = nd["op"], nd.get("op_fields", {}) or {}, list(nd["inputs"])
        tensors = [i for i in ins if i not in scalars]
        consts = [scalars[i] for i in ins if i in scalars]
        if kind == "InputOp":
            g.add_input(nid, shape_of(nid), _dtype(nd["output"].get("dtype", "f32"), cast))
        elif kind == "ConstantOp":
            if nid in scalars:
                continue  # folded into its consumers
            g.add_constant(nid, shape_of(nid), _dtype(nd["output"].get("dtype", "f32"), cast), value=fields.get("value"))
        elif kind == "ElementwiseOp":
            fn = _ELEMENTWISE.get(fields.get("op") or fields.get("name") or "")
            if fn is None:
                raise IngestError(f"node {nid!r}: element-wise op {fields!r} is not traced by this backend")
            if len(consts) > 1 or len(tensors) + len(consts) not in (1, 2):
                raise IngestError(f"node {nid!r}: unexpected operands {ins}")
            add(nid, F.ElementwiseOp(fn=fn, scalar=consts[0] if consts else None, scalar_first=bool(consts) and ins[0] in scalars), tensors)
        elif kind == "LinearOp":
            add(nid, F.LinearOp(has_bias=bool(fields.get("has_bias", False))), tensors)
        elif kind == "SdpaOp":
            if len(tensors) not in (3, 4):
                raise IngestError(f"node {nid!r}: attention takes q, k, v and at most an additive mask")
            q, k = shape_of(tensors[0]), shape_of(tensors[1])
            masked = len(tensors) == 4  # an explicit mask replaces the causal term (decomposition/010_sdpa.py:91-101)
            add(nid, F.SdpaOp(is_causal=not masked and bool(fields.get("is_causal", False)), scale=fields.get("scale"), enable_gqa=q[-3] != k[-3], has_mask=masked), tensors)
        elif kind in ("MeanOp", "SumOp"):
            rank = len(shape_of(tensors[0]))
            keep = len(shape_of(nid)) == rank
            add(nid, (F.MeanOp if kind == "MeanOp" else F.SumOp)(axis=int(fields.get("axis", -1)) % rank, keepdim=keep), tensors[:1])
        elif kind == "RmsNormOp":
            add(nid, F.RmsNormOp(eps=float(consts[0]) if consts else float(fields.get("eps", 1e-6)), has_weight=len(tensors) > 1), tensors)
        elif kind == "SoftmaxOp":
            add(nid, F.SoftmaxOp(axis=int(fields.get("axis", -1)) % len(shape_of(tensors[0]))), tensors[:1])
        elif kind == "ReshapeOp":
            add(nid, F.ViewOp(shape=shape_of(nid)), tensors[:1])
        elif kind == "TransposeOp":
            axes = tuple(int(a) for a in fields.get("axes", ()))
            rank = len(shape_of(tensors[0]))
            if len(axes) == 2:
                add(nid, F.TransposeOp(dim0=axes[0] % rank, dim1=axes[1] % rank), tensors[:1])
            elif len(axes) == len(shape_of(tensors[0])):
                add(nid, F.PermuteOp(dims=axes), tensors[:1])
            else:
                raise IngestError(f"node {nid!r}: transpose axes {axes} fit neither a swap nor a permutation")
        elif kind == "UnsqueezeOp":
            dim = int(fields.get("dim", 0))
            add(nid, F.UnsqueezeOp(dim=dim if dim >= 0 else dim + len(shape_of(tensors[0])) + 1), tensors[:1])
        elif kind == "SliceOp":
            if fields.get("dim") is not None:
                dim, start = int(fields["dim"]), int(fields.get("start") or 0)
            elif len(consts) >= 2:
                dim, start = int(consts[0]), int(consts[1])  # legacy convention: [tensor, dim, start, end]
            else:
                raise IngestError(f"node {nid!r}: slice without a recorded dim")
            src = shape_of(tensors[0])
            dim %= len(src)
            add(nid, F.SliceOp(dim=dim, start=start, end=start + shape_of(nid)[dim], step=1), tensors[:1])
        elif kind == "LoopOp":
            from deplodock_amd.ir import loopnest

            try:
                stmts = loopnest.parse_body(fields.get("body") or [])
            except loopnest.LoopNestError as exc:
                raise IngestError(f"node {nid!r}: {exc}") from exc
            add(nid, F.LoopNestOp(stmts=stmts, loads=tuple(tensors), scalars={i: scalars[i] for i in ins if i in scalars}, out_name=nid), tensors)
        elif kind == "CatOp":
            dim = int(consts[-1]) if consts else int(fields.get("dim", -1))
            add(nid, F.CatOp(dim=dim % len(shape_of(tensors[0]))), tensors)
        else:
            raise IngestError(f"node {nid!r}: op {kind!r} is not part of the frontend stage this backend reads")
    for name in (*data["inputs"], *data["outputs"]):
        if name not in g.nodes:
            raise IngestError(f"boundary tensor {name!r} is not a node")
    g.inputs = list(data["inputs"])
    g.outputs = list(data["outputs"])
    return g


def load_reference_graph(path: str | Path, cast: DType | None = None) -> Graph:
    return graph_from_reference_dict(json.loads(Path(path).read_text()), cast)


__all__ = ["IngestError", "graph_from_reference_dict", "load_reference_graph", "InputOp", "ConstantOp"]
