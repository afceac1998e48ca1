"""JSON form of traced and lowered graphs (on-disk kernel reproducers).

The reference writes every IR stage as JSON (``Graph.to_dict`` /
``Graph.from_dict``, emmy/compiler/graph.py:357-900) and keeps a corpus of
single-kernel reproducers (``kernels/*.json``) that ``emmy run --ir`` replays.
Two stages are serialisable here: the traced frontend graph (``stage:
"torch"``) and the lowered ``Graph[HipOp]`` (``stage: "hip"``: kernel source,
launch geometry, argument order, knobs).  Tensor *values* are never written —
a reloaded graph runs on seeded random data, as the reference's ``--ir`` does.

A lowered graph whose kernels take a size at run time keeps its symbolic parts: shapes
with ``seq_len`` / ``a * seq_len + b`` dims, launch-time grid factors (``CeilDiv``,
``XcdRounds``), the trailing ``int`` arguments, and the symbol's traced size (what a replay
on synthetic inputs runs at) — the reference's JSON likewise keeps ``Dim`` expressions and
symbolic grid factors (emmy/compiler/ir/cuda/ir.py:66-112).
"""

from __future__ import annotations

import dataclasses
import json
from pathlib import Path

from deplodock_amd import dtype as dt
from deplodock_amd.graph import Graph, Node, Tensor
from deplodock_amd.ir import frontend as F
from deplodock_amd.ir import loopnest as _loopnest
from deplodock_amd.ir.base import ConstantOp, InputOp, Op
from deplodock_amd.ir.hip import HipOp
from deplodock_amd.ir.sym import Affine, CeilDiv, XcdRounds

FORMAT = 1
_SKIP_FIELDS = {"source"}
_OPS = {cls.__name__: cls for cls in (InputOp, ConstantOp, HipOp, *(v for v in vars(F).values() if isinstance(v, type) and issubclass(v, Op) and v is not Op))}


class SerializeError(TypeError):
    """The graph holds something with no JSON form (a tile body, a python callable as a launch factor)."""


@dataclasses.dataclass
class TracedSizes:
    """What a reloaded runtime-int graph remembers of its dynamic trace: the symbol's traced size.  (The module
    itself is not in the file, so a reloaded graph cannot be re-traced at another size — it does not need to.)"""

    hints: dict


_LOOP_IR = ("Var", "Lit", "Bin", "Ternary", "Load", "Assign", "Accum", "Select", "Write", "Loop")  # statements of a LoopNestOp (ir/loopnest.py)


def _enc(v, where: str):
    if isinstance(v, dt.DType):
        return {"$dtype": v.name}
    if isinstance(v, (str, int, float, bool)) or v is None:
        return v
    if isinstance(v, Affine):
        return {"$affine": [v.name, v.a, v.b]}
    if isinstance(v, CeilDiv):
        return {"$ceildiv": [_enc(v.value, where), v.div]}
    if isinstance(v, XcdRounds):
        return {"$xcdrounds": [_enc(v.m, where), v.tile_m, v.blocks_n, v.per_block, v.xcds]}
    if isinstance(v, (tuple, list)):
        return {"$tuple": [_enc(x, where) for x in v]} if isinstance(v, tuple) else [_enc(x, where) for x in v]
    if isinstance(v, dict):
        return {"$dict": {str(k): _enc(x, where) for k, x in v.items()}}
    if type(v).__name__ in _LOOP_IR and type(v) is getattr(_loopnest, type(v).__name__):
        return {"$loop": [type(v).__name__, *(_enc(getattr(v, f.name), where) for f in dataclasses.fields(v))]}
    raise SerializeError(f"{where}: cannot serialise {type(v).__name__}")


def _dec(v):
    if isinstance(v, dict):
        if "$dtype" in v:
            return dt.by_name(v["$dtype"])
        if "$tuple" in v:
            return tuple(_dec(x) for x in v["$tuple"])
        if "$dict" in v:
            return {k: _dec(x) for k, x in v["$dict"].items()}
        if "$affine" in v:
            name, a, b = v["$affine"]
            return Affine(str(name), int(a), int(b))
        if "$ceildiv" in v:
            return CeilDiv(_dec(v["$ceildiv"][0]), int(v["$ceildiv"][1]))
        if "$xcdrounds" in v:
            m, *rest = v["$xcdrounds"]
            return XcdRounds(_dec(m), *(int(x) for x in rest))
        if "$loop" in v:
            kind, *fields = v["$loop"]
            if kind not in _LOOP_IR:
                raise SerializeError(f"unknown Loop-IR statement {kind!r}")
            return getattr(_loopnest, kind)(*(_dec(x) for x in fields))
        raise SerializeError(f"unknown encoded object {sorted(v)}")
    if isinstance(v, list):
        return [_dec(x) for x in v]
    return v


def op_to_dict(op: Op, where: str = "op") -> dict:
    name = type(op).__name__
    if name not in _OPS:
        raise SerializeError(f"{where}: {name} has no JSON form (only traced and lowered graphs are serialisable)")
    out = {"type": name}
    for f in dataclasses.fields(op):
        if f.name in _SKIP_FIELDS:
            continue
        out[f.name] = _enc(getattr(op, f.name), f"{where}.{f.name}")
    return out


def op_from_dict(d: dict) -> Op:
    cls = _OPS.get(d.get("type"))
    if cls is None:
        raise SerializeError(f"unknown op type {d.get('type')!r}")
    known = {f.name for f in dataclasses.fields(cls)}
    return cls(**{k: _dec(v) for k, v in d.items() if k != "type" and k in known})


def _hints_to_dict(hints: dict, where: str) -> dict:
    from deplodock_amd.passes.fuse import StackedConstant

    out = {}
    for k, v in hints.items():
        if isinstance(v, StackedConstant):
            out[k] = {"$stacked": list(v.parts), **({"k_scale": v.k_scale} if v.k_scale else {}), **({"transpose": True} if v.transpose else {}), **({"pad_rows_to": v.pad_rows_to} if v.pad_rows_to else {})}
        else:
            out[k] = _enc(v, f"{where}.hints[{k}]")
    return out


def _hints_from_dict(d: dict) -> dict:
    from deplodock_amd.passes.fuse import StackedConstant

    return {k: StackedConstant(tuple(v["$stacked"]), k_scale=v.get("k_scale"), transpose=bool(v.get("transpose", False)), pad_rows_to=int(v.get("pad_rows_to", 0))) if isinstance(v, dict) and "$stacked" in v else _dec(v) for k, v in d.items()}


def graph_to_dict(g: Graph) -> dict:
    stage = "hip" if any(isinstance(n.op, HipOp) for n in g.nodes.values()) else "torch"
    nodes = []
    for nid in g.topological_order():
        n = g.nodes[nid]
        nodes.append(
            {
                "id": nid,
                "op": op_to_dict(n.op, nid),
                "inputs": list(n.inputs),
                "shape": [d if isinstance(d, str) else _enc(d, nid) if isinstance(d, Affine) else int(d) for d in n.output.shape],
                "dtype": n.output.dtype.name,
                "hints": _hints_to_dict(n.hints, nid),
            }
        )
    out = {"format": FORMAT, "stage": stage, "arch": "gfx950", "inputs": list(g.inputs), "outputs": list(g.outputs), "nodes": nodes}
    if getattr(g, "symbolic", None) is not None:
        out["symbolic"] = {"name": g.symbolic, "hints": {k: int(v) for k, v in (getattr(getattr(g, "dynamic", None), "hints", {}) or {}).items()}}
    return out


def graph_from_dict(d: dict) -> Graph:
    if d.get("format") != FORMAT:
        raise SerializeError(f"unsupported graph format {d.get('format')!r}")
    g = Graph()
    for nd in d["nodes"]:
        op = op_from_dict(nd["op"])
        t = Tensor(nd["id"], tuple(_dec(d_) for d_ in nd["shape"]), dt.by_name(nd["dtype"]), constant=isinstance(op, ConstantOp), value=getattr(op, "value", None))
        for i in nd["inputs"]:
            if i not in g.nodes:
                raise SerializeError(f"node {nd['id']!r} references {i!r} before it is defined")
        g.nodes[nd["id"]] = Node(nd["id"], op, list(nd["inputs"]), t, _hints_from_dict(nd.get("hints", {})))
    g.inputs = list(d["inputs"])
    g.outputs = list(d["outputs"])
    g.stage = d.get("stage", "torch")
    if d.get("symbolic"):
        g.symbolic = str(d["symbolic"]["name"])
        g.dynamic = TracedSizes({str(k): int(v) for k, v in d["symbolic"].get("hints", {}).items()})
    return g


def save(g: Graph, path: str | Path) -> None:
    Path(path).write_text(json.dumps(graph_to_dict(g), indent=1) + "\n")


def load(path: str | Path) -> Graph:
    return graph_from_dict(json.loads(Path(path).read_text()))


def random_inputs(g: Graph, seed: int = 0, device=None, sizes: dict | None = None) -> dict:
    """Seeded random tensors for every input and every constant without a static
    value (stacked constants are left to the binder when their parts exist).  A symbolic
    dim takes its size from ``sizes``, else the size the graph was traced at."""
    import torch

    from deplodock_amd.ir.sym import resolve

    gen = torch.Generator().manual_seed(seed)
    out = {}
    env = {**(getattr(getattr(g, "dynamic", None), "hints", {}) or {}), **(sizes or {})}
    stacked_parts = {p for n in g.nodes.values() for p in getattr(n.hints.get("stacked"), "parts", ())}
    for nid, n in g.nodes.items():
        if not isinstance(n.op, (InputOp, ConstantOp)) or (isinstance(n.op, ConstantOp) and n.op.value is not None):
            continue
        if n.hints.get("stacked") is not None and all(p in g.nodes for p in n.hints["stacked"].parts):
            continue
        scale = 0.05 if isinstance(n.op, ConstantOp) else 1.0
        t = (scale * torch.randn(tuple(resolve(d, env) for d in n.output.shape), generator=gen)).to({"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}.get(n.output.dtype.name, torch.float32))
        out[nid] = t.to(device) if device is not None else t
    del stacked_parts
    return out
