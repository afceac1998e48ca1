"""Evaluating a frontend graph in the reference's JSON form, node by node, on the CPU.

TEST INFRASTRUCTURE ONLY (see ``oracle/__init__.py``).  Two interpreters of the same format
(``Graph.to_dict``, emmy/compiler/graph.py:952-1000; read back by ``Graph.from_dict`` :875-907):

``evaluate_numpy``  float64 numpy, each op as the reference's own ``Op.forward`` defines it
                    (emmy/compiler/ir/frontend/ir.py: ``TransposeOp`` :54-61, ``SliceOp`` :122-136, ``CatOp``
                    :138-178, ``UnsqueezeOp`` :191-193, ``LinearOp`` :212-217, ``SdpaOp`` :252-275, ``MeanOp``
                    :291-292; element-wise names as ``emmy/compiler/ir/elementwise.py:36-78`` defines them),
                    through ``oracle.emmy_ops`` where a restatement exists;
``evaluate_torch``  PyTorch eager, one torch call per node, in the dtype of the values it is given — the
                    prescribed oracle (eager on the same computation), with eager's per-op rounding in 16-bit.

Recorded output shapes are not trusted: shapes follow from the operands, so the same graph evaluates at
other operand ranks (the committed TinyLlama trace was taken with ``[1, 1, S, D]`` rotary tables, which makes
its attention operands five-dimensional; fed ``[1, S, D]`` tables the same node list is the ordinary Llama
block, which is what pins these interpreters against ``transformers``' ``LlamaDecoderLayer``).
"""

from __future__ import annotations

import numpy as np

from oracle import emmy_ops as O

_BIG = 2**62


def _scalars(nodes: dict) -> dict[str, float]:
    return {nid: float(nd["op_fields"]["value"]) for nid, nd in nodes.items()
            if nd["op"] == "ConstantOp" and nd.get("op_fields", {}).get("value") is not None and list(nd["output"]["shape"]) in ([1], [])}  # fmt: skip


def _order(nodes: dict) -> list[str]:
    seen: set[str] = set()
    out: list[str] = []

    def visit(n: str) -> None:
        if n in seen:
            return
        seen.add(n)
        for i in nodes[n]["inputs"]:
            visit(i)
        out.append(n)

    for n in nodes:
        visit(n)
    return out


def _reshape_target(fields: dict, x_shape: tuple[int, ...]) -> tuple[int, ...]:
    """``ReshapeOp.shape`` with its one ``-1`` resolved (frontend/ir.py:81-92)."""
    shape = [int(d) for d in fields["shape"]]
    if -1 in shape:
        known = int(np.prod([d for d in shape if d != -1])) if len(shape) > 1 else 1
        shape[shape.index(-1)] = int(np.prod(x_shape)) // known
    return tuple(shape)


def _slice_args(fields: dict, consts: list[float], x_shape: tuple[int, ...], rec_shape: list[int]) -> tuple[int, int, int]:
    """``(dim, start, end)``: recorded fields (``dim`` / ``start`` and the output extent) or the legacy
    ``[tensor, dim, start, end]`` inputs, the end clamped to the operand (frontend/ir.py:100-136)."""
    if fields.get("dim") is not None:
        dim, start = int(fields["dim"]) % len(x_shape), int(fields.get("start") or 0)
        return dim, start, min(start + int(rec_shape[dim]), x_shape[dim])
    dim, start, end = int(consts[0]) % len(x_shape), int(consts[1]), consts[2]
    return dim, start, x_shape[dim] if end >= _BIG else min(int(end), x_shape[dim])


_NP_UNARY = {
    "negative": lambda a: -a, "neg": lambda a: -a, "rsqrt": lambda a: 1.0 / np.sqrt(a), "sqrt": np.sqrt, "exp": np.exp, "silu": O.silu,
    "sigmoid": lambda a: 1.0 / (1.0 + np.exp(-a)), "tanh": np.tanh, "abs": np.abs, "reciprocal": lambda a: 1.0 / a,
}  # fmt: skip
_NP_BINARY = {
    "add": np.add, "subtract": np.subtract, "sub": np.subtract, "multiply": np.multiply, "mul": np.multiply, "divide": np.divide, "div": np.divide,
    "pow": np.power, "maximum": np.maximum, "minimum": np.minimum,
}  # fmt: skip


def evaluate_numpy(data: dict, values: dict[str, np.ndarray]) -> dict[str, np.ndarray]:
    """Every tensor of the graph in float64.  ``values`` supplies inputs and weights by node id."""
    nodes, scal = data["nodes"], _scalars(data["nodes"])
    env: dict[str, np.ndarray] = {}
    for nid in _order(nodes):
        nd = nodes[nid]
        kind, fields, ins = nd["op"], nd.get("op_fields", {}) or {}, nd["inputs"]
        if nid in scal:
            continue
        ts = [env[i] for i in ins if i not in scal]
        cs = [scal[i] for i in ins if i in scal]
        if kind in ("InputOp", "ConstantOp"):
            env[nid] = np.asarray(values[nid], dtype=np.float64)
        elif kind == "ElementwiseOp":
            name = fields.get("op") or fields.get("name")
            if name in _NP_UNARY and len(ts) == 1 and not cs:
                env[nid] = _NP_UNARY[name](ts[0])
            else:
                a, b = (cs[0], ts[0]) if cs and ins[0] in scal else (ts[0], cs[0]) if cs else (ts[0], ts[1])
                env[nid] = _NP_BINARY[name](a, b)
        elif kind == "LinearOp":
            env[nid] = O.linear(ts[0], ts[1], ts[2] if fields.get("has_bias") else None)
        elif kind == "SdpaOp":
            q, k, v = ts[:3]
            while k.ndim < q.ndim:
                k = k[None]
            while v.ndim < q.ndim:
                v = v[None]
            env[nid] = O.sdpa(q, k, v, is_causal=bool(fields.get("is_causal", False)), scale=fields.get("scale"), mask=ts[3] if len(ts) > 3 else None)
        elif kind == "MeanOp":
            env[nid] = np.mean(ts[0], axis=int(fields.get("axis", -1)), keepdims=len(nd["output"]["shape"]) == len(nodes[ins[0]]["output"]["shape"]))
        elif kind == "ReshapeOp":
            env[nid] = np.reshape(ts[0], _reshape_target(fields, ts[0].shape))
        elif kind == "TransposeOp":
            axes = [int(a) for a in fields["axes"]]
            env[nid] = np.swapaxes(ts[0], axes[0] % ts[0].ndim, axes[1] % ts[0].ndim) if len(axes) == 2 else np.transpose(ts[0], axes)
        elif kind == "UnsqueezeOp":
            env[nid] = np.expand_dims(ts[0], int(fields.get("dim", 0)))
        elif kind == "SliceOp":
            dim, start, end = _slice_args(fields, cs, ts[0].shape, nd["output"]["shape"])
            env[nid] = np.take(ts[0], np.arange(start, end), axis=dim)
        elif kind == "CatOp":
            env[nid] = np.concatenate(ts, axis=int(cs[-1]) if cs else -1)
        else:
            raise NotImplementedError(f"{nid}: {kind}")
    return env


def evaluate_torch(data: dict, values: dict, outputs_only: bool = True):
    """The graph through PyTorch eager, one call per node, on the device and in the dtype of ``values``."""
    import torch
    import torch.nn.functional as Fn

    nodes, scal = data["nodes"], _scalars(data["nodes"])
    unary = {"negative": torch.neg, "neg": torch.neg, "rsqrt": torch.rsqrt, "sqrt": torch.sqrt, "exp": torch.exp, "silu": Fn.silu, "sigmoid": torch.sigmoid,
             "tanh": torch.tanh, "abs": torch.abs, "reciprocal": torch.reciprocal}  # fmt: skip
    binary = {"add": torch.add, "subtract": torch.sub, "sub": torch.sub, "multiply": torch.mul, "mul": torch.mul, "divide": torch.div, "div": torch.div,
              "pow": torch.pow, "maximum": torch.maximum, "minimum": torch.minimum}  # fmt: skip
    env: dict = {}
    with torch.no_grad():
        for nid in _order(nodes):
            nd = nodes[nid]
            kind, fields, ins = nd["op"], nd.get("op_fields", {}) or {}, nd["inputs"]
            if nid in scal:
                continue
            ts = [env[i] for i in ins if i not in scal]
            cs = [scal[i] for i in ins if i in scal]
            if kind in ("InputOp", "ConstantOp"):
                env[nid] = values[nid]
            elif kind == "ElementwiseOp":
                name = fields.get("op") or fields.get("name")
                if name in unary and len(ts) == 1 and not cs:
                    env[nid] = unary[name](ts[0])
                else:
                    a, b = (cs[0], ts[0]) if cs and ins[0] in scal else (ts[0], cs[0]) if cs else (ts[0], ts[1])
                    env[nid] = binary[name](a, b)
            elif kind == "LinearOp":
                env[nid] = Fn.linear(ts[0], ts[1], ts[2] if fields.get("has_bias") else None)
            elif kind == "SdpaOp":
                q, k, v = ts[:3]
                while k.ndim < q.ndim:
                    k = k[None]
                while v.ndim < q.ndim:
                    v = v[None]
                lead = q.shape[:-3]
                mask = ts[3].expand(*lead, *ts[3].shape[-3:]).reshape(-1, *ts[3].shape[-3:]) if len(ts) > 3 else None
                o = Fn.scaled_dot_product_attention(q.reshape(-1, *q.shape[-3:]), k.reshape(-1, *k.shape[-3:]), v.reshape(-1, *v.shape[-3:]), attn_mask=mask,
                                                    is_causal=mask is None and bool(fields.get("is_causal", False)), scale=fields.get("scale"), enable_gqa=q.shape[-3] != k.shape[-3])  # fmt: skip
                env[nid] = o.reshape(*lead, *o.shape[-3:])
            elif kind == "MeanOp":
                env[nid] = torch.mean(ts[0], dim=int(fields.get("axis", -1)), keepdim=len(nd["output"]["shape"]) == len(nodes[ins[0]]["output"]["shape"]))
            elif kind == "ReshapeOp":
                env[nid] = ts[0].reshape(_reshape_target(fields, tuple(ts[0].shape)))
            elif kind == "TransposeOp":
                axes = [int(a) for a in fields["axes"]]
                env[nid] = ts[0].transpose(axes[0], axes[1]) if len(axes) == 2 else ts[0].permute(axes)
            elif kind == "UnsqueezeOp":
                env[nid] = ts[0].unsqueeze(int(fields.get("dim", 0)))
            elif kind == "SliceOp":
                dim, start, end = _slice_args(fields, cs, tuple(ts[0].shape), nd["output"]["shape"])
                env[nid] = ts[0].narrow(dim, start, end - start)
            elif kind == "CatOp":
                env[nid] = torch.cat(ts, dim=int(cs[-1]) if cs else -1)
            else:
                raise NotImplementedError(f"{nid}: {kind}")
    return {o: env[o] for o in data["outputs"]} if outputs_only else env


def random_values(data: dict, seed: int = 0, weight_std: float = 0.02, shapes: dict | None = None) -> dict:
    """Seeded fp32 torch tensors for every input and weight: inputs ~N(0,1), matrices ~N(0, weight_std), vectors
    (norm weights) ~N(1, 0.1), rotary tables a real ``cos`` / ``sin`` of positions 0..S-1.  ``shapes`` overrides
    recorded shapes by node id."""
    import torch

    gen = torch.Generator().manual_seed(seed)
    out = {}
    for nid, nd in data["nodes"].items():
        if nd["op"] not in ("InputOp", "ConstantOp") or nd.get("op_fields", {}).get("value") is not None:
            continue
        shape = tuple((shapes or {}).get(nid, nd["output"]["shape"]))
        if nid.startswith("position_embeddings"):
            s, d = shape[-2], shape[-1]
            ang = torch.arange(s, dtype=torch.float32)[:, None] * (1e4 ** (-torch.arange(0, d, 2, dtype=torch.float32) / d))[None]
            emb = torch.cat((ang, ang), -1)
            out[nid] = (emb.cos() if nid.endswith("_0") else emb.sin()).reshape(shape)
        elif nd["op"] == "InputOp":
            out[nid] = torch.randn(shape, generator=gen)
        elif len(shape) == 1 and "bias" not in nid:
            out[nid] = 1.0 + 0.1 * torch.randn(shape, generator=gen)
        else:
            out[nid] = weight_std * torch.randn(shape, generator=gen)
    return out


__all__ = ["evaluate_numpy", "evaluate_torch", "random_values"]
