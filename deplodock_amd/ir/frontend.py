"""Torch IR — one op per traced ATen call.

What each op *means* is fixed by the reference's frontend ops
(emmy/compiler/ir/frontend/ir.py:201-358: LinearOp :212-217 ``x @ W.T``,
SdpaOp :252-275, RmsNormOp :309-312, SoftmaxOp :354-358) and their
decompositions (emmy/compiler/pipeline/passes/frontend/decomposition/*).
The ops here only *describe*; nothing in the product evaluates them on the
host — the fusion pass turns them into scheduled tile kernels.
"""

from __future__ import annotations

from dataclasses import dataclass

from deplodock_amd.dtype import DType
from deplodock_amd.ir.base import Op

ELEMENTWISE_UNARY = {"neg", "rsqrt", "sqrt", "exp", "silu", "sigmoid", "tanh", "abs", "reciprocal"}
ELEMENTWISE_BINARY = {"add", "sub", "mul", "div", "pow", "maximum", "minimum"}


@dataclass
class ElementwiseOp(Op):
    """``fn`` over one or two tensor inputs with numpy broadcasting.  A python
    scalar operand is carried in ``scalar`` (``scalar_first`` when it was the
    left operand)."""

    fn: str = ""
    scalar: float | None = None
    scalar_first: bool = False


@dataclass
class CastOp(Op):
    """``x.to(dtype)``; the node's output dtype is the target."""

    dtype: DType | None = None


@dataclass
class MeanOp(Op):
    axis: int = -1
    keepdim: bool = False


@dataclass
class SumOp(Op):
    axis: int = -1
    keepdim: bool = False


@dataclass
class AmaxOp(Op):
    """``amax`` over one axis (the reference keeps torch's name for it, emmy/compiler/trace/torch.py:590-598)."""

    axis: int = -1
    keepdim: bool = False


@dataclass
class LayerNormOp(Op):
    """``(x - mean) * rsqrt(var + eps) [* weight] [+ bias]`` over the last axis, biased variance
    (frontend/ir.py:316-341, decomposition/085_layer_norm.py).  Inputs: ``x[, weight[, bias]]``."""

    eps: float = 1e-5
    has_weight: bool = False
    has_bias: bool = False


@dataclass
class LinearOp(Op):
    """``x @ W.T (+ b)`` with ``W`` of shape ``[out, in]`` (frontend/ir.py:212-217)."""

    has_bias: bool = False


@dataclass
class BatchedLinearOp(Op):
    """``x[p] @ w[p].T`` for every ``p`` of a leading batch axis: ``x`` is ``[P, M, K]``, ``w`` is ``[P, N, K]`` or
    ``[1, N, K]`` (one weight for every product), the result ``[P, M, N]`` — the per-head products of attention
    written as contractions (``LinearOp`` semantics, emmy/compiler/ir/frontend/ir.py:212-217, per batch entry)."""


@dataclass
class MatmulOp(Op):
    """``a @ b`` with numpy semantics on the last two axes: ``a`` is ``[..., M, K]``, ``b`` is ``[K, N]`` or
    ``[..., K, N]`` with the same leading axes (emmy/compiler/ir/frontend/ir.py ``MatmulOp``; the reference
    decomposes it into a broadcast multiply and a sum, decomposition/070_matmul.py)."""


@dataclass
class RmsNormOp(Op):
    """``x * rsqrt(mean(x^2, -1) + eps) * w`` (frontend/ir.py:309-312)."""

    eps: float = 1e-6
    has_weight: bool = True


@dataclass
class SoftmaxOp(Op):
    """``exp(x - max) / sum(exp(x - max))`` along ``axis`` (frontend/ir.py:354-358)."""

    axis: int = -1


@dataclass
class SdpaOp(Op):
    """``softmax(q k^T * scale + mask) v``; causal masks ``j > i``; grouped KV
    heads use ``kv_head = q_head // group`` (frontend/ir.py:252-275,
    decomposition/010_sdpa.py:28-138)."""

    is_causal: bool = False
    scale: float | None = None
    enable_gqa: bool = False
    has_mask: bool = False  # a fourth input: an additive float bias on the scaled scores (emmy/compiler/trace/torch.py:559-583)


@dataclass
class LoopNestOp(Op):
    """A kernel of the reference's Loop IR (a ``LoopOp``: post-fusion, pre-tiling; emmy/compiler/ir/loop/ir.py:89)
    kept as its statements (``ir/loopnest.py``).  ``loads`` names, per graph input of the node, the name the body's
    ``Load`` statements use for it; ``scalars`` are shape-[1] constants with a recorded value, folded into the body."""

    stmts: tuple = ()
    loads: tuple = ()
    scalars: dict = None
    out_name: str = ""
    label: str = ""  # kernel label (default: from the node id)


@dataclass
class ViewOp(Op):
    """``view`` / ``reshape`` / ``flatten`` to ``shape`` (row-major reinterpretation)."""

    shape: tuple = ()


@dataclass
class TransposeOp(Op):
    dim0: int = 0
    dim1: int = 1


@dataclass
class PermuteOp(Op):
    dims: tuple = ()


@dataclass
class UnsqueezeOp(Op):
    dim: int = 0


@dataclass
class ExpandOp(Op):
    """``expand``: size-1 dims (and new leading dims) repeated up to ``shape`` without moving data — every
    repeated index reads element 0 (emmy/compiler/trace/torch.py:666-676: a broadcast, not a reshape)."""

    shape: tuple = ()


@dataclass
class SqueezeOp(Op):
    dim: int = 0


@dataclass
class SliceOp(Op):
    dim: int = 0
    start: int = 0
    end: int | None = None
    step: int = 1


@dataclass
class CatOp(Op):
    dim: int = 0


@dataclass
class GatherOp(Op):
    """Whole slices picked by an integer vector along ``axis``: ``embedding(table, idx)`` (axis 0, ``idx`` of any
    shape) and ``index_select(x, axis, idx)`` (the reference's ``GatherOp``, emmy/compiler/trace/torch.py:738-756).
    Inputs: ``x, idx``."""

    axis: int = 0


@dataclass
class ContiguousOp(Op):
    """``contiguous`` / ``clone``: a value-preserving copy."""
