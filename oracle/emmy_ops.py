"""Numpy restatement of the semantics the hot-path kernels must reproduce.

TEST INFRASTRUCTURE ONLY (see ``oracle/__init__.py``).  All arithmetic is done
in float64 unless a function says otherwise, so the restatement is a *more*
exact statement of the math than any fp32 implementation; callers compare with
a tolerance.
"""

from __future__ import annotations

import numpy as np

# ---------------------------------------------------------------------------
# bf16 carrier
# ---------------------------------------------------------------------------


def bf16_round(x: np.ndarray) -> np.ndarray:
    """Round fp32 values to bf16 precision (round-to-nearest-even), returned as fp32.

    Follows the closed form the reference uses to encode bf16 constants,
    emmy/compiler/backend/cuda/program.py:259-263:
    ``bits = (bits + 0x7FFF + ((bits >> 16) & 1)) >> 16``."""
    x32 = np.ascontiguousarray(x, dtype=np.float32)
    bits = x32.view(np.uint32).astype(np.uint64)
    rounded = ((bits + 0x7FFF + ((bits >> 16) & 1)) >> 16).astype(np.uint32) << 16
    out = rounded.astype(np.uint32).view(np.float32).reshape(x32.shape).copy()
    nan = np.isnan(x32)
    if nan.any():
        out[nan] = np.nan
    return out


def bf16_bits(x: np.ndarray) -> np.ndarray:
    """bf16 bit patterns (uint16) of fp32 values, same rounding as :func:`bf16_round`."""
    return (bf16_round(x).view(np.uint32) >> 16).astype(np.uint16)


def from_bf16_bits(bits: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


# ---------------------------------------------------------------------------
# Frontend op semantics
# ---------------------------------------------------------------------------


def rms_norm(x: np.ndarray, weight: np.ndarray | None, eps: float) -> np.ndarray:
    """``x * rsqrt(mean(x*x, -1) + eps) * weight``.

    emmy/compiler/ir/frontend/ir.py:309-312 (``RmsNormOp.forward``) and its
    decomposition emmy/compiler/pipeline/passes/frontend/decomposition/080_rms_norm.py:25-57
    (+ 090_mean.py:27-44: sum, divide by count, add eps, rsqrt, times x, times w)."""
    x = np.asarray(x, dtype=np.float64)
    ms = np.sum(x * x, axis=-1, keepdims=True) / x.shape[-1]
    y = x * (1.0 / np.sqrt(ms + eps))
    if weight is not None:
        y = y * np.asarray(weight, dtype=np.float64)
    return y


def rms_norm_sum(x: np.ndarray, weight: np.ndarray, eps: float) -> np.ndarray:
    """The sum-based variant the reference's own e2e tests build by hand,
    ``x * rsqrt(sum(x*x, -1) + eps) * w`` (tests/compiler/e2e/test_accuracy.py:184-212,
    test_ops_vs_torch.py:428-449)."""
    x = np.asarray(x, dtype=np.float64)
    return x * (1.0 / np.sqrt(np.sum(x * x, axis=-1, keepdims=True) + eps)) * np.asarray(weight, dtype=np.float64)


def softmax(x: np.ndarray, axis: int = -1) -> np.ndarray:
    """``exp(x - max) / sum(exp(x - max))`` — emmy/compiler/ir/frontend/ir.py:354-358,
    decomposition ``_helpers.softmax_decompose`` (_helpers.py:113-146)."""
    x = np.asarray(x, dtype=np.float64)
    m = np.max(x, axis=axis, keepdims=True)
    e = np.exp(x - m)
    return e / np.sum(e, axis=axis, keepdims=True)


def linear(x: np.ndarray, w: np.ndarray, bias: np.ndarray | None = None) -> np.ndarray:
    """``x @ w.T (+ bias)`` with ``w`` of shape ``[out, in]`` —
    emmy/compiler/ir/frontend/ir.py:212-217; decomposition 040_linear.py
    (transpose W, then ``matmul_decompose`` = broadcast multiply + sum over K,
    _helpers.py:87-110)."""
    y = np.asarray(x, dtype=np.float64) @ np.asarray(w, dtype=np.float64).T
    if bias is not None:
        y = y + np.asarray(bias, dtype=np.float64)
    return y


def silu(x: np.ndarray) -> np.ndarray:
    """``x * 1/(1 + exp(-x))`` — decomposition/020_silu.py; sigmoid definition
    emmy/compiler/ir/elementwise.py:70-78."""
    x = np.asarray(x, dtype=np.float64)
    return x * (1.0 / (1.0 + np.exp(-x)))


def sdpa(q: np.ndarray, k: np.ndarray, v: np.ndarray, *, is_causal: bool, scale: float | None = None, mask: np.ndarray | None = None) -> np.ndarray:
    """``softmax(q k^T * scale + causal) v`` with grouped KV heads.  ``mask``: an additive bias broadcast onto
    the scaled scores; it replaces the causal term (decomposition/010_sdpa.py:91-101: ``if inp_mask is not
    None ... elif root.op.is_causal``).

    emmy/compiler/ir/frontend/ir.py:252-275 (``SdpaOp.forward``: K/V heads are
    repeated ``group = Hq // Hkv`` times, i.e. ``kv_head = q_head // group``;
    causal subtracts 1e9 where ``j > i``) and decomposition/010_sdpa.py:28-49,
    79-138 (scale = 1/sqrt(head_dim))."""
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    if k.shape[-3] != q.shape[-3]:
        group = q.shape[-3] // k.shape[-3]
        k = np.repeat(k, group, axis=-3)
        v = np.repeat(v, group, axis=-3)
    d = q.shape[-1]
    s = (q @ np.swapaxes(k, -2, -1)) * (scale if scale is not None else 1.0 / np.sqrt(d))
    if mask is not None:
        s = s + np.asarray(mask, dtype=np.float64)
    elif is_causal:
        sq, sk = s.shape[-2], s.shape[-1]
        s = s - np.triu(np.ones((sq, sk)), k=1) * 1e9
    return softmax(s, -1) @ v


# ---------------------------------------------------------------------------
# Streaming carriers (what the fused kernels iterate)
# ---------------------------------------------------------------------------


def online_softmax_merge(a: tuple[np.ndarray, np.ndarray], b: tuple[np.ndarray, np.ndarray]) -> tuple[np.ndarray, np.ndarray]:
    """Combine two partial softmax states ``(m, d)``:
    ``M = max(m, m')``, ``d = d*exp(m - M) + d'*exp(m' - M)``.

    The ``exp``-family monoid of emmy/compiler/ir/stmt/carrier.py:279-345 as
    instantiated for softmax in passes/lowering/tile/_softmax.py:35-123."""
    (m1, d1), (m2, d2) = a, b
    m = np.maximum(m1, m2)
    return m, d1 * np.exp(m1 - m) + d2 * np.exp(m2 - m)


def online_softmax(x: np.ndarray, block: int) -> np.ndarray:
    """Softmax over the last axis computed by folding blocks of ``block`` columns
    with :func:`online_softmax_merge`, then one normalising sweep."""
    x = np.asarray(x, dtype=np.float64)
    n = x.shape[-1]
    state = (np.full(x.shape[:-1], -1e30), np.zeros(x.shape[:-1]))
    for s in range(0, n, block):
        xb = x[..., s : s + block]
        mb = xb.max(-1)
        state = online_softmax_merge(state, (mb, np.exp(xb - mb[..., None]).sum(-1)))
    m, d = state
    return np.exp(x - m[..., None]) / d[..., None]


def flash_attention(q: np.ndarray, k: np.ndarray, v: np.ndarray, *, is_causal: bool, scale: float, block_kv: int, mask: np.ndarray | None = None) -> np.ndarray:
    """Streaming attention over key blocks with the ``(m, l, O)`` carrier:
    statistics start at ``m = -1e30, l = 0``; per block ``mn = max(m, rowmax)``,
    ``alpha = exp(m - mn)``, ``p = exp(s - mn)``, ``l = l*alpha + sum p``,
    ``O = O*alpha + p v``; close ``O / l``.  Masked scores are ``-1e30``.

    emmy/compiler/pipeline/passes/lowering/kernel/_twist.py:229-363 (stats init
    :268-270, close :341-362), combine passes/lowering/tile/_flash.py:96-110,
    GQA ``head // group`` :116-125; the hand-written FA-2 kernel in
    tests/compiler/e2e/test_attention_coverage.py:557-639 is the same algorithm."""
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    B, Hq, Sq, D = q.shape
    Hkv, Skv = k.shape[1], k.shape[2]
    group = Hq // Hkv
    out = np.zeros((B, Hq, Sq, v.shape[-1]))
    rows = np.arange(Sq)[:, None]
    bias = None if mask is None else np.broadcast_to(np.asarray(mask, dtype=np.float64), (B, Hq, Sq, Skv))
    for b in range(B):
        for h in range(Hq):
            kh, vh = k[b, h // group], v[b, h // group]
            m = np.full(Sq, -1e30)
            l = np.zeros(Sq)
            o = np.zeros((Sq, v.shape[-1]))
            for s0 in range(0, Skv, block_kv):
                s = (q[b, h] @ kh[s0 : s0 + block_kv].T) * scale
                if bias is not None:  # the block's slice of the additive mask, in place of the causal term
                    s = s + bias[b, h, :, s0 : s0 + block_kv]
                elif is_causal:
                    cols = np.arange(s0, min(s0 + block_kv, Skv))[None, :]
                    s = np.where(cols > rows, -1e30, s)
                mn = np.maximum(m, s.max(-1))
                alpha = np.exp(m - mn)
                p = np.exp(s - mn[:, None])
                l = l * alpha + p.sum(-1)
                o = o * alpha[:, None] + p @ vh[s0 : s0 + block_kv]
                m = mn
            out[b, h] = o / l[:, None]
    return out


# ---------------------------------------------------------------------------
# Rotary embedding and the decoder block (composition of the above)
# ---------------------------------------------------------------------------


def rotate_half(x: np.ndarray) -> np.ndarray:
    """``cat(-x[..., d/2:], x[..., :d/2])`` — the slice/neg/cat index maps the
    tracer records for RoPE (tests/compiler/fixtures/tinyllama_layer0.json)."""
    d = x.shape[-1]
    return np.concatenate([-x[..., d // 2 :], x[..., : d // 2]], axis=-1)


def rope(x: np.ndarray, cos: np.ndarray, sin: np.ndarray) -> np.ndarray:
    """``x * cos + rotate_half(x) * sin`` with ``cos/sin`` broadcast over heads."""
    x = np.asarray(x, dtype=np.float64)
    return x * cos + rotate_half(x) * sin


def qwen3_block(x, cos, sin, w: dict, *, q_heads: int, kv_heads: int, head_dim: int, eps: float) -> np.ndarray:
    """One pre-norm decoder block: RMSNorm → q/k/v projections → per-head q/k
    RMSNorm → RoPE → causal GQA attention → o_proj + residual → RMSNorm →
    SiLU(gate)·up → down + residual.  ``x`` is ``[B, S, hidden]``; ``cos``/``sin``
    ``[B, S, head_dim]``; ``w`` maps the usual parameter names to arrays."""
    x = np.asarray(x, dtype=np.float64)
    B, S, _ = x.shape
    h = rms_norm(x, w["input_layernorm"], eps)
    q = linear(h, w["q_proj"]).reshape(B, S, q_heads, head_dim)
    k = linear(h, w["k_proj"]).reshape(B, S, kv_heads, head_dim)
    v = linear(h, w["v_proj"]).reshape(B, S, kv_heads, head_dim)
    q = rms_norm(q, w["q_norm"], eps).transpose(0, 2, 1, 3)
    k = rms_norm(k, w["k_norm"], eps).transpose(0, 2, 1, 3)
    v = v.transpose(0, 2, 1, 3)
    c, s = np.asarray(cos, dtype=np.float64)[:, None], np.asarray(sin, dtype=np.float64)[:, None]
    q, k = rope(q, c, s), rope(k, c, s)
    a = sdpa(q, k, v, is_causal=True, scale=1.0 / np.sqrt(head_dim))
    a = a.transpose(0, 2, 1, 3).reshape(B, S, q_heads * head_dim)
    x = x + linear(a, w["o_proj"])
    h = rms_norm(x, w["post_attention_layernorm"], eps)
    mlp = linear(silu(linear(h, w["gate_proj"])) * linear(h, w["up_proj"]), w["down_proj"])
    return x + mlp
