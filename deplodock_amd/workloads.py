"""The benchmark configurations as workloads: ``nn.Module`` + seeded inputs + algorithmic work.

The five configurations the backend is measured on (RMSNorm, softmax, linear, causal GQA
attention, a Qwen3-0.6B-architecture decoder block) and their reduced-size relatives.  Inputs are
generated on the CPU from a seed, so every machine sees identical bits.  ``bench.py``, the
ahead-of-time build and the tests all take their shapes from here; comparing results against
PyTorch eager is the business of the test-side oracle, not of this module.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch
from torch import nn

FP32_RTOL = 1e-5
BF16_RTOL = 2e-2


@dataclass
class Case:
    name: str
    module: nn.Module
    inputs: tuple
    rtol: float
    atol: float
    algo_bytes: int = 0
    algo_flops: int = 0


class Sdpa(nn.Module):
    def __init__(self, causal: bool = True):
        super().__init__()
        self.causal = causal

    def forward(self, q, k, v):
        return nn.functional.scaled_dot_product_attention(q, k, v, is_causal=self.causal, enable_gqa=True)


class MaskedSdpa(nn.Module):
    """Attention with an explicit additive mask, the way a whole-model trace of a HuggingFace decoder reaches it:
    a float ``[1 | B, 1 | H, S, S_kv]`` bias of ``0`` / ``-inf`` (emmy/compiler/trace/torch.py:559-583)."""

    def forward(self, q, k, v, mask):
        return nn.functional.scaled_dot_product_attention(q, k, v, attn_mask=mask, enable_gqa=True)


def rms_norm_case(rows: int = 32, cols: int = 2048, seed: int = 0) -> Case:
    """C1: ``nn.RMSNorm(2048, eps=1e-6)`` on fp32 ``[1, rows, cols]`` ~N(0,1), weight ~N(1, 0.1)."""
    torch.manual_seed(seed)
    x = torch.randn(1, rows, cols)
    m = nn.RMSNorm(cols, eps=1e-6)
    with torch.no_grad():
        m.weight.copy_(1 + 0.1 * torch.randn(cols))
    return Case(f"rms_norm_{rows}x{cols}", m.eval(), (x,), FP32_RTOL, 1e-6, algo_bytes=(2 * rows * cols + cols) * 4)


def softmax_case(shape=(1, 28, 2048, 2048), seed: int = 0) -> Case:
    """C2: ``nn.Softmax(-1)`` on fp32 ~N(0, 2).  The absolute floor covers outputs
    near zero, where a pure relative bound is ill-posed."""
    torch.manual_seed(seed)
    x = 2 * torch.randn(*shape)
    return Case("softmax_" + "x".join(map(str, shape)), nn.Softmax(dim=-1).eval(), (x,), FP32_RTOL, 1e-9, algo_bytes=2 * x.numel() * 4)


def linear_case(m: int = 2048, k: int = 1024, n: int = 3072, seed: int = 0) -> Case:
    """C3: ``nn.Linear(k, n, bias=False)`` bf16, x ~N(0,1), W ~N(0, 0.02)."""
    torch.manual_seed(seed)
    x = torch.randn(m, k).bfloat16()
    lin = nn.Linear(k, n, bias=False)
    with torch.no_grad():
        lin.weight.copy_(0.02 * torch.randn(n, k))
    return Case(f"linear_{m}x{k}x{n}", lin.bfloat16().eval(), (x,), BF16_RTOL, 2e-2, algo_bytes=(m * k + n * k + m * n) * 2, algo_flops=2 * m * n * k)


def sdpa_case(b: int = 1, hq: int = 16, hkv: int = 8, s: int = 2048, d: int = 128, causal: bool = True, seed: int = 0, fp32: bool = False) -> Case:
    """C4: causal GQA attention, bf16 ~N(0,1), scale 1/sqrt(d); ``fp32``: the same values (rounded to bf16) held as fp32,
    the precision of the reference's ``sdpa`` perf cases (tests/perf/cases.py:174-190)."""
    torch.manual_seed(seed)
    q = torch.randn(b, hq, s, d).bfloat16()
    k = torch.randn(b, hkv, s, d).bfloat16()
    v = torch.randn(b, hkv, s, d).bfloat16()
    pairs = s * (s + 1) // 2 if causal else s * s
    if fp32:
        return Case(
            f"sdpa_fp32_{b}x{hq}x{hkv}x{s}x{d}", Sdpa(causal).eval(), (q.float(), k.float(), v.float()), 1e-4, 1e-5,
            algo_bytes=(2 * b * hq * s * d + 2 * b * hkv * s * d) * 4, algo_flops=4 * b * hq * d * pairs,
        )  # fmt: skip
    return Case(
        f"sdpa_{b}x{hq}x{hkv}x{s}x{d}", Sdpa(causal).eval(), (q, k, v), BF16_RTOL, 2e-2,
        algo_bytes=(2 * b * hq * s * d + 2 * b * hkv * s * d) * 2, algo_flops=4 * b * hq * d * pairs,
    )  # fmt: skip


def sdpa_decode_case(q_len: int = 1, kv_len: int = 32768, b: int = 1, hq: int = 16, hkv: int = 8, d: int = 128, seed: int = 0, fp32: bool = False) -> Case:
    """Decode-size attention over a long cache: ``q_len`` new queries see all ``kv_len`` keys (no mask); bound by the K/V
    stream (the algorithmic bytes are K, V, q and the output once).  ``fp32``: the same bf16-valued operands held as fp32."""
    torch.manual_seed(seed)
    q = torch.randn(b, hq, q_len, d).bfloat16()
    k = torch.randn(b, hkv, kv_len, d).bfloat16()
    v = torch.randn(b, hkv, kv_len, d).bfloat16()
    nb = 4 if fp32 else 2
    if fp32:
        q, k, v = q.float(), k.float(), v.float()
    return Case(
        f"sdpa_decode_{'fp32_' if fp32 else ''}{b}x{hq}x{hkv}x{q_len}x{kv_len}x{d}", Sdpa(False).eval(), (q, k, v), 1e-4 if fp32 else BF16_RTOL, 1e-5 if fp32 else 2e-2,
        algo_bytes=(2 * b * hq * q_len * d + 2 * b * hkv * kv_len * d) * nb, algo_flops=4 * b * hq * d * q_len * kv_len,
    )  # fmt: skip


class Qwen3Block(nn.Module):
    """Wraps ``transformers``' ``Qwen3DecoderLayer`` (built from a local config,
    no download) so it takes ``(x, cos, sin)`` and returns the hidden state."""

    def __init__(self, layer):
        super().__init__()
        self.l = layer

    def forward(self, x, cos, sin):
        out = self.l(x, position_embeddings=(cos, sin), attention_mask=None)
        return out[0] if isinstance(out, tuple) else out


class MaskedQwen3Block(nn.Module):
    """The same layer called the way a whole-model trace calls it: with the model's ``[1, 1, S, S]`` float causal
    bias as ``attention_mask``.  The layer then repeats the KV heads itself (unsqueeze / expand / reshape) and
    passes the bias to attention as an explicit mask instead of ``is_causal``."""

    def __init__(self, layer):
        super().__init__()
        self.l = layer

    def forward(self, x, cos, sin, mask):
        out = self.l(x, position_embeddings=(cos, sin), attention_mask=mask)
        return out[0] if isinstance(out, tuple) else out


def causal_bias(seq: int, dtype=torch.bfloat16) -> torch.Tensor:
    """``[1, 1, seq, seq]``: 0 where key <= query, ``-inf`` above the diagonal."""
    above = torch.arange(seq)[None, :] > torch.arange(seq)[:, None]
    return torch.zeros(1, 1, seq, seq).masked_fill(above, -float("inf")).to(dtype)


def masked_qwen3_block_case(seq: int = 512, seed: int = 0, norm_std: float = 0.0) -> Case:
    """:func:`qwen3_block_case` with the causal structure carried by an explicit mask operand."""
    base = qwen3_block_case(seq=seq, seed=seed, norm_std=norm_std)
    return Case(base.name + "_masked", MaskedQwen3Block(base.module.l).eval(), (*base.inputs, causal_bias(seq)), base.rtol, base.atol,
                algo_bytes=base.algo_bytes, algo_flops=base.algo_flops)  # fmt: skip


def qwen3_block_case(seq: int = 512, seed: int = 0, dtype=torch.bfloat16, norm_std: float = 0.0) -> Case:
    """C5: one Qwen3-0.6B-architecture decoder block, weights ~N(0, 0.02), norm
    weights 1 (``norm_std`` > 0: ~N(1, norm_std), so a norm weight paired with the
    wrong column shows), x ~N(0,1), positions 0..seq-1, RoPE theta 1e6."""
    from transformers import Qwen3Config
    from transformers.models.qwen3.modeling_qwen3 import Qwen3DecoderLayer, Qwen3RotaryEmbedding

    cfg = Qwen3Config(
        hidden_size=1024, num_attention_heads=16, num_key_value_heads=8, head_dim=128, intermediate_size=3072,
        rms_norm_eps=1e-6, rope_theta=1e6, num_hidden_layers=1, vocab_size=1024, max_position_embeddings=max(4096, seq),
    )  # fmt: skip
    cfg._attn_implementation = "sdpa"
    torch.manual_seed(seed)
    layer = Qwen3DecoderLayer(cfg, 0)
    with torch.no_grad():
        for name, p in layer.named_parameters():
            if "norm" in name:
                p.fill_(1.0)
                if norm_std:
                    p.add_(norm_std * torch.randn_like(p))
            else:
                p.copy_(0.02 * torch.randn_like(p))
    x = torch.randn(1, seq, 1024)
    cos, sin = Qwen3RotaryEmbedding(cfg)(x, torch.arange(seq)[None])
    h, hq, hkv, d, inter = 1024, 16, 8, 128, 3072
    flops = 2 * seq * h * (hq * d + 2 * hkv * d) + 2 * seq * hq * d * h + 3 * 2 * seq * h * inter + 4 * hq * d * (seq * (seq + 1) // 2)
    wbytes = (h * (hq * d + 2 * hkv * d) + hq * d * h + 3 * h * inter) * 2
    return Case(
        f"qwen3_block_s{seq}" + (f"_nw{norm_std}" if norm_std else ""), Qwen3Block(layer).to(dtype).eval(), (x.to(dtype), cos.to(dtype), sin.to(dtype)),
        BF16_RTOL if dtype is torch.bfloat16 else 1e-4, 4e-2 if dtype is torch.bfloat16 else 1e-4, algo_bytes=wbytes, algo_flops=flops,
    )  # fmt: skip


class LastHiddenState(nn.Module):
    """A ``transformers`` base model taking token ids and returning its last hidden state."""

    def __init__(self, model):
        super().__init__()
        self.m = model

    def forward(self, ids):
        return self.m(input_ids=ids).last_hidden_state


def qwen3_model_case(seq: int = 512, layers: int = 28, seed: int = 0, dtype=torch.bfloat16) -> Case:
    """The whole Qwen3-0.6B-architecture base model (what Qwen3-Embedding-0.6B runs before pooling: hidden 1024,
    16 query / 8 KV heads of 128, intermediate 3072, vocabulary 151 669), random weights scaled so activations keep
    unit size through ``layers`` layers, random token ids: ids in, last hidden state out."""
    from transformers import Qwen3Config, Qwen3Model

    cfg = Qwen3Config(
        hidden_size=1024, num_attention_heads=16, num_key_value_heads=8, head_dim=128, intermediate_size=3072, num_hidden_layers=layers, vocab_size=151669,
        rms_norm_eps=1e-6, rope_theta=1e6, max_position_embeddings=max(32768, seq), pad_token_id=0, eos_token_id=1, bos_token_id=2,
    )  # fmt: skip
    cfg._attn_implementation = "sdpa"
    torch.manual_seed(seed)
    model = Qwen3Model(cfg).eval()
    with torch.no_grad():
        for name, p in model.named_parameters():
            if "norm" not in name:
                p.mul_(0.5)
    ids = torch.randint(3, 151000, (1, seq))
    h, hq, hkv, d, inter = 1024, 16, 8, 128, 3072
    flops = layers * (2 * seq * h * (hq * d + 2 * hkv * d) + 2 * seq * hq * d * h + 3 * 2 * seq * h * inter + 4 * hq * d * (seq * (seq + 1) // 2))
    wbytes = layers * (h * (hq * d + 2 * hkv * d) + hq * d * h + 3 * h * inter) * 2
    return Case(f"qwen3_model_l{layers}_s{seq}", LastHiddenState(model).to(dtype).eval(), (ids,), BF16_RTOL, 4e-2, algo_bytes=wbytes, algo_flops=flops)


class NormedRopeAttention(nn.Module):
    """The front of a Qwen3-style attention layer with ``nn.RMSNorm`` head norms:
    q/k/v projections, per-head norm of q and k, rotary embedding, causal GQA
    attention.  Unlike the block case its norm weights are not all ones, so a
    kernel that pairs a column with the wrong weight or table row shows."""

    def __init__(self, hidden: int, q_heads: int, kv_heads: int, head_dim: int):
        super().__init__()
        self.hq, self.hkv, self.d = q_heads, kv_heads, head_dim
        self.q_proj = nn.Linear(hidden, q_heads * head_dim, bias=False)
        self.k_proj = nn.Linear(hidden, kv_heads * head_dim, bias=False)
        self.v_proj = nn.Linear(hidden, kv_heads * head_dim, bias=False)
        self.q_norm = nn.RMSNorm(head_dim, eps=1e-6)
        self.k_norm = nn.RMSNorm(head_dim, eps=1e-6)

    @staticmethod
    def _rotate_half(x):
        half = x.shape[-1] // 2
        return torch.cat((-x[..., half:], x[..., :half]), dim=-1)

    def forward(self, x, cos, sin):
        b, s, _ = x.shape
        q = self.q_norm(self.q_proj(x).view(b, s, self.hq, self.d)).transpose(1, 2)
        k = self.k_norm(self.k_proj(x).view(b, s, self.hkv, self.d)).transpose(1, 2)
        v = self.v_proj(x).view(b, s, self.hkv, self.d).transpose(1, 2)
        c, sn = cos.unsqueeze(1), sin.unsqueeze(1)
        q = q * c + self._rotate_half(q) * sn
        k = k * c + self._rotate_half(k) * sn
        o = nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True, enable_gqa=True)
        return o.transpose(1, 2).reshape(b, s, self.hq * self.d)


def normed_rope_attention_case(hidden: int = 256, q_heads: int = 4, kv_heads: int = 2, head_dim: int = 64, seq: int = 100, seed: int = 0) -> Case:
    """bf16; projection weights ~N(0, 0.05), norm weights ~N(1, 0.2), x ~N(0,1), rotary base 1e4."""
    torch.manual_seed(seed)
    m = NormedRopeAttention(hidden, q_heads, kv_heads, head_dim)
    with torch.no_grad():
        for name, p in m.named_parameters():
            p.copy_(1 + 0.2 * torch.randn_like(p) if "norm" in name else 0.05 * torch.randn_like(p))
    x = torch.randn(1, seq, hidden)
    ang = torch.arange(seq)[:, None] * (1e4 ** (-torch.arange(0, head_dim, 2) / head_dim))[None]
    emb = torch.cat((ang, ang), -1)
    return Case(
        f"normed_rope_attention_h{hidden}_{q_heads}x{kv_heads}x{head_dim}_s{seq}", m.to(torch.bfloat16).eval(),
        (x.to(torch.bfloat16), emb.cos()[None].to(torch.bfloat16), emb.sin()[None].to(torch.bfloat16)), BF16_RTOL, 2e-2,
    )  # fmt: skip


__all__ = ["Case", "FP32_RTOL", "BF16_RTOL", "Sdpa", "Qwen3Block", "NormedRopeAttention", "rms_norm_case", "softmax_case", "linear_case",
           "sdpa_case", "sdpa_decode_case", "qwen3_block_case", "normed_rope_attention_case"]  # fmt: skip
