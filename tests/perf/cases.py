"""The kernel-level perf cases of the reference's suite (tests/perf/cases.py:35-232), re-derived for this backend.

One case per fused launch of a Qwen3-Embedding-0.6B decoder layer (hidden 1024, intermediate 3072, 16 query heads,
8 KV heads, head_dim 128) at 32 / 128 / 512 tokens, each an inline expression in the ``run -c`` grammar whose tensors
are all run-time fp32 inputs — the only precision the reference compiles.  Case names are the reference's, so two
result files can be joined on them.
"""

from __future__ import annotations

import os
from dataclasses import dataclass

HIDDEN, INTERMEDIATE, HEADS, KV_HEADS, HEAD_DIM = 1024, 3072, 16, 8, 128
SEQ_LENS = (32, 128, 512)
TAG = "qwen3emb"
HEAVY_ELEMENTS = 50_000_000  # input elements above which a case runs 20 timed iterations instead of 100 (cases.py:80-85)


@dataclass(frozen=True)
class Case:
    name: str
    op: str  # matmul | rmsnorm | sdpa | matmul_add | gated_mlp
    shapes: tuple[tuple[int, ...], ...]
    dtype: str = "fp32"

    @property
    def shape_str(self) -> str:
        return " x ".join("(" + ",".join(map(str, s)) + ")" for s in self.shapes)

    @property
    def code(self) -> str:
        s = self.shapes
        kw = "" if self.dtype == "fp32" else f", dtype=torch.{TORCH_DTYPE[self.dtype]}"
        rand = [f"torch.randn({tuple(x)}{kw})" for x in s]
        if self.op == "matmul":
            return f"a={rand[0]}; b={rand[1]}; torch.matmul(a,b)"
        if self.op == "rmsnorm":
            return f"x={rand[0]}; w={rand[1]}; F.rms_norm(x, {tuple(s[1])}, w, eps=1e-6)"
        if self.op == "sdpa":
            return f"q={rand[0]}; k={rand[1]}; v={rand[2]}; F.scaled_dot_product_attention(q, k, v, is_causal=True, enable_gqa={s[0][-3] != s[1][-3]})"
        if self.op == "matmul_add":
            return f"x={rand[0]}; w={rand[1]}; r={rand[2]}; torch.matmul(x,w)+r"
        if self.op == "gated_mlp":
            return f"x={rand[0]}; wg={rand[1]}; wu={rand[2]}; F.silu(torch.matmul(x,wg))*torch.matmul(x,wu)"
        raise ValueError(self.op)

    @property
    def iters(self) -> int:
        total = 0
        for s in self.shapes:
            n = 1
            for d in s:
                n *= d
            total += n
        return 20 if total > HEAVY_ELEMENTS else 100


TORCH_DTYPE = {"fp32": "float32", "bf16": "bfloat16", "fp16": "float16"}


def _cases(dtype: str = "fp32") -> list[Case]:
    if dtype not in TORCH_DTYPE:
        raise ValueError(f"EMMY_PERF_DTYPE: expected one of {sorted(TORCH_DTYPE)}, got {dtype!r}")
    out: list[Case] = []
    q_dim, kv_dim = HEADS * HEAD_DIM, KV_HEADS * HEAD_DIM
    for s in SEQ_LENS:  # input / post-attention layer norm
        out.append(Case(f"rmsnorm.{TAG}.layer.s{s}", "rmsnorm", ((1, s, HIDDEN), (HIDDEN,))))
    for s in SEQ_LENS:  # per-head q / k norm
        for tag, heads in (("q_norm", HEADS), ("k_norm", KV_HEADS)):
            out.append(Case(f"rmsnorm.{TAG}.{tag}.s{s}", "rmsnorm", ((1, heads, s, HEAD_DIM), (HEAD_DIM,))))
    for s in SEQ_LENS:  # q and k / v projections
        for proj, n in (("q_proj", q_dim), ("kv_proj", kv_dim)):
            out.append(Case(f"matmul.{TAG}.{proj}.s{s}", "matmul", ((1, s, HIDDEN), (HIDDEN, n))))
    for s in SEQ_LENS:
        out.append(Case(f"sdpa.{TAG}.s{s}", "sdpa", ((1, HEADS, s, HEAD_DIM), (1, KV_HEADS, s, HEAD_DIM), (1, KV_HEADS, s, HEAD_DIM))))
    for s in SEQ_LENS:  # o_proj / down_proj with the residual add
        for proj, k in (("o_proj", q_dim), ("down_proj", INTERMEDIATE)):
            out.append(Case(f"matmul_add.{TAG}.{proj}.s{s}", "matmul_add", ((1, s, k), (k, HIDDEN), (1, s, HIDDEN))))
    for s in SEQ_LENS:
        out.append(Case(f"gated_mlp.{TAG}.s{s}", "gated_mlp", ((1, s, HIDDEN), (HIDDEN, INTERMEDIATE), (HIDDEN, INTERMEDIATE))))
    return [Case(c.name, c.op, c.shapes, dtype) for c in out]


# The reference runs fp32 only and keeps ``dtype`` "so an FP16 column can be added later" (cases.py:20-23); here
# ``EMMY_PERF_DTYPE=bf16`` (or ``fp16``) runs the same cases on this backend's 16-bit tier.
CASES = _cases(os.environ.get("EMMY_PERF_DTYPE", "fp32"))
