"""Seeded random shapes through the heuristic schedule: every kernel family of the path, sizes that
do not fill tiles, token counts that coincide with head counts, reduction extents with a short last
slab, cross attention with a single query row.  Each case is checked against PyTorch eager on the
same module and inputs (fp32 rtol 1e-5, 16-bit rtol 2e-2)."""

from __future__ import annotations

import random

import pytest
import torch
import torch.nn.functional as F
from torch import nn

from deplodock_amd import HipBackend, trace_module
from oracle import eager
from oracle.eager import Case

pytestmark = pytest.mark.gpu


class GatedMlp(nn.Module):
    def __init__(self, hidden: int, inter: int, norm: bool):
        super().__init__()
        self.norm = nn.RMSNorm(hidden, eps=1e-6) if norm else None
        self.gate, self.up, self.down = nn.Linear(hidden, inter, bias=False), nn.Linear(hidden, inter, bias=False), nn.Linear(inter, hidden, bias=False)

    def forward(self, x):
        h = self.norm(x) if self.norm is not None else x
        y = self.down(F.silu(self.gate(h)) * self.up(h))
        return x + y if self.norm is not None else y


class NormLinear(nn.Module):
    def __init__(self, hidden: int, n: int, bias: bool):
        super().__init__()
        self.norm, self.lin = nn.RMSNorm(hidden, eps=1e-5), nn.Linear(hidden, n, bias=bias)

    def forward(self, x):
        return self.lin(self.norm(x))


class CrossAttention(nn.Module):
    def forward(self, q, k, v):
        return F.scaled_dot_product_attention(q, k, v, enable_gqa=True)


def _init(m: nn.Module, dtype) -> nn.Module:
    with torch.no_grad():
        for p in m.parameters():
            p.copy_(0.03 * torch.randn_like(p) if p.dim() > 1 else 1 + 0.1 * torch.randn_like(p))
    return m.to(dtype).eval()


def _case(kind: str, rnd: random.Random, seed: int) -> Case:
    torch.manual_seed(seed)
    dt = rnd.choice([torch.bfloat16, torch.bfloat16, torch.float16])
    rows = rnd.choice([rnd.randint(1, 40), rnd.randint(1, 600), rnd.choice([64, 128, 256, 512])])
    if kind == "linear":
        k = rnd.choice([64, 128, 256, 512, 1024, 2048, 96, 160, 72, 200])
        n = rnd.choice([rnd.randint(1, 260) * 8, rnd.choice([1024, 3072, 4096, 96, 192])])
        return eager.linear_case(m=rows, k=k, n=n, seed=seed)
    if kind == "sdpa":
        hkv, group = rnd.choice([1, 2, 4, 8]), rnd.choice([1, 2, 4])
        s = rnd.choice([rnd.randint(1, 64), rnd.randint(1, 700), rnd.choice([128, 256, 512, 1024])])
        return eager.sdpa_case(b=rnd.choice([1, 2, 3]), hq=hkv * group, hkv=hkv, s=s, d=rnd.choice([64, 128]), causal=rnd.random() < 0.6, seed=seed)
    if kind == "cross":
        hkv, group, d = rnd.choice([1, 2, 4]), rnd.choice([1, 2, 4]), rnd.choice([64, 128])
        sq, skv = rnd.choice([1, 1, rnd.randint(1, 300)]), rnd.randint(1, 900)
        q, k, v = torch.randn(2, hkv * group, sq, d).to(dt), torch.randn(2, hkv, skv, d).to(dt), torch.randn(2, hkv, skv, d).to(dt)
        return Case(f"cross {hkv * group}/{hkv} heads {sq}x{skv} d={d} {dt}", CrossAttention().eval(), (q, k, v), 2e-2, 2e-2)
    if kind == "softmax":
        shape = tuple(rnd.randint(1, 9) for _ in range(rnd.randint(1, 3))) + (rnd.choice([rnd.randint(1, 300), rnd.randint(1, 5000), 2048, 16384]),)
        return eager.softmax_case(shape=shape, seed=seed)
    if kind == "rms":
        return eager.rms_norm_case(rows=rnd.randint(1, 300), cols=rnd.choice([rnd.randint(1, 600) * 4, 2048, 128, 8192]), seed=seed)
    if kind == "block":
        return eager.qwen3_block_case(seq=rnd.choice([rnd.randint(1, 40), rnd.randint(1, 400)]), seed=seed)
    if kind == "rope":
        qh = rnd.choice([2, 4, 8])
        kvh = rnd.choice([h for h in (1, 2, 4, 8) if qh % h == 0])
        return eager.normed_rope_attention_case(hidden=rnd.choice([256, 512, 1024]), q_heads=qh, kv_heads=kvh, head_dim=rnd.choice([64, 128]), seq=rnd.randint(1, 300), seed=seed)
    if kind == "mlp":
        hidden, inter, norm = rnd.choice([64, 128, 256, 512, 1024]), rnd.choice([96, 128, 256, 384, 1024, 3072, 200]), rnd.random() < 0.5
        return Case(f"mlp {hidden}->{inter} rows={rows} norm={norm} {dt}", _init(GatedMlp(hidden, inter, norm), dt), (torch.randn(1, rows, hidden).to(dt),), 2e-2, 4e-2)
    hidden, n, bias = rnd.choice([64, 128, 256, 512, 1024, 2048, 96]), rnd.choice([rnd.randint(1, 200) * 8, 1024, 3072]), rnd.random() < 0.5
    return Case(f"norm->linear {hidden}->{n} rows={rows} bias={bias} {dt}", _init(NormLinear(hidden, n, bias), dt), (torch.randn(rows, hidden).to(dt),), 2e-2, 4e-2)


@pytest.mark.parametrize("kind", ["linear", "sdpa", "cross", "softmax", "rms", "block", "rope", "mlp", "normlinear"])
def test_seeded_random_shapes(device, kind):
    rnd = random.Random(f"emmy-{kind}")
    be = HipBackend()
    for i in range(12):
        case = _case(kind, rnd, seed=1000 + i)
        print(f"{kind} #{i}: {case.name}", flush=True)  # names the case should the device fault
        compiled = be.compile(trace_module(case.module, case.inputs))
        prog = be.program(compiled, {n: t.to(device) for n, t in zip(compiled.inputs, case.inputs)})
        try:
            prog.run()
            torch.cuda.synchronize()
            ours = prog.output_tensors()[compiled.outputs[0]].clone()
        finally:
            prog.close()
        want = eager.run_eager(case, device)
        eager.assert_close(ours.reshape(want.shape), want, case.rtol, case.atol, f"{kind} #{i} {case.name}")
