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


class _MatMul(nn.Module):
    def forward(self, a, b):
        return a @ b


class _MatMulT(nn.Module):
    def forward(self, a, b):
        return a @ b.transpose(-1, -2)


class _Attention(nn.Module):
    def __init__(self, causal: bool, gqa: bool, scale):
        super().__init__()
        self.kw = dict(is_causal=causal, enable_gqa=gqa, scale=scale)

    def forward(self, q, k, v, mask=None):
        return F.scaled_dot_product_attention(q, k, v, attn_mask=mask, **self.kw)


class _BiasLinear(nn.Module):
    def __init__(self, k: int, n: int, bias: bool, residual: bool):
        super().__init__()
        self.lin, self.residual = nn.Linear(k, n, bias=bias), residual

    def forward(self, x, r):
        y = self.lin(x)
        return y + r if self.residual else y


def _wide_case(kind: str, rnd: random.Random, seed: int):
    """``(name, module, inputs, 16-bit?)`` for the families whose reference is the module in float64."""
    torch.manual_seed(seed)
    if kind == "matmul":
        dt = rnd.choice([torch.float32, torch.float32, torch.bfloat16])
        lead = rnd.choice([(), (rnd.randint(1, 5),), (2, rnd.randint(1, 3))])
        m, k, n = rnd.choice([rnd.randint(1, 70), rnd.randint(1, 300), 128]), rnd.choice([rnd.randint(1, 40) * 8, rnd.randint(1, 300), 1024]), rnd.choice([rnd.randint(1, 60) * 4, rnd.randint(1, 200), 256])
        transposed = rnd.random() < 0.4
        shared = rnd.random() < 0.5 or not lead
        b_shape = ((n, k) if transposed else (k, n)) if shared else (*lead, *((n, k) if transposed else (k, n)))
        a, b = torch.randn(*lead, m, k).to(dt), (0.3 * torch.randn(*b_shape)).to(dt)
        return f"matmul {tuple(a.shape)} @ {tuple(b.shape)}{'^T' if transposed else ''} {dt}", (_MatMulT() if transposed else _MatMul()).eval(), (a, b), dt is not torch.float32
    if kind == "attention32":
        hkv, group = rnd.choice([1, 2, 3]), rnd.choice([1, 2, 4])
        sq = rnd.choice([rnd.randint(1, 40), rnd.randint(1, 200), 128])
        causal = rnd.random() < 0.4
        skv = sq if causal or rnd.random() < 0.5 else rnd.randint(1, 250)
        d, dv = rnd.choice([16, 32, 40, 64, 128]), None
        b = rnd.choice([1, 2])
        q, k, v = torch.randn(b, hkv * group, sq, d), torch.randn(b, hkv, skv, d), torch.randn(b, hkv, skv, d)
        mask = None
        if not causal and rnd.random() < 0.5:
            mask = torch.randn(*rnd.choice([(sq, skv), (1, 1, sq, skv), (b, 1, 1, skv), (b, hkv * group, sq, skv)]))
        scale = rnd.choice([None, None, 0.25])
        return f"attention fp32 {hkv * group}/{hkv} heads {sq}x{skv} d={d} causal={causal} mask={None if mask is None else tuple(mask.shape)}", _Attention(causal, group > 1, scale).eval(), (q, k, v) + ((mask,) if mask is not None else ()), False
    # fp32 linear (+ bias, + residual): the underfilled-launch split and the exact-round tiles
    m = rnd.choice([rnd.randint(17, 200), 32, 128, 512])
    k, n = rnd.choice([256, 512, 1024, 2048, 3072, 96, 160]), rnd.choice([rnd.randint(1, 64) * 8, 256, 1024, 3072])
    bias, residual = rnd.random() < 0.5, rnd.random() < 0.5
    mod = _BiasLinear(k, n, bias, residual)
    with torch.no_grad():
        for p in mod.parameters():
            p.copy_(0.05 * torch.randn_like(p))
    return f"linear fp32 {m}x{k}x{n} bias={bias} residual={residual}", mod.eval(), (torch.randn(m, k), torch.randn(m, n)), False


@pytest.mark.parametrize("kind", ["matmul", "attention32", "linear32"])
def test_seeded_random_shapes_against_float64(device, kind):
    """Families that reach the batched contraction, the layout-change copy, zero-padded ragged extents, the
    fp32 streaming attention kernel and the fp32 tier's split of an underfilled launch: against the module in float64
    (fp32: 1e-4 of the output's RMS; 16-bit: rtol 2e-2)."""
    import copy

    rnd = random.Random(f"emmy-wide-{kind}")
    be = HipBackend()
    for i in range(14):
        name, mod, inputs, half = _wide_case(kind, rnd, seed=2000 + i)
        print(f"{kind} #{i}: {name}", flush=True)  # names the case should the device fault
        compiled = be.compile(trace_module(mod, inputs))
        prog = be.program(compiled, {n: t.to(device) for n, t in zip(compiled.inputs, inputs)})
        try:
            prog.run()
            torch.cuda.synchronize()
            ours = prog.output_tensors()[compiled.outputs[0]].clone().cpu()
        finally:
            prog.close()
        with torch.no_grad():
            want = copy.deepcopy(mod).double()(*(t.double() for t in inputs)).float()
        rms = float(want.pow(2).mean().sqrt())
        rtol, atol = (2e-2, 2e-2 * max(rms, 1.0)) if half else (1e-4, 1e-4 * max(rms, 1e-3))
        eager.assert_close(ours.reshape(want.shape).float(), want, rtol, atol, f"{kind} #{i} {name}")
