"""Cross-workgroup splits of a reduction axis beyond the contraction's: ``REDUCE=g<n>k`` on rows that reduce to one value
(partial row kernel + combine row kernel) and on attention (key slices leave ``(m, l, O)`` in a workspace, a combine
kernel merges them) — the carriers of the reference's cross-CTA finalize matrix
(tests/compiler/e2e/test_reduce_coverage.py:280-345)."""

from __future__ import annotations

import pytest
import torch
from torch import nn

from deplodock_amd import HipBackend, trace_module
from deplodock_amd.ir.hip import HipOp
from oracle import eager


class _Sum(nn.Module):
    def forward(self, x):
        return x.sum(-1)


class _Mean(nn.Module):
    def forward(self, x):
        return x.mean(-1)


class _Amax(nn.Module):
    def forward(self, x):
        return x.amax(-1)


class _L2(nn.Module):
    def forward(self, x):
        return torch.linalg.vector_norm(x, dim=-1)


def _kernels(compiled):
    return [n.op for n in compiled.nodes.values() if isinstance(n.op, HipOp)]


def _decode_case(q_len, kv_len, hq=16, hkv=8, d=128, causal=False, seed=7, batch=1):
    torch.manual_seed(seed)
    q = torch.randn(batch, hq, q_len, d).bfloat16()
    k = torch.randn(batch, hkv, kv_len, d).bfloat16()
    v = torch.randn(batch, hkv, kv_len, d).bfloat16()
    return eager.Case(f"decode_{q_len}x{kv_len}", eager.Sdpa(causal).eval(), (q, k, v), 2e-2, 2e-2)


# -- host side --------------------------------------------------------------------------------------------------


def test_row_split_is_a_partial_and_a_combine_row_kernel(launcher_lib, monkeypatch):
    monkeypatch.setenv("EMMY_REDUCE", "g4k")
    compiled = HipBackend().compile(trace_module(_Mean().eval(), (torch.randn(8, 4096),)))
    part, comb = sorted(_kernels(compiled), key=lambda k: "combine" in k.kernel_name)
    assert "partial" in part.kernel_name and "combine" in comb.kernel_name and part.knobs["REDUCE"].startswith("g4k") and comb.knobs["REDUCE"].startswith("g4k")
    ws = next(n for n in compiled.nodes.values() if n.op is part)
    assert tuple(ws.output.shape) == (8, 4) and ws.output.dtype.name == "f32"  # one bare statistic per (row, slice)
    assert "0x1.0000000000000p+12f" in comb.kernel_source and "p+12f" not in part.kernel_source  # the projection (1 / 4096 columns) is applied once, by the combine
    # the atomic arm has no form for a projected row: it is taken as the kernel arm, and says so in the stamped knob
    monkeypatch.setenv("EMMY_REDUCE", "g2a")
    compiled = HipBackend().compile(trace_module(_Sum().eval(), (torch.randn(8, 4096),)))
    assert all(k.knobs["REDUCE"].startswith("g2k") for k in _kernels(compiled)) and len(_kernels(compiled)) == 2
    # rows that write a row back, and column counts that do not split into whole chunks, keep the unsplit kernel
    monkeypatch.setenv("EMMY_REDUCE", "g4k")
    assert len(_kernels(HipBackend().compile(trace_module(nn.Softmax(-1).eval(), (torch.randn(8, 4096),))))) == 1
    assert len(_kernels(HipBackend().compile(trace_module(_Sum().eval(), (torch.randn(8, 4090),))))) == 1


def test_attention_key_split_is_a_partial_and_a_combine_kernel(launcher_lib, monkeypatch):
    monkeypatch.setenv("EMMY_REDUCE", "g4k")
    case = _decode_case(16, 1024)
    compiled = HipBackend().compile(trace_module(case.module, case.inputs))
    part, comb = sorted(_kernels(compiled), key=lambda k: "combine" in k.kernel_name)
    assert part.knobs["REDUCE"] == "g4k" and part.grid[1] == (4,) and "#define KV_CTAS 4" in part.kernel_source and "#define KV_CHUNK 256" in part.kernel_source
    ws = next(n for n in compiled.nodes.values() if n.op is part)
    assert tuple(ws.output.shape) == (4, 1, 16, 16, 132) and ws.output.dtype.name == "f32"
    assert comb.arg_order[0] == ws.id and "exp2f" in comb.kernel_source
    # the atomic spelling is the kernel arm here (the carrier's rescale is not an addition)
    monkeypatch.setenv("EMMY_REDUCE", "g2a")
    assert [k.knobs.get("REDUCE") for k in _kernels(HipBackend().compile(trace_module(case.module, case.inputs)))] == ["g2k", "g2k"]


def test_decode_sized_queries_over_a_long_cache_split_their_keys_by_default(launcher_lib):
    """16 heads x 1 query block cover 16 of 256 CUs: the keys are split until the launch covers the machine."""
    case = _decode_case(1, 32768)
    compiled = HipBackend().compile(trace_module(case.module, case.inputs))
    part = next(k for k in _kernels(compiled) if "partial" in k.kernel_name)
    assert part.knobs["REDUCE"] == "g16k" and part.grid[1] == (16,)
    # a prefill-size problem keeps the single kernel
    case = eager.sdpa_case()
    assert len(_kernels(HipBackend().compile(trace_module(case.module, case.inputs)))) == 1


# -- GPU parity ---------------------------------------------------------------------------------------------------


def _run(case, device):
    be = HipBackend()
    compiled = be.compile(trace_module(case.module, case.inputs))
    prog = be.program(compiled, {n: t.to(device) for n, t in zip(compiled.inputs, case.inputs)})
    try:
        prog.run()
        torch.cuda.synchronize()
        ours = prog.output_tensors()[compiled.outputs[0]].clone()
    finally:
        prog.close()
    want = eager.run_eager(case, device)
    return ours.reshape(want.shape), want, compiled


@pytest.mark.gpu
@pytest.mark.parametrize("pin", ["g2k", "g4k", "g8k"])
@pytest.mark.parametrize("mod,dtype", [(_Sum, torch.float32), (_Mean, torch.float32), (_Amax, torch.float32), (_L2, torch.float32), (_Mean, torch.bfloat16)])
def test_row_split_matches_eager(device, pin, mod, dtype, monkeypatch):
    monkeypatch.setenv("EMMY_REDUCE", pin)
    torch.manual_seed(5)
    x = torch.randn(37, 8192).to(dtype)
    case = eager.Case("rows", mod().eval(), (x,), 1e-5 if dtype is torch.float32 else 2e-2, 1e-5 if dtype is torch.float32 else 2e-2)
    ours, want, compiled = _run(case, device)
    split = [k for k in _kernels(compiled) if "partial" in k.kernel_name or "combine" in k.kernel_name]
    assert len(split) == 2 and all(k.knobs["REDUCE"].startswith(pin) for k in split)  # (the 2-norm has a map on either side of its row sum)
    if dtype is torch.float32:
        # Against the float64 result, on the scale the sum's terms set (signed terms cancel: the result can be far smaller
        # than what was added up): 8192 fp32 terms folded in any tree order stay within ~1e-7 of sum |x| per row.
        exact = mod()(x.double()).to(device)
        scale = {"_Sum": x.double().abs().sum(-1), "_Mean": x.double().abs().mean(-1), "_Amax": torch.zeros(37, dtype=torch.float64), "_L2": exact.cpu()}[mod.__name__].to(device)
        err = (ours.double() - exact).abs()
        assert bool((err <= 2e-7 * scale).all()), f"{mod.__name__} {pin}: worst error {float(err.max()):.3g} against scale {float(scale.max()):.3g}"
        assert bool(((want.double() - exact).abs() <= 2e-7 * scale).all())  # eager meets the same bound: the criterion is not vacuous for it
    else:
        eager.assert_close(ours, want, case.rtol, case.atol, f"{mod.__name__} {pin} vs eager")


@pytest.mark.gpu
@pytest.mark.parametrize("q_len,kv_len", [(1, 4096), (16, 4096), (1, 32768), (16, 32768), (5, 4000), (16, 2050)])
def test_attention_key_split_matches_eager_at_decode_sizes(device, q_len, kv_len):
    """Default schedule: these shapes split by themselves (ragged cache lengths included: the last slice is short)."""
    case = _decode_case(q_len, kv_len)
    ours, want, compiled = _run(case, device)
    assert any("partial" in k.kernel_name for k in _kernels(compiled))
    q, k, v = (t.to(device).float() for t in case.inputs)
    exact = nn.functional.scaled_dot_product_attention(q, k, v, enable_gqa=True)
    eager.assert_close(ours, exact, 2e-2, 2e-2, f"decode {q_len}x{kv_len} vs fp32 eager")
    eager.assert_rows_within_baseline(ours, want, exact, 1.5, f"decode {q_len}x{kv_len} rows")


@pytest.mark.gpu
@pytest.mark.parametrize("pin,flash", [("g2k", None), ("g4k", None), ("g3k", None), ("g4k", "w2/kv64/s2"), ("g2k", "w4/kv64/s1"), ("g8k", "w1/kv32/s4")])
def test_pinned_key_split_matches_eager_with_a_causal_mask_and_grouped_heads(device, pin, flash, monkeypatch):
    """A square causal problem split by a pin: slices beyond a query block's diagonal contribute nothing (their state is
    the identity of the merge), the slice that holds the diagonal masks it, position-coded values catch a misplaced slice."""
    monkeypatch.setenv("EMMY_REDUCE", pin)
    if flash:
        monkeypatch.setenv("EMMY_FLASH", flash)
    case = eager.sdpa_case(b=2, hq=8, hkv=2, s=1000, d=128, seed=13)
    ours, want, compiled = _run(case, device)
    part = next(k for k in _kernels(compiled) if "partial" in k.kernel_name)
    assert part.knobs["REDUCE"].startswith("g") and (flash is None or part.knobs["FLASH"] == flash)
    q, k, v = (t.to(device).float() for t in case.inputs)
    exact = nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True, enable_gqa=True)
    eager.assert_rows_within_baseline(ours, want, exact, 1.5, f"causal split {pin} rows")
    vpos = eager.position_coded_values(case.inputs[2])
    coded = eager.Case("pos", case.module, (case.inputs[0], case.inputs[1], vpos), 2e-2, 2e-2)
    op_, wp, _ = _run(coded, device)
    exact_p = nn.functional.scaled_dot_product_attention(q, k, vpos.to(device).float(), is_causal=True, enable_gqa=True)
    eager.assert_rows_within_baseline(op_, wp, exact_p, 1.5, f"causal split {pin} position-coded V")


@pytest.mark.gpu
def test_key_split_head_dim_64_and_fp16(device, monkeypatch):
    monkeypatch.setenv("EMMY_REDUCE", "g4k")
    torch.manual_seed(3)
    q, k, v = (torch.randn(2, h, s, 64).half() for h, s in ((4, 8), (2, 2048), (2, 2048)))
    case = eager.Case("d64", eager.Sdpa(False).eval(), (q, k, v), 2e-2, 2e-2)
    ours, want, compiled = _run(case, device)
    assert any("partial" in k.kernel_name for k in _kernels(compiled))
    eager.assert_close(ours, want, 2e-2, 2e-2, "split d=64 fp16 vs eager")
