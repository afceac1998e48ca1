"""Parity of the HIP path with the oracle (PyTorch eager on the same module and
seeded inputs), through the public backend API and therefore through the C-ABI
library.  Tolerances: fp32 rtol 1e-5 (plus a stated absolute floor), bf16 rtol
2e-2 with fp32 accumulation."""

from __future__ import annotations

import copy

import numpy as np
import pytest
import torch
from torch import nn

from deplodock_amd import HipBackend, trace_module
from deplodock_amd.backend.hip import program
from deplodock_amd.dtype import BF16, F32
from deplodock_amd.graph import Graph, Tensor
from deplodock_amd.ir import expr as E
from deplodock_amd.ir.hip import HipOp
from deplodock_amd.ir.schedule import ReducePlan
from deplodock_amd.ir.tile import RowReduce, Stat, TileOp
from deplodock_amd.passes.lower import lower
from oracle import eager
from oracle import emmy_ops as O

pytestmark = pytest.mark.gpu


def run_case(case, device, **env):
    """Trace → compile → run on the device; returns (our output tensor, eager-on-GPU output)."""
    be = HipBackend()
    compiled = be.compile(trace_module(case.module, case.inputs))
    names = compiled.inputs
    prog = be.program(compiled, {n: t.to(device) for n, t in zip(names, case.inputs)})
    try:
        prog.run()
        torch.cuda.synchronize()
        ours = prog.output_tensors()[compiled.outputs[0]].clone()
    finally:
        prog.close()
    want = eager.run_eager(case, device)
    return ours.reshape(want.shape), want, compiled


# -- C1 ---------------------------------------------------------------------------


@pytest.mark.parametrize("rows", [32, 32768])
def test_c1_rms_norm(device, rows):
    case = eager.rms_norm_case(rows=rows)
    ours, want, _ = run_case(case, device)
    eager.assert_close(ours, want, case.rtol, case.atol, "rms_norm vs eager (GPU)")
    if rows == 32:
        eager.assert_close(ours, eager.run_eager(case, "cpu"), case.rtol, case.atol, "rms_norm vs eager (CPU)")
    # size-independent property: rows of y / w have unit RMS
    w = case.module.weight.detach().to(device)
    rms = ((ours / w).double().pow(2).mean(-1)).sqrt()
    assert float((rms - 1).abs().max()) < 1e-5


@pytest.mark.parametrize("coop", ["b16", "b64", "b128", "b256", "b1024"])
def test_c1_every_cooperative_width(device, coop, monkeypatch):
    monkeypatch.setenv("EMMY_REDUCE", coop)
    case = eager.rms_norm_case(rows=37, cols=1024, seed=1)
    ours, want, compiled = run_case(case, device)
    assert [n.op.knobs["REDUCE"] for n in compiled.nodes.values() if isinstance(n.op, HipOp)] == [coop]
    eager.assert_close(ours, want, case.rtol, case.atol, f"rms_norm {coop}")


def test_reference_recipe_rms_sum_variant(device, golden):
    """``x * rsqrt(sum(x^2) + eps) * w`` — the graph the reference's own e2e tests build
    (tests/compiler/e2e/test_accuracy.py:184-212), as a hand-written tile."""
    x = E.Var("x")
    body = RowReduce(rows=8, cols=64, x="X", x_dtype=F32, out="out", out_dtype=F32, stats=(Stat("ss", "sum", x * x),),
                     project=x * E.Un("rsqrt", E.Var("ss") + 1e-6) * E.Var("w"), col_operands=(("w", F32),), reduce=ReducePlan(coop=16))  # fmt: skip
    g = Graph()
    g.add_input("X", (8, 64))
    g.add_input("w", (64,))
    g.add_node(TileOp(name="k_rms_sum", body=body), ["X", "w"], Tensor("out", (8, 64), F32))
    g.outputs = ["out"]
    res, _ = HipBackend().run(lower(g), input_data={"X": golden["rms_sum_x"], "w": golden["rms_sum_w"]})
    np.testing.assert_allclose(res.outputs["out"], golden["rms_sum_y"], rtol=1e-5, atol=1e-7)
    np.testing.assert_allclose(res.outputs["out"], O.rms_norm_sum(golden["rms_sum_x"], golden["rms_sum_w"], 1e-6), rtol=1e-5, atol=1e-7)


# -- C2 ---------------------------------------------------------------------------


def test_c2_softmax_full_size(device):
    case = eager.softmax_case()
    ours, want, _ = run_case(case, device)
    eager.assert_close(ours, want, case.rtol, case.atol, "softmax vs eager (GPU)")
    assert float((ours.double().sum(-1) - 1).abs().max()) < 1e-5  # rows sum to one
    sl = (0, 3, slice(100, 164))
    cpu = torch.softmax(case.inputs[0][sl], -1)
    eager.assert_close(ours[sl], cpu, case.rtol, case.atol, "softmax slice vs eager (CPU)")


@pytest.mark.parametrize("shape", [(4, 8), (4, 2048), (3, 5, 1000), (7, 7), (1, 2050), (130, 16384), (2, 3, 1)])
def test_c2_softmax_ragged_and_small(device, shape, golden):
    case = eager.softmax_case(shape=shape, seed=2)
    ours, want, _ = run_case(case, device)
    eager.assert_close(ours, want, case.rtol, case.atol, f"softmax {shape}")
    eager.assert_close(ours, torch.from_numpy(O.softmax(case.inputs[0].numpy())).float(), case.rtol, case.atol, f"softmax {shape} vs numpy restatement")


def test_c2_softmax_golden_and_extremes(device, golden):
    for key in ("4x8", "4x2048"):
        m = nn.Softmax(dim=-1)
        x = torch.from_numpy(golden[f"softmax_{key}_x"])
        ours, _, _ = run_case(eager.Case("g", m, (x,), 1e-5, 1e-9), device)
        np.testing.assert_allclose(ours.cpu().numpy(), golden[f"softmax_{key}_y"], rtol=1e-5, atol=1e-9)
    # large magnitudes and a fully dominated row stay finite and exact
    x = torch.tensor([[1e4, 1e4 - 1, -1e4, 0.0] * 16, [-80.0] * 63 + [80.0]], dtype=torch.float32)
    ours, want, _ = run_case(eager.Case("x", nn.Softmax(dim=-1), (x,), 1e-5, 1e-30), device)
    eager.assert_close(ours, want, 1e-5, 1e-30, "softmax extremes")


# -- C3 ---------------------------------------------------------------------------


@pytest.mark.parametrize("m", [1, 16, 128, 2048])
def test_c3_linear(device, m):
    case = eager.linear_case(m=m)
    ours, want, _ = run_case(case, device)
    eager.assert_close(ours, want, case.rtol, case.atol, f"linear M={m} vs eager (GPU)")
    # fp32-accumulated then rounded once: must sit within one bf16 ulp of the exact product
    x, w = case.inputs[0][: min(m, 8)].double(), case.module.weight.detach().double().cpu()
    exact = x @ w.T
    eager.assert_close(ours[: min(m, 8)], exact, 2 ** -7, 1e-3, f"linear M={m} vs float64")


@pytest.mark.parametrize("waves", [None, 8, 4, 2, 1])
@pytest.mark.parametrize("m,k,n", [(1, 1024, 3072), (16, 1024, 3072), (5, 512, 1960), (13, 3072, 1024), (16, 2048, 24), (3, 16384, 256), (2, 32, 40), (16, 8192, 64), (32, 1024, 3072), (24, 2048, 1000), (47, 1024, 520), (64, 512, 264)])
def test_few_row_linear_k_split_over_waves(device, m, k, n, waves, monkeypatch):
    """A few rows (up to four 16-row MFMA tiles): the reduction axis is split over the waves of a workgroup, every
    weight fragment is requested at once, the activation rows go through LDS where they fit (two rows of 16384 do,
    16 of 8192 do not), long reduction extents loop over 16-step groups, and a column count that is no multiple of 16
    re-reads the last row without storing it.  By default up to 48 rows of at most 96 KiB together take the form (more
    than 16 rows only up to a reduction extent of 1024)."""
    if waves is not None:
        monkeypatch.setenv("EMMY_STAGE", f"d{waves}/ks")
    case = eager.linear_case(m=m, k=k, n=n, seed=m + k)
    ours, want, compiled = run_case(case, device)
    op = next(n_.op for n_ in compiled.nodes.values() if isinstance(n_.op, HipOp))
    if waves is not None or (m <= 48 and m * k * 2 <= 96 * 1024 and (m <= 16 or k <= 1024)):
        assert "/ks" in op.knobs["STAGE"], op.knobs  # a wave count that does not divide the extent degrades to the default one
    else:
        assert "/ks" not in op.knobs["STAGE"], op.knobs
    if waves is not None and k % (32 * waves) == 0:
        assert op.knobs["STAGE"] == f"d{waves}/ks"
    eager.assert_close(ours, want, case.rtol, case.atol, f"few-row linear {m}x{k}x{n} vs eager (GPU)")
    exact = case.inputs[0].double() @ case.module.weight.detach().double().cpu().T
    eager.assert_close(ours, exact, 2 ** -7, 2e-3, f"few-row linear {m}x{k}x{n} vs float64")


@pytest.mark.parametrize("m,k,n", [(17, 512, 200), (40, 1024, 1000), (70, 256, 136), (130, 2048, 1024), (260, 512, 96), (300, 1024, 4096), (1024, 1024, 3072), (2048, 512, 4096),
                                   (30, 72, 192), (64, 200, 712), (4, 200, 4096), (300, 1000, 512), (128, 40, 64)])  # the last five: K is not a multiple of the MFMA depth
def test_linear_heuristic_tiles_on_ragged_and_one_round_shapes(device, m, k, n):
    """What the tile picker chooses by itself — small multi-wave tiles with direct-to-LDS rings below 512 rows,
    the largest tile that makes one workgroup per CU above — with rows and columns that do not fill the tiles,
    and with a reduction extent whose last slab is short (zero-filled on its way through registers)."""
    case = eager.linear_case(m=m, k=k, n=n, seed=m)
    ours, want, compiled = run_case(case, device)
    eager.assert_close(ours, want, case.rtol, case.atol, f"linear {m}x{k}x{n} vs eager (GPU)")
    exact = case.inputs[0].double() @ case.module.weight.detach().double().cpu().T
    eager.assert_close(ours, exact, 2 ** -7, 1e-3, f"linear {m}x{k}x{n} vs float64")


@pytest.mark.parametrize(
    "tile,stage",
    [
        ("a:mfma_32x32x16_bf16/w2x2/f2x3/k4", "d2/sync"),
        ("a:mfma_32x32x16_bf16/w2x2/f2x3/k4", "d3/dl"),
        ("a:mfma_32x32x16_bf16/w2x2/f2x3/k2", "d4/dl"),
        ("a:mfma_16x16x32_bf16/w4x2/f2x6/k2", "d2/sync"),
        ("a:mfma_16x16x32_bf16/w2x2/f2x2/k2", "d2/dl"),
        ("a:mfma_32x32x16_bf16/w1x4/f2x1/k2", "d2/sync"),
    ],
)
@pytest.mark.parametrize("shape", [(2048, 1024, 3072), (200, 128, 388), (129, 256, 72)])
def test_c3_linear_every_tier(device, tile, stage, shape, monkeypatch):
    monkeypatch.setenv("EMMY_TILE", tile)
    monkeypatch.setenv("EMMY_STAGE", stage)
    m, k, n = shape
    case = eager.linear_case(m=m, k=k, n=n, seed=4)
    ours, want, compiled = run_case(case, device)
    knobs = [n_.op.knobs for n_ in compiled.nodes.values() if isinstance(n_.op, HipOp)][0]
    assert knobs["TILE"] == tile
    eager.assert_close(ours, want, case.rtol, case.atol, f"linear {shape} {tile} {stage}")


def test_c3_golden(device, golden):
    case = eager.linear_case(32, 128, 96)
    ours, _, _ = run_case(case, device)
    want = torch.from_numpy(golden["c3_y_bits"].view(np.int16).copy()).view(torch.bfloat16).float()
    eager.assert_close(ours, want, 2e-2, 2e-2, "linear golden")


@pytest.mark.parametrize("cols", [4, 8, 12, 16])
@pytest.mark.parametrize("m,k,n", [(1, 1024, 3072), (16, 3072, 1032), (32, 1024, 1536), (40, 512, 24)])
def test_few_row_columns_per_workgroup(device, m, k, n, cols, monkeypatch):
    """4, 8, 12 or 16 output columns a workgroup: the spare weight rows of the MFMA tile request nothing and count as
    zeros, and only the workgroup's own columns are stored.  A column count that does not divide N is refused (the
    default form runs instead)."""
    monkeypatch.setenv("EMMY_STAGE", f"d8/ks/c{cols}" if cols != 16 else "d8/ks")
    case = eager.linear_case(m=m, k=k, n=n, seed=cols + m)
    ours, want, compiled = run_case(case, device)
    op = next(n_.op for n_ in compiled.nodes.values() if isinstance(n_.op, HipOp))
    if cols == 16 or n % cols == 0:
        assert op.knobs["STAGE"] == (f"d8/ks/c{cols}" if cols != 16 else "d8/ks") and op.grid[0] == (-(-n // cols),)
    eager.assert_close(ours, want, case.rtol, case.atol, f"few-row linear {m}x{k}x{n} c{cols} vs eager (GPU)")
    exact = case.inputs[0].double() @ case.module.weight.detach().double().cpu().T
    eager.assert_close(ours, exact, 2 ** -7, 2e-3, f"few-row linear {m}x{k}x{n} c{cols} vs float64")


class _GateUp(nn.Module):
    """``down(silu(gate(norm(x))) * up(norm(x)))`` without the down projection: a gate / up pair behind an RMSNorm."""

    def __init__(self, k, n):
        super().__init__()
        self.norm = nn.RMSNorm(k, eps=1e-6)
        self.gate = nn.Linear(k, n, bias=False)
        self.up = nn.Linear(k, n, bias=False)
        with torch.no_grad():
            self.norm.weight.copy_(1.0 + 0.1 * torch.randn(k))

    def forward(self, x):
        h = self.norm(x)
        return nn.functional.silu(self.gate(h)) * self.up(h)


@pytest.mark.parametrize("m,k,n", [(1, 1024, 3072), (16, 1024, 3072), (32, 1024, 768), (7, 512, 264)])
def test_few_row_gate_up_pair_behind_a_deferred_norm(device, m, k, n):
    """One launch: the norm's column weight is folded into both weight matrices, the row statistic is accumulated from
    the fragments each lane holds (lanes of a row through a butterfly, waves through LDS) and scales both accumulators
    before ``silu(gate) * up``."""
    torch.manual_seed(m + n)
    mod = _GateUp(k, n).bfloat16().eval()
    case = eager.Case("gate_up", mod, (torch.randn(m, k).bfloat16(),), 2e-2, 2e-2)
    ours, want, compiled = run_case(case, device)
    ops = [n_.op for n_ in compiled.nodes.values() if isinstance(n_.op, HipOp)]
    assert len(ops) == 1 and "/ks" in ops[0].knobs["STAGE"] and "silu" in ops[0].kernel_name, [o.knobs for o in ops]
    with torch.no_grad():
        exact = copy.deepcopy(mod).cpu().double()(case.inputs[0].cpu().double())
    eager.assert_close(ours, want, 2e-2, 2e-2, f"gate/up {m}x{k}x{n} vs eager")
    eager.assert_mean_error_within_baseline(ours, want, exact.float(), 1.5, f"gate/up {m}x{k}x{n} vs float64")


# -- C4 ---------------------------------------------------------------------------


def test_c4_sdpa_full_size(device):
    case = eager.sdpa_case()
    ours, want, _ = run_case(case, device)
    eager.assert_close(ours, want, case.rtol, case.atol, "sdpa vs eager (GPU)")
    q, k, v = (t.to(device).float() for t in case.inputs)
    exact = nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True, enable_gqa=True)
    eager.assert_close(ours, exact, case.rtol, case.atol, "sdpa vs fp32 eager")
    # Scale-aware: at S=2048 a late row is an average over ~2000 values and is only ~0.03 large, so the absolute
    # floor above is most of the value.  Per row, relative L2 error against the fp32 run, bounded by 1.5 x what
    # bf16 eager shows on the same inputs (worst row and mean).
    eager.assert_rows_within_baseline(ours, want, exact, 1.5, "sdpa S=2048 rows vs fp32 eager")
    # size-independent property: attention rows sum to one, so V = 1 gives O = 1
    ones = eager.Case("ones", case.module, (case.inputs[0], case.inputs[1], torch.ones_like(case.inputs[2])), 2e-2, 2e-2)
    o1, _, _ = run_case(ones, device)
    assert float((o1.float() - 1).abs().max()) <= 2 ** -7
    # V[j, :] = j / S: the output is each query's weighted mean key position; a key block that is skipped (it
    # drops out of numerator and denominator alike, which V = 1 cannot see) or fetched from the wrong place
    # shifts the row.  Same criterion, against fp32 eager on the same (bf16-valued) operands.
    vpos = eager.position_coded_values(case.inputs[2])
    coded = eager.Case("pos", case.module, (case.inputs[0], case.inputs[1], vpos), 2e-2, 2e-2)
    op, wp, _ = run_case(coded, device)
    exact_p = nn.functional.scaled_dot_product_attention(q, k, vpos.to(device).float(), is_causal=True, enable_gqa=True)
    eager.assert_rows_within_baseline(op, wp, exact_p, 1.5, "sdpa S=2048 position-coded V vs fp32 eager")


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("dims", [(1, 2, 1, 128, 128), (2, 4, 2, 200, 200), (1, 4, 4, 96, 160), (1, 6, 2, 33, 33), (1, 2, 2, 1, 70)])
def test_c4_sdpa_shapes_against_streaming_restatement(device, causal, dims):
    b, hq, hkv, sq, skv = dims
    torch.manual_seed(6)
    q = torch.randn(b, hq, sq, 128).bfloat16()
    k = torch.randn(b, hkv, skv, 128).bfloat16()
    v = torch.randn(b, hkv, skv, 128).bfloat16()
    case = eager.Case("s", eager.Sdpa(causal), (q, k, v), 2e-2, 2e-2)
    ours, want, _ = run_case(case, device)
    eager.assert_close(ours, want, 2e-2, 2e-2, f"sdpa {dims} causal={causal} vs eager")
    ref = O.flash_attention(q.float().numpy(), k.float().numpy(), v.float().numpy(), is_causal=causal, scale=128 ** -0.5, block_kv=64)
    eager.assert_close(ours, torch.from_numpy(ref).float(), 2e-2, 2e-2, f"sdpa {dims} causal={causal} vs streaming restatement")


@pytest.mark.parametrize("mask_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("dims,mask_shape", [
    ((1, 2, 1, 128, 128), (1, 1, 128, 128)), ((2, 4, 2, 200, 200), (2, 1, 200, 200)), ((2, 4, 2, 96, 160), (2, 4, 96, 160)),
    ((1, 6, 2, 33, 33), (1, 1, 33, 33)), ((2, 4, 4, 70, 300), (2, 1, 1, 300)), ((1, 2, 2, 1, 70), (1, 2, 1, 70)),
])  # fmt: skip
def test_c4_sdpa_with_an_additive_mask(device, dims, mask_shape, mask_dtype):
    """An explicit float mask (emmy/compiler/trace/torch.py:559-583) in every broadcast form, random finite
    biases with ``-inf`` holes: key 0 stays open so no row is empty.  Against eager with the same mask and against
    the streaming restatement in float64."""
    b, hq, hkv, sq, skv = dims
    torch.manual_seed(23)
    q, k, v = torch.randn(b, hq, sq, 128).bfloat16(), torch.randn(b, hkv, skv, 128).bfloat16(), torch.randn(b, hkv, skv, 128).bfloat16()
    mask = (2 * torch.randn(mask_shape)).to(mask_dtype)
    mask[torch.rand(mask_shape) < 0.3] = -float("inf")
    mask[..., 0] = 0.5
    case = eager.Case("masked", eager.MaskedSdpa().eval(), (q, k, v, mask), 2e-2, 2e-2)
    ours, want, compiled = run_case(case, device)
    assert len([n for n in compiled.nodes.values() if isinstance(n.op, HipOp)]) == 1
    eager.assert_close(ours, want, 2e-2, 2e-2, f"masked sdpa {dims} mask {mask_shape} {mask_dtype} vs eager")
    ref = O.flash_attention(q.float().numpy(), k.float().numpy(), v.float().numpy(), is_causal=False, scale=128 ** -0.5, block_kv=64, mask=mask.float().numpy())
    eager.assert_close(ours, torch.from_numpy(ref).float(), 2e-2, 2e-2, f"masked sdpa {dims} mask {mask_shape} vs streaming restatement")


@pytest.mark.parametrize("seq", [64, 200, 512])
def test_c5_block_called_with_an_attention_mask(device, seq):
    """The block as a whole-model trace reaches it (mask operand, KV heads repeated by the layer): against eager on
    the same call, and — the bias being the causal one — against the ``is_causal`` block's fp32 eager truth."""
    case = eager.masked_qwen3_block_case(seq=seq, norm_std=0.1)
    ours, want, compiled = run_case(case, device)
    assert len([n for n in compiled.nodes.values() if isinstance(n.op, HipOp)]) == 5
    plain = eager.qwen3_block_case(seq=seq, norm_std=0.1)
    exact = eager.run_eager_fp32(plain, device)
    eager.assert_mean_error_within_baseline(ours, want, exact, 1.5, f"masked block S={seq}")
    eager.assert_rows_within_baseline(ours, want, exact, 1.5, f"masked block S={seq} rows")


def test_c4_causal_bias_mask_equals_the_causal_kernel(device):
    """HuggingFace's ``[1, 1, S, S]`` ``0 / -inf`` causal bias, at the benchmark's size: the masked kernel's rows
    agree with the ``is_causal`` kernel's to the rounding of the output."""
    case = eager.sdpa_case()
    q, k, v = case.inputs
    s = q.shape[-2]
    tri = torch.zeros(1, 1, s, s).masked_fill(torch.arange(s)[None, :] > torch.arange(s)[:, None], -float("inf")).bfloat16()
    ours, want, _ = run_case(eager.Case("tri", eager.MaskedSdpa().eval(), (q, k, v, tri), 2e-2, 2e-2), device)
    causal, _, _ = run_case(case, device)
    eager.assert_close(ours, want, 2e-2, 2e-2, "bias-masked sdpa S=2048 vs eager")
    exact = nn.functional.scaled_dot_product_attention(q.to(device).float(), k.to(device).float(), v.to(device).float(), is_causal=True, enable_gqa=True)
    eager.assert_rows_within_baseline(ours, causal, exact, 1.5, "bias-masked sdpa vs the causal kernel, fp32 eager as the truth")


@pytest.mark.parametrize("d,dtype,causal", [(256, torch.bfloat16, True), (256, torch.bfloat16, False), (128, torch.float16, True), (64, torch.bfloat16, True), (64, torch.bfloat16, False), (64, torch.float16, True)])
def test_c4_wide_heads_and_fp16(device, d, dtype, causal):
    """head_dim 256 (two 128-wide accumulator groups; the schedule shrinks the key block to fit the LDS),
    head_dim 64 (128-byte K/V rows: two rows per bank line, their own swizzles) and fp16 operands."""
    torch.manual_seed(14)
    q, k, v = (torch.randn(2, h, 192, d).to(dtype) for h in (4, 2, 2))
    case = eager.Case("wide", eager.Sdpa(causal), (q, k, v), 2e-2, 2e-2)
    ours, want, _ = run_case(case, device)
    eager.assert_close(ours, want, 2e-2, 2e-2, f"sdpa d={d} {dtype} causal={causal} vs eager")
    exact = nn.functional.scaled_dot_product_attention(q.to(device).float(), k.to(device).float(), v.to(device).float(), is_causal=causal, enable_gqa=True)
    eager.assert_close(ours, exact, 2e-2, 2e-2, f"sdpa d={d} {dtype} causal={causal} vs fp32 eager")


@pytest.mark.parametrize("d,causal,dtype", [(40, True, torch.bfloat16), (80, True, torch.bfloat16), (96, False, torch.float16), (112, True, torch.bfloat16), (24, False, torch.bfloat16), (192, True, torch.bfloat16), (8, True, torch.float16)])
def test_c4_head_dims_between_the_kernels_widths_are_padded_not_decomposed(device, d, causal, dtype):
    """A 16-bit head_dim of whole 16-byte chunks that is not 64 / 128 / 256 runs on the flash kernel at the next width up:
    the missing columns of q count as zeros, k's and v's are never looked at, the output's are not stored.  Neighbouring
    memory is checked too: the output buffer is a window of a larger one whose other bytes must stay as they were."""
    torch.manual_seed(16)
    q, k, v = (torch.randn(2, h, 150, d).to(dtype) for h in (4, 2, 2))
    case = eager.Case("pad", eager.Sdpa(causal), (q, k, v), 2e-2, 2e-2)
    ours, want, compiled = run_case(case, device)
    ops = [n_.op for n_ in compiled.nodes.values() if isinstance(n_.op, HipOp)]
    assert len(ops) == 1 and f"#define DR {d}\n" in ops[0].kernel_source
    eager.assert_close(ours, want, 2e-2, 2e-2, f"sdpa d={d} {dtype} causal={causal} vs eager")
    exact = nn.functional.scaled_dot_product_attention(q.to(device).float(), k.to(device).float(), v.to(device).float(), is_causal=causal, enable_gqa=True)
    eager.assert_rows_within_baseline(ours, want, exact, 1.5, f"sdpa d={d} rows vs fp32 eager")
    # values placed so that a wrong column would show: v[..., j] = j
    vcol = torch.arange(d, dtype=torch.float32).expand_as(v).to(dtype)
    o2, w2, _ = run_case(eager.Case("cols", eager.Sdpa(causal), (q, k, vcol), 2e-2, 2e-2), device)
    eager.assert_close(o2, w2, 2e-2, 2e-2, f"sdpa d={d} column-coded V")


@pytest.mark.parametrize("pin", ["w4/kv64/s2", "w2/kv64/s1", "w1/kv64/s2", "w2/kv128/s2", "w2/kv64/s2/p"])
def test_c4_head_dim_64_workgroup_shapes(device, pin, monkeypatch):
    monkeypatch.setenv("EMMY_FLASH", pin)
    torch.manual_seed(15)
    q, k, v = (torch.randn(1, h, 512, 64).bfloat16() for h in (8, 2, 2))
    case = eager.Case("d64", eager.Sdpa(True), (q, k, v), 2e-2, 2e-2)
    ours, want, compiled = run_case(case, device)
    assert [n_.op.knobs["FLASH"] for n_ in compiled.nodes.values() if isinstance(n_.op, HipOp)] == [pin]
    eager.assert_close(ours, want, 2e-2, 2e-2, f"sdpa d=64 {pin} vs eager")


@pytest.mark.parametrize("pin", ["w4/kv64/s1", "w4/kv64/s2", "w2/kv64/s2", "w4/kv32/s2", "w1/kv32/s4", "w2/kv32/s4", "w8/kv64/s1", "w2/kv32/s4/ms", "w4/kv64/s2/ms"])
def test_c4_every_workgroup_shape(device, pin, monkeypatch):
    """Key-split groups, direct-to-LDS staging and the final (m, l, O) merge: the first
    key blocks are consumed right after they are staged, so every launch is checked."""
    monkeypatch.setenv("EMMY_FLASH", pin)
    case = eager.sdpa_case(b=1, hq=8, hkv=4, s=320, d=128, seed=9)
    be = HipBackend()
    compiled = be.compile(trace_module(case.module, case.inputs))
    assert [n.op.knobs["FLASH"] for n in compiled.nodes.values() if isinstance(n.op, HipOp)] == [pin]
    want = eager.run_eager(case, device)
    prog = be.program(compiled, {n: t.to(device) for n, t in zip(compiled.inputs, case.inputs)})
    try:
        out = prog.output_tensors()[compiled.outputs[0]]
        for rep in range(10):
            out.zero_()
            prog.run()
            torch.cuda.synchronize()
            eager.assert_close(out.reshape(want.shape), want, case.rtol, case.atol, f"sdpa {pin} launch {rep}")
    finally:
        prog.close()


@pytest.mark.parametrize("split", [2, 4, 8])
@pytest.mark.parametrize("d", [128, 64])
def test_c4_key_split_waves(device, split, d, monkeypatch):
    """``FLASH=w1/kv32/s<k>/pv``: one 32-row group per workgroup whose k waves take every k-th key block and stage for
    themselves, merged once at the close.  Causal and not, grouped heads, ragged lengths (a last query block that is
    partly empty, keys that end inside a block, fewer blocks than waves), unequal lengths, an additive mask with holes;
    ten launches of the first shape (the first blocks are consumed right after they land); against eager and the
    streaming restatement in float64."""
    monkeypatch.setenv("EMMY_FLASH", f"w1/kv32/s{split}/pv")
    torch.manual_seed(61)
    shapes = [(1, 8, 4, 320, 320, True), (2, 4, 2, 200, 200, True), (1, 4, 4, 96, 160, False), (1, 6, 2, 33, 33, True), (1, 2, 2, 1, 70, False), (1, 4, 2, 70, 45, True)]
    for n_case, (b, hq, hkv, sq, skv, causal) in enumerate(shapes):
        q, k, v = torch.randn(b, hq, sq, d).bfloat16(), torch.randn(b, hkv, skv, d).bfloat16(), torch.randn(b, hkv, skv, d).bfloat16()
        case = eager.Case("pv", eager.Sdpa(causal), (q, k, v), 2e-2, 2e-2)
        be = HipBackend()
        compiled = be.compile(trace_module(case.module, case.inputs))
        assert [n.op.knobs["FLASH"] for n in compiled.nodes.values() if isinstance(n.op, HipOp)] == [f"w1/kv32/s{split}/pv"]
        want = eager.run_eager(case, device)
        prog = be.program(compiled, {n: t.to(device) for n, t in zip(compiled.inputs, case.inputs)})
        try:
            out = prog.output_tensors()[compiled.outputs[0]]
            for rep in range(10 if n_case == 0 else 1):
                out.zero_()
                prog.run()
                torch.cuda.synchronize()
                eager.assert_close(out.reshape(want.shape), want, 2e-2, 2e-2, f"sdpa pv s{split} d={d} {(b, hq, hkv, sq, skv, causal)} launch {rep}")
            ref = O.flash_attention(q.float().numpy(), k.float().numpy(), v.float().numpy(), is_causal=causal, scale=d ** -0.5, block_kv=64)
            eager.assert_close(out.reshape(want.shape), torch.from_numpy(ref).float(), 2e-2, 2e-2, f"sdpa pv s{split} d={d} vs streaming restatement")
        finally:
            prog.close()
    q, k, v = torch.randn(2, 4, 70, d).bfloat16(), torch.randn(2, 2, 300, d).bfloat16(), torch.randn(2, 2, 300, d).bfloat16()
    mask = (2 * torch.randn(2, 1, 70, 300)).bfloat16()
    mask[torch.rand(2, 1, 70, 300) < 0.3] = -float("inf")
    mask[..., 0] = 0.5
    case = eager.Case("pv masked", eager.MaskedSdpa().eval(), (q, k, v, mask), 2e-2, 2e-2)
    ours, want, compiled = run_case(case, device)
    assert [n.op.knobs["FLASH"] for n in compiled.nodes.values() if isinstance(n.op, HipOp)] == [f"w1/kv32/s{split}/pv"]
    eager.assert_close(ours, want, 2e-2, 2e-2, f"masked sdpa pv s{split} d={d} vs eager")


@pytest.mark.parametrize("pin", ["w2/kv32/s4/p", "w1/kv64/s2/p", "w4/kv64/s2/p", "w2/kv64/s1/p", "w8/kv64/s1/p"])
def test_c4_mirrored_query_block_pairs(device, pin, monkeypatch):
    """A workgroup that takes query block b and then block n-1-b reuses its LDS and
    registers for the second block: both halves of every pair are checked, on repeated launches."""
    monkeypatch.setenv("EMMY_FLASH", pin)
    case = eager.sdpa_case(b=2, hq=4, hkv=2, s=512, d=128, seed=11)
    be = HipBackend()
    compiled = be.compile(trace_module(case.module, case.inputs))
    assert [n.op.knobs["FLASH"] for n in compiled.nodes.values() if isinstance(n.op, HipOp)] == [pin]
    want = eager.run_eager(case, device)
    prog = be.program(compiled, {n: t.to(device) for n, t in zip(compiled.inputs, case.inputs)})
    try:
        out = prog.output_tensors()[compiled.outputs[0]]
        for rep in range(5):
            out.zero_()
            prog.run()
            torch.cuda.synchronize()
            eager.assert_close(out.reshape(want.shape), want, case.rtol, case.atol, f"sdpa {pin} launch {rep}")
    finally:
        prog.close()


def test_c4_golden(device, golden):
    ours, _, _ = run_case(eager.sdpa_case(1, 4, 2, 96, 128), device)
    want = torch.from_numpy(golden["c4_y_bits"].view(np.int16).copy()).view(torch.bfloat16).float()
    eager.assert_close(ours, want, 2e-2, 2e-2, "sdpa golden")


# -- C5 ---------------------------------------------------------------------------


@pytest.mark.parametrize("dims", [(256, 4, 2, 64, 100), (512, 4, 2, 128, 72), (512, 8, 8, 64, 256)])
def test_head_norm_and_rope_in_the_projection_epilogue(device, dims):
    """q/k/v projection -> per-head RMSNorm (weights != 1) -> rotary embedding -> attention:
    two launches, the norm and rotation applied to the projection's output tile.  Ragged
    token counts exercise the row guards, 64-wide heads the eight-lane group reduce."""
    case = eager.normed_rope_attention_case(*dims)
    ours, want, compiled = run_case(case, device)
    ks = [n.op for n in compiled.nodes.values() if isinstance(n.op, HipOp)]
    assert len(ks) == 2 and "row-epilogue" in ks[0].comment
    eager.assert_close(ours, want, case.rtol, case.atol, f"{case.name} vs eager (GPU)")


@pytest.mark.parametrize("seq", [1, 2, 8, 16, 17, 32, 64, 128, 256, 512])  # 16 tokens = as many as query heads, 8 = as many as KV heads
def test_c5_qwen3_block(device, seq, golden):
    case = eager.qwen3_block_case(seq=seq)
    ours, want, compiled = run_case(case, device)
    eager.assert_close(ours, want, case.rtol, case.atol, f"block S={seq} vs eager (GPU)")
    # five launches; up to 32 tokens six: the q / k head norms + rotary embedding are one small launch of their own behind
    # a q/k/v projection in the few-row form (one token included: its unit token dim is not a row dim of the plan)
    names = [n.op.kernel_name.rsplit("_", 1)[0] for n in compiled.nodes.values() if isinstance(n.op, HipOp)]
    if seq <= 32:
        assert names == ["k_rms_norm_linear", "k_rms_norm_rope", "k_sdpa_reduce", "k_linear_add", "k_rms_norm_linear_silu_mul", "k_linear_add"], names
    else:
        assert names == ["k_rms_norm_linear_rope", "k_sdpa_reduce", "k_linear_add", "k_rms_norm_linear_silu_mul", "k_linear_add"], names
    # Scale-aware: the block's own contribution out - x has std ~0.3 and bf16 eager sits ~0.003 (mean) from the
    # fp32 run, so the absolute floor above is loose.  On out - x: our mean distance from fp32 eager may be at
    # most 1.5 x bf16 eager's, and no row may be further (relative L2) than 1.5 x bf16 eager's worst row.
    exact = eager.run_eager_fp32(case, device)
    x = case.inputs[0].to(device).float()
    eager.assert_mean_error_within_baseline(ours.float() - x, want.float() - x, exact - x, 1.5, f"block S={seq} (out - x) vs fp32 eager")
    eager.assert_rows_within_baseline(ours.float() - x, want.float() - x, exact - x, 1.5, f"block S={seq} rows of (out - x) vs fp32 eager")
    if seq == 32:
        gold = torch.from_numpy(golden["c5_y_bits"].view(np.int16).copy()).view(torch.bfloat16).float()
        eager.assert_close(ours, gold.reshape(ours.shape), case.rtol, case.atol, "block golden (CPU eager bf16)")
        eager.assert_close(ours, torch.from_numpy(golden["c5_y_f32"]).reshape(ours.shape), 2e-2, 6e-2, "block vs fp32 eager")
        xc = case.inputs[0].float().reshape(ours.shape)
        eager.assert_mean_error_within_baseline(ours.float().cpu() - xc, gold.reshape(ours.shape) - xc, torch.from_numpy(golden["c5_y_f32"]).reshape(ours.shape) - xc, 1.5, "block golden (out - x) vs fp32 eager")


@pytest.mark.parametrize("seq", [512, 40, 9, 1])
def test_c5_qwen3_block_with_random_norm_weights(device, seq):
    """Layer-norm and head-norm weights ~N(1, 0.1) instead of ones: the fold of a norm weight into the stacked
    projection weights and the pairing of head-norm weights with columns carry real values."""
    case = eager.qwen3_block_case(seq=seq, norm_std=0.1, seed=3)
    ours, want, _ = run_case(case, device)
    eager.assert_close(ours, want, case.rtol, case.atol, f"block S={seq} random norm weights vs eager (GPU)")
    exact = eager.run_eager_fp32(case, device)
    x = case.inputs[0].to(device).float()
    eager.assert_mean_error_within_baseline(ours.float() - x, want.float() - x, exact - x, 1.5, f"block S={seq} random norm weights (out - x) vs fp32 eager")
    eager.assert_rows_within_baseline(ours.float() - x, want.float() - x, exact - x, 1.5, f"block S={seq} random norm weights rows vs fp32 eager")


def test_run_api_returns_host_arrays_with_bf16_as_bits(device):
    case = eager.linear_case(m=16)
    be = HipBackend()
    compiled = be.compile(trace_module(case.module, case.inputs))
    marker = []
    res, pre = be.run(compiled, input_data={compiled.inputs[0]: case.inputs[0].view(torch.int16).numpy().view(np.uint16)}, pre_run=lambda: marker.append(1) or "pre")
    assert pre == "pre" and marker == [1]
    out = res.outputs[compiled.outputs[0]]
    assert out.dtype == np.uint16 and out.shape == (16, 3072)
    want = eager.run_eager(case, device).float().cpu()
    eager.assert_close(torch.from_numpy(O.from_bf16_bits(out)), want, 2e-2, 2e-2, "run() output")


def test_c5_block_dynamic_seq_len(device, monkeypatch):
    """One compile with a symbolic ``seq_len``: every kernel takes the length as a runtime ``int``, so the same five
    code objects run the block at every length — at most one hipRTC compile and one loaded module per kernel across
    all of them — and each length matches eager (ragged lengths exercise the row / key-block guards)."""
    from deplodock_amd.backend.hip import hiprtc, launcher

    case = eager.qwen3_block_case(seq=64)
    be = HipBackend()
    compiled = be.compile(trace_module(case.module, case.inputs, dynamic_shapes={"x": {1: "seq_len"}, "cos": {1: "seq_len"}, "sin": {1: "seq_len"}}))
    assert compiled.symbolic == "seq_len"
    ops = [n.op for n in compiled.nodes.values() if isinstance(n.op, HipOp)]
    assert len(ops) == 5 and all(op.runtime_args == ("seq_len",) for op in ops)
    compiles: list[str] = []
    real = launcher.Launcher.compile
    monkeypatch.setattr(launcher.Launcher, "compile", lambda self, source, name, arch, options: compiles.append(name) or real(self, source, name, arch, options))
    before = hiprtc.loaded_module_count()
    for seq in (64, 96, 32, 200, 7, 513):
        other = eager.qwen3_block_case(seq=seq)
        data = {n: t.to(device) for n, t in zip(compiled.inputs, other.inputs)}
        prog = be.program(compiled, data)
        try:
            assert prog.sym_values == {"seq_len": seq}
            prog.run()
            torch.cuda.synchronize()
            ours = prog.output_tensors()[compiled.outputs[0]]
            assert tuple(ours.shape) == (1, seq, 1024)
            want = eager.run_eager(other, device)
            eager.assert_close(ours.reshape(want.shape), want, other.rtol, other.atol, f"block with seq_len={seq} through the runtime-int kernels")
            exact = eager.run_eager_fp32(other, device)
            x = other.inputs[0].to(device).float()
            eager.assert_mean_error_within_baseline(ours.float() - x, want.float() - x, exact - x, 1.5, f"block seq_len={seq} (out - x) vs fp32 eager")
        finally:
            prog.close()
    assert len(compiles) <= 5 and len(set(compiles)) == len(compiles), compiles
    assert hiprtc.loaded_module_count() - before <= 5
    # a captured graph of one length replays correctly after programs of other lengths ran in between
    data = {n: t.to(device) for n, t in zip(compiled.inputs, eager.qwen3_block_case(seq=96).inputs)}
    prog = be.program(compiled, data)
    try:
        prog.capture_program_graph()
        for _ in range(3):
            prog.output_tensors()[compiled.outputs[0]].zero_()
            prog.replay_program()
            torch.cuda.synchronize()
            want = eager.run_eager(eager.qwen3_block_case(seq=96), device)
            eager.assert_close(prog.output_tensors()[compiled.outputs[0]].reshape(want.shape), want, 2e-2, 4e-2, "graph replay at seq_len=96")
    finally:
        prog.close()


def test_dynamic_seq_len_per_size_variants_still_work(device):
    """The fallback for modules that do not symbolise (forced here): a re-trace and re-lowering per size."""
    case = eager.qwen3_block_case(seq=64)
    be = HipBackend()
    be.symbolic_kernels = False
    compiled = be.compile(trace_module(case.module, case.inputs, dynamic_shapes={"x": {1: "seq_len"}, "cos": {1: "seq_len"}, "sin": {1: "seq_len"}}))
    for seq in (64, 96):
        other = eager.qwen3_block_case(seq=seq)
        prog = be.program(compiled, {n: t.to(device) for n, t in zip(compiled.inputs, other.inputs)})
        try:
            prog.run()
            torch.cuda.synchronize()
            want = eager.run_eager(other, device)
            eager.assert_close(prog.output_tensors()[compiled.outputs[0]].reshape(want.shape), want, other.rtol, other.atol, f"block with seq_len={seq} through a per-size variant")
        finally:
            prog.close()
    assert len(compiled.variants) == 2


@pytest.mark.parametrize("which", ["rms_norm", "softmax", "silu_mul", "sdpa", "sdpa_masked", "embedding", "linear_bias", "linear_f32"])
def test_runtime_int_kernels_of_every_family(device, which):
    """Row kernels (rows symbolic), a pointwise map (element count symbolic), attention on ``[B, H, S, D]`` operands
    (lengths and the batch stride symbolic) and a biased linear (rows symbolic), each compiled once and run at
    several sizes of the axis, including sizes below one tile and sizes that leave ragged tiles."""

    class SiluMul(nn.Module):
        def forward(self, x, y):
            return nn.functional.silu(x) * y

    torch.manual_seed(12)
    if which == "rms_norm":
        mod = nn.RMSNorm(1024, eps=1e-6).eval()
        make = lambda s: (torch.randn(2, s, 1024),)  # noqa: E731
        dyn, tol = {"x": {1: "s"}}, (1e-5, 1e-6)
    elif which == "softmax":
        mod = nn.Softmax(dim=-1).eval()
        make = lambda s: (torch.randn(s, 777),)  # noqa: E731
        dyn, tol = {"input": {0: "s"}}, (1e-5, 1e-9)
    elif which == "silu_mul":
        mod = SiluMul().eval()
        make = lambda s: (torch.randn(s, 96).bfloat16(), torch.randn(s, 96).bfloat16())  # noqa: E731
        dyn, tol = {"x": {0: "s"}, "y": {0: "s"}}, (2e-2, 2e-2)
    elif which == "sdpa":
        mod = eager.Sdpa(True).eval()
        make = lambda s: (torch.randn(2, 4, s, 128).bfloat16(), torch.randn(2, 2, s, 128).bfloat16(), torch.randn(2, 2, s, 128).bfloat16())  # noqa: E731
        dyn, tol = {"q": {2: "s"}, "k": {2: "s"}, "v": {2: "s"}}, (2e-2, 2e-2)
    elif which == "sdpa_masked":
        # a float bias [1, 1, S, S] broadcast over batch and heads, the way a whole-model trace passes its mask: only the
        # row stride follows the axis; rows start on a four-element boundary at some sizes (vector loads) and not at others
        mod = eager.MaskedSdpa().eval()

        def make(s):
            bias = torch.zeros(1, 1, s, s).masked_fill(torch.ones(s, s, dtype=torch.bool).triu(1), float("-inf")).bfloat16()
            return (torch.randn(2, 4, s, 128).bfloat16(), torch.randn(2, 2, s, 128).bfloat16(), torch.randn(2, 2, s, 128).bfloat16(), bias)

        dyn, tol = {"q": {2: "s"}, "k": {2: "s"}, "v": {2: "s"}, "mask": {2: "s", 3: "s"}}, (2e-2, 2e-2)
    elif which == "embedding":
        # token ids [batch, s] into a table that does not follow the axis: the looked-up row count does
        mod = nn.Embedding(300, 64).eval()
        make = lambda s: (torch.randint(0, 300, (2, s)),)  # noqa: E731
        dyn, tol = {"input": {1: "s"}}, (0.0, 0.0)
    elif which == "linear_f32":
        # at the traced size the static fp32 lowering would split the reduction axis across workgroups (a kernel pair
        # with the row count baked in): the runtime-int form must stay unsplit and serve every size
        mod = nn.Linear(1024, 1024).eval()
        make = lambda s: (torch.randn(s, 1024),)  # noqa: E731
        dyn, tol = {"input": {0: "s"}}, (1e-5, 1e-5)
    else:
        mod = nn.Linear(256, 520).bfloat16().eval()
        make = lambda s: (torch.randn(s, 256).bfloat16(),)  # noqa: E731
        dyn, tol = {"input": {0: "s"}}, (2e-2, 2e-2)
    be = HipBackend()
    compiled = be.compile(trace_module(mod, make(48), dynamic_shapes=dyn))
    assert compiled.symbolic == "s"
    assert all(n.op.runtime_args == ("s",) for n in compiled.nodes.values() if isinstance(n.op, HipOp))
    for size in (48, 1, 200, 33):
        inputs = make(size)
        prog = be.program(compiled, {n: t.to(device) for n, t in zip(compiled.inputs, inputs)})
        try:
            prog.run()
            torch.cuda.synchronize()
            with torch.no_grad():
                want = mod.to(device)(*(t.to(device) for t in inputs))
            eager.assert_close(prog.output_tensors()[compiled.outputs[0]].reshape(want.shape), want, *tol, f"{which} at s={size}")
        finally:
            prog.close()


class _HfRmsNorm(nn.Module):
    """The RMSNorm HF decoder layers trace to: fp32 statistics, round, then the weight."""

    def __init__(self, n, eps=1e-6):
        super().__init__()
        self.weight = nn.Parameter(1.0 + 0.1 * torch.randn(n))
        self.eps = eps

    def forward(self, x):
        h = x.to(torch.float32)
        h = h * torch.rsqrt(h.pow(2).mean(-1, keepdim=True) + self.eps)
        return self.weight * h.to(x.dtype)


class _NormLinear(nn.Module):
    def __init__(self, k, n, norm, share=False):
        super().__init__()
        self.norm = norm
        self.lin = nn.Linear(k, n, bias=False)
        self.share = share

    def forward(self, x):
        h = self.norm(x)
        y = self.lin(h)
        return (y, h) if self.share else y


@pytest.mark.parametrize("kind,m,k,n", [("hf", 512, 1024, 768), ("hf", 100, 512, 264), ("torch", 256, 1024, 512), ("hf", 16, 1024, 3072)])
def test_row_norm_as_contraction_prologue(device, kind, m, k, n):
    """``norm -> linear`` is one launch; the operand the MFMAs see carries the norm's own rounding points."""
    torch.manual_seed(3)
    norm = _HfRmsNorm(k) if kind == "hf" else nn.RMSNorm(k, eps=1e-6)
    if kind == "torch":
        with torch.no_grad():
            norm.weight.copy_(1.0 + 0.1 * torch.randn(k))
    mod = _NormLinear(k, n, norm).bfloat16().eval()
    x = (3.0 * torch.randn(m, k)).bfloat16()
    be = HipBackend()
    compiled = be.compile(trace_module(mod, (x,)))
    ops = [n_.op for n_ in compiled.nodes.values() if isinstance(n_.op, HipOp)]
    assert len(ops) == 1 and ops[0].kernel_name.startswith("k_rms_norm_linear") and "a=row-normalised" in ops[0].comment
    prog = be.program(compiled, {compiled.inputs[0]: x.to(device)})
    try:
        prog.run()
        torch.cuda.synchronize()
        ours = prog.output_tensors()[compiled.outputs[0]]
        with torch.no_grad():
            want = mod.to(device)(x.to(device))
        eager.assert_close(ours.reshape(want.shape), want, 2e-2, 2e-2, f"{kind} norm -> linear {m}x{k}x{n}")
        # against the unfused pipeline's own numbers (norm kernel, then linear kernel): far tighter
        with torch.no_grad():
            h = mod.norm(x.to(device))
            ref = (h.float() @ mod.lin.weight.float().T).to(torch.bfloat16)
        assert (ours.reshape(ref.shape).float() - ref.float()).abs().max() <= 2e-2 * ref.float().abs().max()
    finally:
        prog.close()


class _NormGateUp(nn.Module):
    def __init__(self, k, n, norm):
        super().__init__()
        self.norm, self.gate, self.up = norm, nn.Linear(k, n, bias=False), nn.Linear(k, n, bias=False)

    def forward(self, x):
        h = self.norm(x)
        return nn.functional.silu(self.gate(h)) * self.up(h)


@pytest.mark.parametrize("kind,m,k,n", [("hf", 512, 1024, 768), ("torch", 100, 512, 256), ("hf", 64, 2048, 384)])
def test_row_norm_deferred_into_a_stacked_projection(device, kind, m, k, n):
    """``norm -> gate/up``: the norm weight (not all ones) is folded into the stacked weights when they are
    bound, the rows are staged untouched and the accumulators take the row's ``rsqrt(mean x^2 + eps)``."""
    torch.manual_seed(5)
    norm = _HfRmsNorm(k) if kind == "hf" else nn.RMSNorm(k, eps=1e-6)
    with torch.no_grad():
        norm.weight.copy_(1.0 + 0.3 * torch.randn(k))
    mod = _NormGateUp(k, n, norm).bfloat16().eval()
    x = (2.0 * torch.randn(m, k)).bfloat16()
    be = HipBackend()
    compiled = be.compile(trace_module(mod, (x,)))
    ops = [n_.op for n_ in compiled.nodes.values() if isinstance(n_.op, HipOp)]
    assert len(ops) == 1 and "a=row-scaled-after" in ops[0].comment and len(ops[0].arg_order) == 3
    bound = be.bind(compiled, {})
    (wname,) = [a for a in ops[0].arg_order if "__k*" in a]
    want_w = (torch.cat([mod.gate.weight, mod.up.weight]).float() * mod.norm.weight.float()[None, :]).to(torch.bfloat16)
    assert torch.equal(torch.as_tensor(bound[wname]).cpu(), want_w)
    prog = be.program(compiled, {compiled.inputs[0]: x.to(device)})
    try:
        prog.run()
        torch.cuda.synchronize()
        ours = prog.output_tensors()[compiled.outputs[0]]
        with torch.no_grad():
            want = mod.to(device)(x.to(device))
            exact = mod.float()(x.to(device).float())  # the same module without any 16-bit rounding inside
        eager.assert_close(ours.reshape(want.shape), want, 2e-2, 2e-2, f"{kind} norm -> gate/up {m}x{k}x{n}")
        # never rounding the normalised rows must not be *worse* than eager against the exact result
        ours_err = (ours.reshape(exact.shape).float() - exact).abs().max().item()
        eager_err = (want.float() - exact).abs().max().item()
        assert ours_err <= 1.5 * eager_err + 1e-3, (ours_err, eager_err)
    finally:
        prog.close()


def test_row_norm_with_a_second_reader_stays_a_kernel(device):
    torch.manual_seed(4)
    mod = _NormLinear(512, 256, _HfRmsNorm(512), share=True).bfloat16().eval()
    x = torch.randn(64, 512).bfloat16()
    be = HipBackend()
    compiled = be.compile(trace_module(mod, (x,)))
    names = [n_.op.kernel_name.rsplit("_", 1)[0] for n_ in compiled.nodes.values() if isinstance(n_.op, HipOp)]
    assert names == ["k_rms_norm_reduce", "k_linear"]
    prog = be.program(compiled, {compiled.inputs[0]: x.to(device)})
    try:
        prog.run()
        torch.cuda.synchronize()
        outs = prog.output_tensors()
        with torch.no_grad():
            want_y, want_h = mod.to(device)(x.to(device))
        eager.assert_close(outs[compiled.outputs[0]].reshape(want_y.shape), want_y, 2e-2, 2e-2, "linear of a shared norm")
        eager.assert_close(outs[compiled.outputs[1]].reshape(want_h.shape), want_h, 2e-2, 2e-2, "shared norm")
    finally:
        prog.close()


@pytest.mark.parametrize("m,k,n,dtype", [(128, 512, 768, torch.bfloat16), (100, 512, 260, torch.bfloat16), (16, 1024, 3072, torch.float16), (2048, 1024, 3072, torch.bfloat16),
                                         (1, 1024, 3072, torch.bfloat16), (7, 512, 260, torch.float16)])
def test_linear_with_bias(device, m, k, n, dtype):
    """``nn.Linear``'s default has a bias: it is added to the fp32 accumulator before the one rounding."""
    torch.manual_seed(5)
    mod = nn.Linear(k, n).to(dtype).eval()
    with torch.no_grad():
        mod.bias.copy_(torch.randn(n))
    x = torch.randn(m, k).to(dtype)
    be = HipBackend()
    compiled = be.compile(trace_module(mod, (x,)))
    assert sum(isinstance(n_.op, HipOp) for n_ in compiled.nodes.values()) == 1
    prog = be.program(compiled, {compiled.inputs[0]: x.to(device)})
    try:
        prog.run()
        torch.cuda.synchronize()
        ours = prog.output_tensors()[compiled.outputs[0]]
        want = (x.to(device).float() @ mod.weight.to(device).float().T + mod.bias.to(device).float()).to(dtype)
        eager.assert_close(ours.reshape(want.shape), want, 2e-2, 2e-2, f"linear+bias {m}x{k}x{n} vs fp32-accumulated reference")
        with torch.no_grad():
            eager.assert_close(ours.reshape(want.shape), mod.to(device)(x.to(device)), 2e-2, 2e-2, f"linear+bias {m}x{k}x{n} vs eager")
    finally:
        prog.close()


def test_residual_linear_with_bias(device):
    class Res(nn.Module):
        def __init__(self):
            super().__init__()
            self.lin = nn.Linear(256, 256)

        def forward(self, x):
            return x + self.lin(x)

    torch.manual_seed(6)
    mod = Res().bfloat16().eval()
    x = torch.randn(192, 256).bfloat16()
    be = HipBackend()
    compiled = be.compile(trace_module(mod, (x,)))
    ops = [n_.op for n_ in compiled.nodes.values() if isinstance(n_.op, HipOp)]
    assert len(ops) == 1 and ops[0].kernel_name.startswith("k_linear_add")
    prog = be.program(compiled, {compiled.inputs[0]: x.to(device)})
    try:
        prog.run()
        torch.cuda.synchronize()
        with torch.no_grad():
            want = mod.to(device)(x.to(device))
        eager.assert_close(prog.output_tensors()[compiled.outputs[0]].reshape(want.shape), want, 2e-2, 2e-2, "x + linear(x) with bias")
    finally:
        prog.close()


@pytest.mark.parametrize("bias", [False, True])
@pytest.mark.parametrize("m,k,n", [(2048, 1024, 3072), (512, 2048, 2048), (37, 200, 52), (1, 1024, 3072), (16, 512, 64), (300, 1000, 512), (130, 64, 1028)])
def test_fp32_linear(device, m, k, n, bias):
    """The fp32 contraction tier (fp32 MFMA, full-precision products): fp32 rtol 1e-5 against float64 and against
    eager, with the absolute floor a sum of k products of unit-scale terms needs (1e-5; outputs are O(1))."""
    torch.manual_seed(m + k)
    lin = nn.Linear(k, n, bias=bias).eval()
    x = torch.randn(m, k)
    be = HipBackend()
    compiled = be.compile(trace_module(lin, (x,)))
    ops = [n_.op for n_ in compiled.nodes.values() if isinstance(n_.op, HipOp)]
    assert all("_f32/" in op.knobs["TILE"] for op in ops)
    # one row over a 12 MiB weight leaves most CUs idle on 32-column tiles: the reduction axis is split across workgroups
    # (partials + combine); every other case here is one launch
    assert sorted(op.kernel_name.rsplit("_", 1)[0] for op in ops) == (["k_linear_combine", "k_linear_partial"] if (m, k, n) == (1, 1024, 3072) else ["k_linear"])
    prog = be.program(compiled, {compiled.inputs[0]: x.to(device)})
    try:
        prog.run()
        torch.cuda.synchronize()
        ours = prog.output_tensors()[compiled.outputs[0]].clone()
    finally:
        prog.close()
    exact = x.double() @ lin.weight.detach().double().T + (lin.bias.detach().double() if bias else 0.0)
    eager.assert_close(ours.reshape(exact.shape), exact, 1e-5, 1e-5, f"fp32 linear {m}x{k}x{n} vs float64")
    tf32 = torch.backends.cuda.matmul.allow_tf32
    torch.backends.cuda.matmul.allow_tf32 = False
    try:
        with torch.no_grad():
            want = lin.to(device)(x.to(device))
    finally:
        torch.backends.cuda.matmul.allow_tf32 = tf32
    eager.assert_close(ours.reshape(want.shape), want, 1e-5, 2e-5, f"fp32 linear {m}x{k}x{n} vs eager")


@pytest.mark.parametrize("stage", ["d2/sync", "d2/sync/p2", "d2/dl", "d3/dl", "d3/dli", "d2/dlm", "d3/dlm"])
def test_fp32_linear_every_transport_is_bit_identical(device, stage, monkeypatch):
    monkeypatch.setenv("EMMY_TILE", "a:mfma_16x16x4_f32/w2x2/f2x2/k8")
    torch.manual_seed(8)
    lin = nn.Linear(512, 256, bias=False).eval()
    x = torch.randn(192, 512)
    outs = {}
    for st in ("d2/sync", stage):
        monkeypatch.setenv("EMMY_STAGE", st)
        be = HipBackend()
        compiled = be.compile(trace_module(lin, (x,)))
        (op,) = [n_.op for n_ in compiled.nodes.values() if isinstance(n_.op, HipOp)]
        assert op.knobs["STAGE"] == st
        prog = be.program(compiled, {compiled.inputs[0]: x.to(device)})
        try:
            for _ in range(5):
                prog.run()
                torch.cuda.synchronize()
                y = prog.output_tensors()[compiled.outputs[0]].clone()
                assert st not in outs or torch.equal(y, outs[st])
                outs[st] = y
        finally:
            prog.close()
    assert torch.equal(outs[stage], outs["d2/sync"])


@pytest.mark.parametrize("reduce", ["g2k", "g4k", "g2a", "g4a"])
@pytest.mark.parametrize("m,k,n", [(1, 1024, 3072), (16, 1024, 3072), (128, 1024, 3072), (40, 1536, 1000), (130, 4096, 264)])
def test_split_k_linear(device, m, k, n, reduce, monkeypatch):
    """Cross-workgroup split of the reduction axis, workspace + combine (``k``) and atomic adds into a cleared
    workspace (``a``), on the decode / few-row shapes it is meant for, ragged rows and columns, a 1536-deep
    reduction (three slabs of 512 for g2/g4... whole 64-deep slabs per slice): against eager and against float64.
    The ``k`` arm adds its planes in a fixed order, so repeated launches are bit-identical."""
    monkeypatch.setenv("EMMY_REDUCE", reduce)
    monkeypatch.setenv("EMMY_TILE", "a:mfma_16x16x32_bf16/w2x2/f1x2/k2")  # 64-deep slabs: every shape here splits into whole ones
    case = eager.linear_case(m=m, k=k, n=n, seed=m + n)
    be = HipBackend()
    compiled = be.compile(trace_module(case.module, case.inputs))
    ops = [n_.op for n_ in compiled.nodes.values() if isinstance(n_.op, HipOp)]
    assert len(ops) == 2 and all(o.knobs["REDUCE"] == reduce for o in ops)
    want = eager.run_eager(case, device)
    exact = case.inputs[0].double() @ case.module.weight.detach().double().cpu().T
    prog = be.program(compiled, {compiled.inputs[0]: case.inputs[0].to(device)})
    try:
        out = prog.output_tensors()[compiled.outputs[0]]
        first = None
        for rep in range(4):
            out.zero_()
            prog.run()
            torch.cuda.synchronize()
            eager.assert_close(out.reshape(want.shape), want, case.rtol, case.atol, f"split-K {reduce} {m}x{k}x{n} launch {rep} vs eager")
            eager.assert_close(out.reshape(want.shape), exact, 2 ** -7, 2e-3, f"split-K {reduce} {m}x{k}x{n} launch {rep} vs float64")
            if reduce.endswith("k"):
                first = out.clone() if first is None else first
                assert torch.equal(out, first), "workspace + combine must be bit-reproducible"
    finally:
        prog.close()


def test_split_k_combine_owns_bias_and_residual(device, monkeypatch):
    """The combine kernel applies what the unsplit kernel's output stage applies: bias into the fp32 sum, one
    rounding, then the residual add and the second rounding — bit-identical to the unsplit kernel for the ``k`` arm."""

    class Res(nn.Module):
        def __init__(self):
            super().__init__()
            self.lin = nn.Linear(512, 512)

        def forward(self, x):
            return x + self.lin(x)

    torch.manual_seed(6)
    mod = Res().bfloat16().eval()
    with torch.no_grad():
        mod.lin.bias.copy_(torch.randn(512))
    x = torch.randn(96, 512).bfloat16()
    monkeypatch.setenv("EMMY_TILE", "a:mfma_16x16x32_bf16/w2x2/f1x2/k2")
    outs = {}
    for reduce in ("", "g2k", "g4a"):
        monkeypatch.setenv("EMMY_REDUCE", reduce)
        be = HipBackend()
        compiled = be.compile(trace_module(mod, (x,)))
        assert sum(isinstance(n_.op, HipOp) for n_ in compiled.nodes.values()) == (2 if reduce else 1)
        prog = be.program(compiled, {compiled.inputs[0]: x.to(device)})
        try:
            prog.run()
            torch.cuda.synchronize()
            outs[reduce] = prog.output_tensors()[compiled.outputs[0]].clone()
        finally:
            prog.close()
    with torch.no_grad():
        want = mod.to(device)(x.to(device))
    for reduce, y in outs.items():
        eager.assert_close(y.reshape(want.shape), want, 2e-2, 2e-2, f"x + linear(x) with bias, REDUCE={reduce or '-'}")
    # same fp32 terms, same rounding points; only the association of the k sum differs between split and unsplit
    assert float((outs["g2k"].float() - outs[""].float()).abs().max()) <= 2 ** -6


def test_fused_pointwise_with_broadcasts_and_row_reductions(device):
    class Mix(nn.Module):
        def forward(self, x, y, w, s):
            centred = x - x.mean(-1, keepdim=True)  # one value per row, broadcast back
            return torch.exp(torch.neg(centred)) * y + w * s + x.sum(-1, keepdim=True) * 0.01  # vector, scalar

    torch.manual_seed(8)
    args = (torch.randn(96, 320), torch.randn(96, 320), torch.randn(320), torch.randn(1))
    mod = Mix().eval()
    be = HipBackend()
    compiled = be.compile(trace_module(mod, args))
    prog = be.program(compiled, {n: t.to(device) for n, t in zip(compiled.inputs, args)})
    try:
        prog.run()
        torch.cuda.synchronize()
        want = mod(*[a.to(device) for a in args])
        eager.assert_close(prog.output_tensors()[compiled.outputs[0]].reshape(want.shape), want, 1e-5, 1e-5, "fused pointwise + row reductions (fp32)")
    finally:
        prog.close()

    class Bf16Chain(nn.Module):
        def forward(self, x, y):
            return torch.nn.functional.silu(x) * y + x  # every op rounds to bf16 in eager

    xb, yb = torch.randn(64, 512).bfloat16(), torch.randn(64, 512).bfloat16()
    compiled = be.compile(trace_module(Bf16Chain().eval(), (xb, yb)))
    assert sum(isinstance(n_.op, HipOp) for n_ in compiled.nodes.values()) == 1
    prog = be.program(compiled, {n: t.to(device) for n, t in zip(compiled.inputs, (xb, yb))})
    try:
        prog.run()
        torch.cuda.synchronize()
        want = Bf16Chain()(xb.to(device), yb.to(device))
        eager.assert_close(prog.output_tensors()[compiled.outputs[0]].reshape(want.shape), want, 2e-2, 2e-2, "bf16 element-wise chain")
    finally:
        prog.close()


def test_mixed_staging_with_a_normalised_operand(device, monkeypatch):
    """``STAGE=d2/mix``: the normalised operand goes through registers, the weight slab direct to LDS."""
    monkeypatch.setenv("EMMY_STAGE", "d2/mix")
    case = eager.qwen3_block_case(seq=64)
    ours, want, compiled = run_case(case, device)
    stages = [n.op.knobs.get("STAGE") for n in compiled.nodes.values() if isinstance(n.op, HipOp) and "TILE" in n.op.knobs]
    assert stages and all(s == "d2/mix" for s in stages)
    eager.assert_close(ours, want, case.rtol, case.atol, "block with mixed staging vs eager (GPU)")


def test_staging_transports_are_bit_identical(device, monkeypatch):
    """How operands reach LDS (through registers, or direct-to-LDS at any depth) must not change a
    single output bit: same tile, same MFMA order (the reference pins the same property across its
    staging transports, tests/compiler/e2e/test_matmul_coverage.py:298-328)."""
    case = eager.linear_case(m=256, k=1024, n=512)
    graph = trace_module(case.module, case.inputs)
    x = case.inputs[0].to(device)
    monkeypatch.setenv("EMMY_TILE", "a:mfma_32x32x16_bf16/w2x2/f1x2/k4")
    outs = {}
    for stage in ("d2/sync", "d2/sync/p2", "d2/sync/p3", "d2/mix", "d2/dl", "d3/dl", "d4/dl", "d3/dli", "d4/dli", "d2/dlm", "d3/dlm", "d4/dlm"):  # 16 slabs: not a multiple of three register sets
        monkeypatch.setenv("EMMY_STAGE", stage)
        be = HipBackend()
        compiled = be.compile(graph)
        (op,) = [n_.op for n_ in compiled.nodes.values() if isinstance(n_.op, HipOp)]
        assert op.knobs["STAGE"] == stage
        prog = be.program(compiled, {compiled.inputs[0]: x})
        try:
            for _ in range(40):  # direct-to-LDS publication races would show as run-to-run differences
                prog.run()
                torch.cuda.synchronize()
                y = prog.output_tensors()[compiled.outputs[0]].clone()
                if stage in outs:
                    assert torch.equal(y, outs[stage]), f"{stage}: outputs differ between launches"
                outs[stage] = y
        finally:
            prog.close()
    for stage, y in outs.items():
        assert torch.equal(y, outs["d2/sync"]), f"{stage} differs from d2/sync"
    eager.assert_close(outs["d2/sync"], eager.run_eager(case, device), case.rtol, case.atol, "pinned tile vs eager")


@pytest.mark.parametrize("dims,tile", [((256, 1024, 384), "a:mfma_16x16x32_bf16/w2x4/f4x3/k2"), ((200, 512, 388), "a:mfma_16x16x32_bf16/w2x4/f4x3/k2"),
                                       ((512, 192, 512), "a:mfma_16x16x32_bf16/w4x2/f2x4/k2"), ((384, 64, 256), "a:mfma_32x32x16_bf16/w2x4/f1x1/k4")])  # fmt: skip
def test_wave_specialised_ring_is_bit_identical_to_register_staging(device, dims, tile, monkeypatch):
    """``STAGE d<n>/pp`` (four staging waves, the tile's eight waves alternating in two groups) at every ring depth
    it takes, on whole and ragged tiles, long and short reduction axes (fewer slabs than the ring holds included):
    the same bits as ``d2/sync`` on the same tile, launch after launch."""
    m, k, n = dims
    case = eager.linear_case(m=m, k=k, n=n, seed=31)
    graph = trace_module(case.module, case.inputs)
    x = case.inputs[0].to(device)
    monkeypatch.setenv("EMMY_TILE", tile)
    outs = {}
    for stage in ("d2/sync", "d3/pp", "d4/pp", "d5/pp"):
        monkeypatch.setenv("EMMY_STAGE", stage)
        be = HipBackend()
        compiled = be.compile(graph)
        (op,) = [n_.op for n_ in compiled.nodes.values() if isinstance(n_.op, HipOp)]
        if op.knobs["STAGE"] != stage:
            assert stage == "d5/pp"  # the deepest ring does not fit the LDS on the larger tiles
            continue
        assert stage.endswith("sync") or op.block[0] == (768,)
        prog = be.program(compiled, {compiled.inputs[0]: x})
        try:
            for _ in range(30):
                prog.run()
                torch.cuda.synchronize()
                y = prog.output_tensors()[compiled.outputs[0]].clone()
                if stage in outs:
                    assert torch.equal(y, outs[stage]), f"{stage}: outputs differ between launches"
                outs[stage] = y
        finally:
            prog.close()
    assert len(outs) >= 3
    for stage, y in outs.items():
        assert torch.equal(y, outs["d2/sync"]), f"{stage} differs from d2/sync"
    eager.assert_close(outs["d2/sync"], eager.run_eager(case, device), case.rtol, case.atol, f"{tile} vs eager")


def _soak(prog, out_name: str, launches: int, what: str) -> None:
    """``launches`` runs of a bound program on fixed inputs, every output compared bit for bit with the first
    launch's; stops at the first mismatch."""
    out = prog.output_tensors()[out_name]
    prog.run()
    torch.cuda.synchronize()
    first = out.clone()
    for i in range(1, launches):
        out.zero_()
        prog.run()
        torch.cuda.synchronize()
        if not torch.equal(out, first):
            bad = int((out.view(torch.int16) != first.view(torch.int16)).sum())
            pytest.fail(f"{what}: launch {i} of {launches} differs from the first launch in {bad} elements")


@pytest.mark.parametrize("stage", ["d3/dl", "d3/dli", "d2/dlm", "d3/dlm", "d4/pp", "d3/pp"])
def test_soak_direct_to_lds_contraction_is_bit_stable_over_thousands_of_launches(device, stage, monkeypatch):
    """The publication fence of the direct-to-LDS rings (a flat LDS read of the issuing wave, waited for on the
    LDS counter, before the barrier) as a test: a race that let one wave read a slab before another wave's loads
    were visible showed as run-to-run differences in about a quarter of the launches without it.  3000 launches
    of a machine-filling contraction on fixed inputs must reproduce the first launch bit for bit, and that
    result must be the register-staged transport's."""
    monkeypatch.setenv("EMMY_TILE", "a:mfma_16x16x32_bf16/w2x4/f4x3/k2")
    monkeypatch.setenv("EMMY_STAGE", stage)
    case = eager.linear_case(m=2048, k=1024, n=3072, seed=21)
    be = HipBackend()
    compiled = be.compile(trace_module(case.module, case.inputs))
    (op,) = [n_.op for n_ in compiled.nodes.values() if isinstance(n_.op, HipOp)]
    assert op.knobs["STAGE"] == stage
    prog = be.program(compiled, {compiled.inputs[0]: case.inputs[0].to(device)})
    try:
        _soak(prog, compiled.outputs[0], 3000, f"contraction {stage}")
        got = prog.output_tensors()[compiled.outputs[0]].clone()
    finally:
        prog.close()
    monkeypatch.setenv("EMMY_STAGE", "d2/sync")
    ref, _, _ = run_case(case, device)
    assert torch.equal(got.reshape(ref.shape), ref), f"{stage} differs from register staging"


@pytest.mark.parametrize("pin", ["w2/kv32/s4/p", "w4/kv64/s2", "w8/kv64/s1/p"])
def test_soak_flash_staging_is_bit_stable_over_thousands_of_launches(device, pin, monkeypatch):
    """The same for the attention kernel's K/V blocks (one family per workgroup shape: key-split pairs, key
    split, eight query waves): 2000 launches on fixed inputs, bit-identical to the first, which matches eager."""
    monkeypatch.setenv("EMMY_FLASH", pin)
    case = eager.sdpa_case(b=1, hq=16, hkv=8, s=1024, d=128, seed=22)
    be = HipBackend()
    compiled = be.compile(trace_module(case.module, case.inputs))
    assert [n.op.knobs["FLASH"] for n in compiled.nodes.values() if isinstance(n.op, HipOp)] == [pin]
    prog = be.program(compiled, {n: t.to(device) for n, t in zip(compiled.inputs, case.inputs)})
    try:
        _soak(prog, compiled.outputs[0], 2000, f"flash {pin}")
        got = prog.output_tensors()[compiled.outputs[0]].clone()
    finally:
        prog.close()
    want = eager.run_eager(case, device)
    eager.assert_close(got.reshape(want.shape), want, case.rtol, case.atol, f"flash {pin} after the soak vs eager")


@pytest.mark.parametrize("cols", [151936, 70000])
def test_streamed_softmax_over_a_vocabulary(device, cols):
    """Rows too long for registers are streamed; max and sum-of-exponentials share one pass (online carrier)."""
    torch.manual_seed(12)
    x = 3.0 * torch.randn(5, cols)
    x[1, 1000:60000] = float("-inf")  # masked logits, including whole chunks of a lane
    x[2, 7] = 80.0  # one dominant entry
    be = HipBackend()
    compiled = be.compile(trace_module(nn.Softmax(-1).eval(), (x,)))
    (op,) = [n_.op for n_ in compiled.nodes.values() if isinstance(n_.op, HipOp)]
    assert op.knobs["REDUCE"] == "b1024/stream" and "2 reads of the row" in op.comment
    prog = be.program(compiled, {compiled.inputs[0]: x.to(device)})
    try:
        prog.run()
        torch.cuda.synchronize()
        ours = prog.output_tensors()[compiled.outputs[0]]
        want = torch.softmax(x.to(device), -1)
        eager.assert_close(ours, want, 1e-5, 1e-9, f"streamed softmax over {cols} columns")
        assert torch.allclose(ours.sum(-1), torch.ones(5, device=device), atol=1e-4)
        ref = O.softmax(x[:1, :].double().numpy())
        eager.assert_close(ours[:1].double().cpu(), torch.from_numpy(ref), 1e-5, 1e-9, "streamed softmax vs numpy restatement")
    finally:
        prog.close()


def test_streamed_rms_norm_and_pinned_streaming(device, monkeypatch):
    torch.manual_seed(13)
    mod = nn.RMSNorm(100000, eps=1e-6).eval()
    with torch.no_grad():
        mod.weight.copy_(1.0 + 0.1 * torch.randn(100000))
    x = torch.randn(3, 100000)
    be = HipBackend()
    compiled = be.compile(trace_module(mod, (x,)))
    prog = be.program(compiled, {compiled.inputs[0]: x.to(device)})
    try:
        prog.run()
        torch.cuda.synchronize()
        eager.assert_close(prog.output_tensors()[compiled.outputs[0]], mod.to(device)(x.to(device)), 1e-5, 1e-6, "streamed RMSNorm")
    finally:
        prog.close()
    # the streaming form can be pinned on a row that would fit in registers; results agree with the resident form
    case = eager.softmax_case(shape=(2, 3, 64, 2048))
    monkeypatch.setenv("EMMY_REDUCE", "b1024/stream")
    ours, want, compiled = run_case(case, device)
    assert [n_.op.knobs["REDUCE"] for n_ in compiled.nodes.values() if isinstance(n_.op, HipOp)] == ["b1024/stream"]
    eager.assert_close(ours, want, case.rtol, case.atol, "pinned streaming softmax")


@pytest.mark.gpu
@pytest.mark.parametrize(
    "dtype, p, m, n, k, shared",
    [("bf16", 32, 128, 128, 64, False), ("bf16", 6, 100, 72, 96, True), ("f32", 32, 128, 64, 128, False), ("f32", 5, 37, 40, 72, True), ("bf16", 16, 512, 512, 64, False)],
)
def test_batched_linear(device, dtype, p, m, n, k, shared):
    """``[P, M, K] x [P | 1, N, K] -> [P, M, N]``: the per-head products of attention as one launch of the MFMA
    contraction (workgroup row ``p`` takes product ``p``), ragged tiles included, against a float64 product."""
    from deplodock_amd.ir import frontend as F

    dt, tdt = (BF16, torch.bfloat16) if dtype == "bf16" else (F32, torch.float32)
    torch.manual_seed(21)
    x = torch.randn(p, m, k).to(tdt)
    w = (0.1 * torch.randn(1 if shared else p, n, k)).to(tdt)
    g = Graph()
    g.add_input("x", tuple(x.shape), dt)
    g.add_input("w", tuple(w.shape), dt)
    g.add_node(F.BatchedLinearOp(), ["x", "w"], Tensor("y", (p, m, n), dt), "y")
    g.outputs = ["y"]
    be = HipBackend()
    compiled = be.compile(g)
    ks = [nd.op for nd in compiled.nodes.values() if isinstance(nd.op, HipOp)]
    assert len(ks) == 1 and ks[0].kernel_name.startswith("k_batched_linear_") and ks[0].grid[1] == (p,)
    prog = be.program(compiled, {"x": x.to(device), "w": w.to(device)})
    try:
        prog.run()
        torch.cuda.synchronize()
        ours = prog.output_tensors()["y"].clone()
    finally:
        prog.close()
    want = torch.matmul(x.double(), w.double().transpose(-1, -2))
    if dtype == "bf16":
        eager.assert_close(ours.reshape(want.shape), want.float(), 2e-2, 2e-2, "batched linear bf16 vs float64")
    else:
        eager.assert_close(ours.reshape(want.shape), want.float(), 1e-4, 1e-4 * float(want.pow(2).mean().sqrt()), "batched linear fp32 vs float64")


class _EagerAttention(nn.Module):
    """Attention spelled with matmuls, as a model without the fused op traces it."""

    def forward(self, q, k, v):
        s = torch.matmul(q, k.transpose(-1, -2)) * (1.0 / float(q.shape[-1]) ** 0.5)
        return torch.softmax(s, -1) @ v


class _Mm(nn.Module):
    def forward(self, a, b):
        return a @ b


@pytest.mark.gpu
@pytest.mark.parametrize("seq", [104, 100, 36])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_matmul_spelled_attention(device, dtype, seq):
    """``q @ k.T`` reads ``k`` as it lies (the transpose is a view whose reduction axis is contiguous); ``p @ v`` needs
    ``v`` transposed, which a copy nest does; both products are batched contractions over batch x heads."""
    torch.manual_seed(31)
    q, k, v = (torch.randn(2, 4, seq, 64).to(dtype) for _ in range(3))  # (a key count that is not whole 16-byte chunks: the second product's operands are padded)
    mod = _EagerAttention().eval()
    be = HipBackend()
    compiled = be.compile(trace_module(mod, (q, k, v)))
    names = [n.op.kernel_name.rsplit("_", 1)[0] for n in compiled.nodes.values() if isinstance(n.op, HipOp)]
    if dtype is torch.bfloat16:
        assert names == ["k_sdpa_reduce"]  # 16-bit: raised to the fused kernel
    else:
        assert names.count("k_matmul") == 2 and names.count("k_gather") == (1 if seq % 8 == 0 else 2) and "k_softmax_reduce" in names
    prog = be.program(compiled, dict(zip(compiled.inputs, (t.to(device) for t in (q, k, v)))))
    try:
        prog.run()
        torch.cuda.synchronize()
        ours = prog.output_tensors()[compiled.outputs[0]].clone()
    finally:
        prog.close()
    want = mod(q.double(), k.double(), v.double()).float()
    tol = (2e-2, 2e-2) if dtype is torch.bfloat16 else (1e-4, 1e-5)
    eager.assert_close(ours.reshape(want.shape), want, *tol, f"matmul-spelled attention {dtype}")


@pytest.mark.gpu
@pytest.mark.parametrize("shape_a, shape_b", [((70, 96), (96, 40)), ((3, 50, 64), (64, 72)), ((2, 3, 33, 32), (2, 3, 32, 48)), ((5, 19, 50), (50, 20))])
def test_plain_matmul(device, shape_a, shape_b):
    """``a @ b`` with ``b`` stored ``[K, N]``: shared by every product or one per product."""
    torch.manual_seed(32)
    a, b = torch.randn(*shape_a), 0.2 * torch.randn(*shape_b)
    be = HipBackend()
    compiled = be.compile(trace_module(_Mm().eval(), (a, b)))
    prog = be.program(compiled, dict(zip(compiled.inputs, (a.to(device), b.to(device)))))
    try:
        prog.run()
        torch.cuda.synchronize()
        ours = prog.output_tensors()[compiled.outputs[0]].clone()
    finally:
        prog.close()
    want = (a.double() @ b.double()).float()
    eager.assert_close(ours.reshape(want.shape), want, 1e-4, 1e-4 * float(want.pow(2).mean().sqrt()), f"matmul {shape_a} @ {shape_b}")


class _MmAdd(nn.Module):
    def forward(self, a, b, r):
        return torch.matmul(a, b) + r


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows, k, n", [(512, 2048, 1024), (32, 3072, 1024), (100, 64, 72), (7, 50, 20)])
def test_matmul_plus_residual_is_one_contraction(device, dtype, rows, k, n):
    """``a @ w + residual`` (the reference's ``matmul_add`` perf cases, tests/perf/cases.py:193-210): the residual is added in
    the contraction's output stage where the product is a single unpadded one (``k`` whole 8s, ``n`` whole 4s); other
    shapes keep the separate add.  Against float64."""
    torch.manual_seed(36)
    a, b, r = torch.randn(1, rows, k).to(dtype), (0.05 * torch.randn(k, n)).to(dtype), torch.randn(1, rows, n).to(dtype)
    be = HipBackend()
    compiled = be.compile(trace_module(_MmAdd().eval(), (a, b, r)))
    names = [nd.op.kernel_name.rsplit("_", 1)[0] for nd in compiled.nodes.values() if isinstance(nd.op, HipOp)]
    fused = k % 8 == 0 and n % 4 == 0
    assert ("k_pointwise_elementwise" not in names) == fused, names
    prog = be.program(compiled, dict(zip(compiled.inputs, (t.to(device) for t in (a, b, r)))))
    try:
        prog.run()
        torch.cuda.synchronize()
        ours = prog.output_tensors()[compiled.outputs[0]].clone()
    finally:
        prog.close()
    want = a.double() @ b.double() + r.double()
    tol = (2e-2, 2e-2) if dtype is torch.bfloat16 else (1e-4, 1e-4 * float(want.pow(2).mean().sqrt()))
    eager.assert_close(ours.reshape(want.shape).double(), want, *tol, f"matmul + residual {rows}x{k}x{n} {dtype}")


class _GatedMm(nn.Module):
    def __init__(self, act):
        super().__init__()
        self.act = act

    def forward(self, x, g, u):
        return self.act(torch.matmul(x, g)) * torch.matmul(x, u)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows", [512, 32, 50])
@pytest.mark.parametrize("act", ["silu", "gelu_tanh"])
def test_gated_matmul_pair_is_two_contractions(device, rows, act, dtype):
    """``act(x @ wg) * (x @ wu)`` on run-time operands (the reference's ``gated_mlp`` perf cases,
    tests/perf/cases.py:213-232): the activation of the gate product and the product with it ride in the up contraction's
    output stage — no element-wise launch; also where the contractions are split over workgroups (few rows).  Against float64."""
    fn = {"silu": torch.nn.functional.silu, "gelu_tanh": lambda t: torch.nn.functional.gelu(t, approximate="tanh")}[act]
    torch.manual_seed(37)
    x, g, u = torch.randn(1, rows, 1024).to(dtype), (0.03 * torch.randn(1024, 768)).to(dtype), (0.03 * torch.randn(1024, 768)).to(dtype)
    be = HipBackend()
    compiled = be.compile(trace_module(_GatedMm(fn).eval(), (x, g, u)))
    names = [nd.op.kernel_name.rsplit("_", 1)[0] for nd in compiled.nodes.values() if isinstance(nd.op, HipOp)]
    assert not any(nm.startswith("k_pointwise") for nm in names) and any(nm.startswith(f"k_matmul_{act}_mul") for nm in names), names
    prog = be.program(compiled, dict(zip(compiled.inputs, (t.to(device) for t in (x, g, u)))))
    try:
        prog.run()
        torch.cuda.synchronize()
        ours = prog.output_tensors()[compiled.outputs[0]].clone()
    finally:
        prog.close()
    want = fn(x.double() @ g.double()) * (x.double() @ u.double())
    tol = (2e-2, 2e-2 * float(want.pow(2).mean().sqrt())) if dtype is torch.bfloat16 else (1e-4, 1e-4 * float(want.pow(2).mean().sqrt()))
    eager.assert_close(ours.reshape(want.shape).double(), want, *tol, f"gated matmul pair, {rows} rows, {act}, {dtype}")


class _EagerMaskedAttention(nn.Module):
    def forward(self, q, k, v, mask):
        s = torch.matmul(q, k.transpose(-1, -2)) / float(q.shape[-1]) ** 0.5 + mask
        return torch.softmax(s, -1) @ v


@pytest.mark.gpu
@pytest.mark.parametrize("masked", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_matmul_spelled_attention_is_raised_to_the_fused_kernel(device, dtype, masked):
    """16-bit ``softmax(q @ k.T * scale [+ mask]) @ v`` becomes one attention kernel (what the reference reaches by
    decomposing the fused op and finding the streaming form again); fp32 keeps its matmuls — and a ``[1, 1, S, S]``
    mask broadcast into ``[B, H, S, S]`` goes through a dense copy."""
    torch.manual_seed(33)
    q, k, v = (torch.randn(2, 4, 200, 128).to(dtype) for _ in range(3))
    args = [q, k, v]
    mod = _EagerAttention().eval()
    if masked:
        args.append(causal_mask := torch.zeros(1, 1, 200, 200).masked_fill(torch.arange(200)[None, :] > torch.arange(200)[:, None], float("-inf")).to(dtype))
        mod = _EagerMaskedAttention().eval()
        assert causal_mask.shape == (1, 1, 200, 200)
    be = HipBackend()
    compiled = be.compile(trace_module(mod, tuple(args)))
    names = [n.op.kernel_name.rsplit("_", 1)[0] for n in compiled.nodes.values() if isinstance(n.op, HipOp)]
    if dtype is torch.bfloat16:
        assert names == ["k_sdpa_reduce"]
    else:
        assert names.count("k_matmul") == 2 and "k_sdpa_reduce" not in names
    prog = be.program(compiled, dict(zip(compiled.inputs, (t.to(device) for t in args))))
    try:
        prog.run()
        torch.cuda.synchronize()
        ours = prog.output_tensors()[compiled.outputs[0]].clone()
    finally:
        prog.close()
    want = mod(*(t.double() for t in args)).float()
    tol = (2e-2, 2e-2) if dtype is torch.bfloat16 else (1e-4, 1e-5)
    eager.assert_close(ours.reshape(want.shape), want, *tol, f"matmul-spelled attention {dtype} masked={masked}")


class _FusedAttention(nn.Module):
    def __init__(self, **kw):
        super().__init__()
        self.kw = kw

    def forward(self, q, k, v, mask=None):
        return torch.nn.functional.scaled_dot_product_attention(q, k, v, attn_mask=mask, **self.kw)


class _TokenMajorAttention(nn.Module):
    """Heads split from token-major projections and merged back, as a decoder block does around the fused op."""

    def forward(self, q, k, v):
        o = torch.nn.functional.scaled_dot_product_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), is_causal=True, enable_gqa=True)
        return o.transpose(1, 2).reshape(q.shape[0], q.shape[1], -1)


class _RepeatKvAttention(nn.Module):
    def forward(self, q, k, v):
        b, h, s, d = k.shape
        g = q.shape[1] // h
        k = k[:, :, None].expand(b, h, g, s, d).reshape(b, h * g, s, d)
        v = v[:, :, None].expand(b, h, g, s, d).reshape(b, h * g, s, d)
        return torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True)


_FP32_ATTENTION = {
    # the reference's fp32 perf cases: q [1, 16, S, 128], k / v [1, 8, S, 128], causal, grouped heads (tests/perf/cases.py:174-190)
    "perf_s32": (_FusedAttention(is_causal=True, enable_gqa=True), [(1, 16, 32, 128), (1, 8, 32, 128), (1, 8, 32, 128)], None),
    "perf_s128": (_FusedAttention(is_causal=True, enable_gqa=True), [(1, 16, 128, 128), (1, 8, 128, 128), (1, 8, 128, 128)], None),
    "perf_s512": (_FusedAttention(is_causal=True, enable_gqa=True), [(1, 16, 512, 128), (1, 8, 512, 128), (1, 8, 512, 128)], None),
    "perf_s2048": (_FusedAttention(is_causal=True, enable_gqa=True), [(1, 16, 2048, 128), (1, 8, 2048, 128), (1, 8, 2048, 128)], None),
    "ragged_keys": (_FusedAttention(), [(2, 4, 100, 64), (2, 4, 100, 64), (2, 4, 100, 64)], None),
    "ragged_everything": (_FusedAttention(is_causal=True), [(1, 2, 33, 21), (1, 2, 33, 21), (1, 2, 33, 21)], None),
    "cross_gqa": (_FusedAttention(enable_gqa=True, scale=0.2), [(1, 4, 50, 40), (1, 2, 70, 40), (1, 2, 70, 40)], None),
    "cross_causal_more_keys": (_FusedAttention(is_causal=True), [(2, 3, 45, 32), (2, 3, 150, 32), (2, 3, 150, 32)], None),
    "cross_causal_more_queries": (_FusedAttention(is_causal=True), [(1, 3, 150, 32), (1, 3, 45, 32), (1, 3, 45, 32)], None),
    "one_query_long_cache": (_FusedAttention(enable_gqa=True), [(2, 8, 1, 128), (2, 2, 1000, 128), (2, 2, 1000, 128)], None),
    "head_dim_256": (_FusedAttention(is_causal=True), [(1, 3, 200, 256)] * 3, None),
    "head_dim_3": (_FusedAttention(), [(1, 2, 70, 3)] * 3, None),
    "mask_1_1_s_s": (_FusedAttention(), [(2, 3, 72, 64)] * 3, lambda: torch.zeros(72, 72).masked_fill(torch.arange(72)[None, :] > torch.arange(72)[:, None], float("-inf"))[None, None]),
    "mask_per_batch_keys": (_FusedAttention(), [(2, 4, 40, 32)] * 3, lambda: torch.randn(2, 1, 1, 40)),
    "mask_full_odd_keys": (_FusedAttention(), [(2, 2, 37, 20), (2, 2, 51, 20), (2, 2, 51, 20)], lambda: torch.randn(2, 2, 37, 51)),
    "mask_s_s": (_FusedAttention(), [(1, 2, 64, 16)] * 3, lambda: torch.randn(64, 64)),
    "token_major": (_TokenMajorAttention(), [(1, 128, 16, 128), (1, 128, 8, 128), (1, 128, 8, 128)], None),
    "repeat_kv": (_RepeatKvAttention(), [(2, 8, 64, 64), (2, 2, 64, 64), (2, 2, 64, 64)], None),
}


@pytest.mark.gpu
@pytest.mark.parametrize("case", sorted(_FP32_ATTENTION))
def test_fp32_attention_streams_on_fp32_atoms(device, case):
    """The fused attention op on fp32 operands (what the reference's perf suite runs) is one streaming kernel on fp32 MFMA
    atoms — no scores in device memory — for every head_dim up to 256, ragged lengths, grouped heads, causal masks with
    unequal lengths (top-left aligned, as eager's) and additive masks of every broadcast form; against eager in float64."""
    mod, shapes, mask = _FP32_ATTENTION[case]
    torch.manual_seed(41)
    args = [torch.randn(*s) for s in shapes] + ([mask()] if mask else [])
    be = HipBackend()
    compiled = be.compile(trace_module(mod.eval(), tuple(args)))
    names = [n.op.kernel_name.rsplit("_", 1)[0] for n in compiled.nodes.values() if isinstance(n.op, HipOp)]
    assert names.count("k_sdpa_reduce") == 1 and "k_batched_linear" not in names, names
    prog = be.program(compiled, dict(zip(compiled.inputs, (t.to(device) for t in args))))
    try:
        prog.run()
        torch.cuda.synchronize()
        ours = prog.output_tensors()[compiled.outputs[0]].clone()
    finally:
        prog.close()
    want = mod(*(t.double() for t in args)).float()
    eager.assert_close(ours.reshape(want.shape), want, 1e-4, 1e-5, f"fp32 attention {case}")


@pytest.mark.gpu
@pytest.mark.parametrize("form", ["w1", "w2", "w4", "s2", "s4", "s8", "s2/sp", "s4/sp", "s8/sp", "s2/o", "s4/o", "s8/o"])
def test_fp32_attention_forms(device, form, monkeypatch):
    """``EMMY_FLASH=f32/w<n>``: 1, 2 or 4 of a workgroup's four waves own query rows and share the staged K / V blocks;
    ``f32/s<k>``: the k waves of a workgroup split the key blocks of one row group and stage for themselves.  Here with a
    last query block that is partly empty, keys that end inside a block, grouped heads and an additive mask."""
    monkeypatch.setenv("EMMY_FLASH", f"f32/{form}")
    torch.manual_seed(43)
    for mod, args in (
        (_FusedAttention(is_causal=True, enable_gqa=True), [torch.randn(2, 4, 300, 64), torch.randn(2, 2, 300, 64), torch.randn(2, 2, 300, 64)]),
        (_FusedAttention(enable_gqa=True), [torch.randn(1, 4, 70, 64), torch.randn(1, 2, 333, 64), torch.randn(1, 2, 333, 64), torch.randn(1, 4, 70, 333)]),
    ):
        be = HipBackend()
        compiled = be.compile(trace_module(mod.eval(), tuple(args)))
        (op,) = [n.op for n in compiled.nodes.values() if isinstance(n.op, HipOp)]
        assert op.knobs["FLASH"] == f"f32/{form}"
        prog = be.program(compiled, dict(zip(compiled.inputs, (t.to(device) for t in args))))
        try:
            prog.run()
            torch.cuda.synchronize()
            ours = prog.output_tensors()[compiled.outputs[0]].clone()
        finally:
            prog.close()
        want = mod(*(t.double() for t in args)).float()
        eager.assert_close(ours.reshape(want.shape), want, 1e-4, 1e-5, f"fp32 attention {form}")


@pytest.mark.gpu
@pytest.mark.parametrize("masked", [False, True])
def test_fp32_attention_with_a_runtime_sequence_length(device, masked):
    """One compilation of fp32 attention (causal, or with a ``[1, 1, S, S]`` additive mask whose row stride follows the
    length) with the sequence length as the kernel's trailing ``int``, bound at several lengths (ragged blocks, one key
    block, more blocks than waves), against eager in float64."""
    mod = _FusedAttention(enable_gqa=True) if masked else _FusedAttention(is_causal=True, enable_gqa=True)
    torch.manual_seed(47)

    def mk(s):
        qkv = [torch.randn(1, 4, s, 128), torch.randn(1, 2, s, 128), torch.randn(1, 2, s, 128)]
        if masked:
            m = torch.randn(1, 1, s, s)
            m[torch.rand(1, 1, s, s) < 0.3] = -float("inf")
            m[..., 0] = 0.5
            qkv.append(m)
        return qkv

    dyn = {"q": {2: "s"}, "k": {2: "s"}, "v": {2: "s"}, **({"mask": {2: "s", 3: "s"}} if masked else {})}
    be = HipBackend()
    compiled = be.compile(trace_module(mod.eval(), tuple(mk(64)), dynamic_shapes=dyn))
    (op,) = [n.op for n in compiled.nodes.values() if isinstance(n.op, HipOp)]
    assert op.runtime_args and op.knobs["FLASH"].startswith("f32/s")
    for s in (64, 1, 31, 200, 513):
        args = mk(s)
        prog = be.program(compiled, dict(zip(compiled.inputs, (t.to(device) for t in args))))
        try:
            prog.run()
            torch.cuda.synchronize()
            ours = prog.output_tensors()[compiled.outputs[0]].clone()
        finally:
            prog.close()
        want = mod(*(t.double() for t in args)).float()
        eager.assert_close(ours.reshape(want.shape), want, 1e-4, 1e-5, f"fp32 attention, runtime length {s}, masked={masked}")


@pytest.mark.gpu
@pytest.mark.parametrize("q_len, kv_len", [(1, 32768), (16, 4096), (7, 5000), (40, 2100)])
def test_fp32_decode_attention_splits_the_keys_across_workgroups(device, q_len, kv_len):
    """Decode-size fp32 queries over a long cache (no mask): the keys are split over workgroups as well — the partial
    kernel leaves each slice's ``(O, m, l)`` in a workspace and the combine kernel merges them (``REDUCE=g<n>k``, the
    form the 16-bit kernel has) — ragged last slices and grouped heads included; against eager in float64."""
    mod = _FusedAttention(enable_gqa=True)
    torch.manual_seed(53)
    args = [torch.randn(1, 16, q_len, 128), torch.randn(1, 8, kv_len, 128), torch.randn(1, 8, kv_len, 128)]
    be = HipBackend()
    compiled = be.compile(trace_module(mod.eval(), tuple(args)))
    names = [n.op.kernel_name.rsplit("_", 1)[0] for n in compiled.nodes.values() if isinstance(n.op, HipOp)]
    assert sorted(names) == ["k_sdpa_reduce_combine", "k_sdpa_reduce_partial"], names
    prog = be.program(compiled, dict(zip(compiled.inputs, (t.to(device) for t in args))))
    try:
        for _ in range(2):
            prog.run()
            torch.cuda.synchronize()
        ours = prog.output_tensors()[compiled.outputs[0]].clone()
    finally:
        prog.close()
    want = mod(*(t.double() for t in args)).float()
    eager.assert_close(ours.reshape(want.shape), want, 1e-4, 1e-5, f"fp32 decode attention q={q_len} kv={kv_len}")


@pytest.mark.gpu
def test_fp32_attention_key_split_across_workgroups_by_pin(device, monkeypatch):
    """``EMMY_REDUCE=g4k`` on a non-causal fp32 attention that would not split by itself, with a batch and a ragged length;
    a causal one ignores the pin."""
    monkeypatch.setenv("EMMY_REDUCE", "g4k")
    torch.manual_seed(54)
    for causal in (False, True):
        mod = _FusedAttention(is_causal=causal, enable_gqa=True)
        args = [torch.randn(2, 4, 100, 64), torch.randn(2, 2, 1100, 64), torch.randn(2, 2, 1100, 64)]
        be = HipBackend()
        compiled = be.compile(trace_module(mod.eval(), tuple(args)))
        names = [n.op.kernel_name.rsplit("_", 1)[0] for n in compiled.nodes.values() if isinstance(n.op, HipOp)]
        assert (sorted(names) == ["k_sdpa_reduce_combine", "k_sdpa_reduce_partial"]) == (not causal), names
        prog = be.program(compiled, dict(zip(compiled.inputs, (t.to(device) for t in args))))
        try:
            prog.run()
            torch.cuda.synchronize()
            ours = prog.output_tensors()[compiled.outputs[0]].clone()
        finally:
            prog.close()
        want = mod(*(t.double() for t in args)).float()
        eager.assert_close(ours.reshape(want.shape), want, 1e-4, 1e-5, f"fp32 attention g4k causal={causal}")


_NARROW_ON_FP32_ATOMS = {
    # 16-bit rows that are not whole 16-byte chunks (the 16-bit flash kernel pads whole chunks only)
    "bf16_head_dim_36": (_FusedAttention(is_causal=True), torch.bfloat16, [(2, 4, 64, 36)] * 3, None),
    "bf16_head_dim_100": (_FusedAttention(), torch.bfloat16, [(2, 4, 50, 100)] * 3, None),
    "fp16_head_dim_20_gqa_mask": (_FusedAttention(enable_gqa=True), torch.float16, [(2, 4, 70, 20), (2, 2, 90, 20), (2, 2, 90, 20)], lambda: torch.randn(2, 1, 70, 90)),
    "bf16_head_dim_250_causal": (_FusedAttention(is_causal=True), torch.bfloat16, [(1, 2, 130, 250)] * 3, None),
}


@pytest.mark.gpu
@pytest.mark.parametrize("case", sorted(_NARROW_ON_FP32_ATOMS))
def test_16_bit_attention_with_rows_that_are_not_whole_chunks_streams_on_fp32_atoms(device, case):
    """16-bit attention whose head_dim is not a multiple of 8 takes the streaming kernel on fp32 atoms (operands converted
    as they are staged, probabilities kept in fp32): one launch, no scores in device memory; against eager in float64."""
    mod, dtype, shapes, mask = _NARROW_ON_FP32_ATOMS[case]
    torch.manual_seed(41)
    args = [torch.randn(*s).to(dtype) for s in shapes] + ([mask().to(dtype)] if mask else [])
    be = HipBackend()
    compiled = be.compile(trace_module(mod.eval(), tuple(args)))
    (op,) = [n.op for n in compiled.nodes.values() if isinstance(n.op, HipOp)]
    assert op.kernel_name.startswith("k_sdpa_reduce") and op.knobs["FLASH"].startswith("f32/w")
    prog = be.program(compiled, dict(zip(compiled.inputs, (t.to(device) for t in args))))
    try:
        prog.run()
        torch.cuda.synchronize()
        ours = prog.output_tensors()[compiled.outputs[0]].clone()
    finally:
        prog.close()
    want = mod(*(t.double() for t in args)).float()
    eager.assert_close(ours.float().reshape(want.shape), want, 2e-2, 2e-2, f"16-bit attention on fp32 atoms {case}")


_DECOMPOSED_ATTENTION = {
    # head dims beyond the streaming kernels' registers, value rows of another length than the keys', a mask without a key axis
    "bf16_head_dim_320": (_FusedAttention(is_causal=True), torch.bfloat16, [(1, 2, 48, 320)] * 3, None),
    "fp32_head_dim_320": (_FusedAttention(is_causal=True), torch.float32, [(1, 2, 48, 320)] * 3, None),
    "fp32_value_rows_24": (_FusedAttention(), torch.float32, [(1, 2, 40, 16), (1, 2, 56, 16), (1, 2, 56, 24)], None),
    "fp32_column_mask": (_FusedAttention(), torch.float32, [(2, 2, 40, 32)] * 3, lambda: torch.randn(2, 1, 40, 1)),
}


@pytest.mark.gpu
@pytest.mark.parametrize("case", sorted(_DECOMPOSED_ATTENTION))
def test_attention_outside_the_flash_kernel(device, case):
    """The fused attention op in shapes no streaming kernel takes: two batched MFMA contractions (fp32 atoms keep fp32
    accuracy) around loop-nest stages, against eager in float64."""
    mod, dtype, shapes, mask = _DECOMPOSED_ATTENTION[case]
    torch.manual_seed(41)
    args = [torch.randn(*s).to(dtype) for s in shapes] + ([mask().to(dtype)] if mask else [])
    be = HipBackend()
    compiled = be.compile(trace_module(mod.eval(), tuple(args)))
    names = [n.op.kernel_name.rsplit("_", 1)[0] for n in compiled.nodes.values() if isinstance(n.op, HipOp)]
    assert names.count("k_batched_linear") == 2 and "k_sdpa_reduce" not in names
    prog = be.program(compiled, dict(zip(compiled.inputs, (t.to(device) for t in args))))
    try:
        prog.run()
        torch.cuda.synchronize()
        ours = prog.output_tensors()[compiled.outputs[0]].clone()
    finally:
        prog.close()
    want = mod(*(t.double() for t in args)).float()
    tol = (2e-2, 2e-2) if dtype is torch.bfloat16 else (1e-4, 1e-5)
    eager.assert_close(ours.reshape(want.shape), want, *tol, f"decomposed attention {case}")


@pytest.mark.gpu
@pytest.mark.parametrize("seq", [128, 40])
def test_c5_qwen3_block_in_fp32(device, seq):
    """The decoder block with fp32 parameters and activations — the only precision the reference compiles
    (tests/perf/cases.py:20-23).  The fused forms written for 16-bit tiles (norm prologue, gate/up pair, head-norm +
    rotary epilogue) stand down: plain fp32-atom contractions, row kernels and the fp32 streaming attention kernel;
    against the module in float64."""
    import copy

    case = eager.qwen3_block_case(seq=seq, dtype=torch.float32, norm_std=0.1, seed=5)
    ours, want, compiled = run_case(case, device)
    names = [n.op.kernel_name.rsplit("_", 1)[0] for n in compiled.nodes.values() if isinstance(n.op, HipOp)]
    assert names.count("k_sdpa_reduce") == 1 and "k_batched_linear" not in names
    with torch.no_grad():
        exact = copy.deepcopy(case.module).cpu().double()(*(t.double() for t in case.inputs))
    exact = (exact[0] if isinstance(exact, tuple) else exact).float()
    scale = float(exact.pow(2).mean().sqrt())
    eager.assert_close(ours.cpu(), exact.reshape(ours.shape), 1e-4, 1e-4 * scale, f"fp32 block S={seq} vs float64")
    eager.assert_close(ours, want, 1e-4, 1e-4 * scale, f"fp32 block S={seq} vs eager fp32 (GPU)")


_COPIES = {
    # name: (source shape, dtype, result-order of the source axes, pad rows to, pad last to)
    "transpose_2d": ((1024, 2048), torch.float32, (1, 0), None, None),
    "transpose_ragged_padded": ((100, 37), torch.float32, (1, 0), 40, 104),
    "batched_transpose_bf16": ((6, 70, 130), torch.bfloat16, (0, 2, 1), 132, 72),
    "heads_to_tokens": ((16, 128, 64), torch.float32, (1, 0, 2), None, None),
    "rows_padded": ((5, 33, 50), torch.float32, (0, 1, 2), 36, 56),
    "unit_axis_in_the_middle": ((7, 65, 3), torch.float32, (2, 0, 1), None, None),
    "one_column": ((300, 1), torch.float32, (1, 0), None, None),
}


@pytest.mark.gpu
@pytest.mark.parametrize("case", sorted(_COPIES))
def test_strided_copy(device, case):
    """The layout-change kernel (rows written as they lie, or 64 x 64 tiles transposed through LDS) against torch's
    ``permute`` + zero padding: bit-exact, it moves values."""
    from deplodock_amd.dtype import from_torch
    from deplodock_amd.ir.tile import StridedCopy

    shape, dtype, order, pad_rows, pad_last = _COPIES[case]
    torch.manual_seed(51)
    # a window of a larger buffer, so offset and strides are not the dense ones
    big = torch.randn(*(d + 3 for d in shape)).to(dtype)
    view = big[tuple(slice(2, 2 + d) for d in shape)]
    axes = [[shape[i], shape[i], view.stride(i)] for i in order]
    if pad_last:
        axes[-1][0] = pad_last
    if pad_rows:
        axes[-2][0] = pad_rows
    out_shape = tuple(a[0] for a in axes)
    dt = from_torch(dtype)
    body = StridedCopy(src="X", out="out", dtype=dt, src_offset=view.storage_offset(), src_numel=big.numel(), axes=tuple(tuple(a) for a in axes))
    g = Graph()
    g.add_input("X", (big.numel(),), dt)
    g.add_node(TileOp(name="k_gather", body=body), ["X"], Tensor("out", out_shape, dt))
    g.outputs = ["out"]
    be = HipBackend()
    compiled = lower(g)
    prog = be.program(compiled, {"X": big.reshape(-1).to(device)})
    try:
        prog.run()
        torch.cuda.synchronize()
        ours = prog.output_tensors()["out"].clone().cpu()
    finally:
        prog.close()
    want = torch.zeros(out_shape, dtype=dtype)
    want[tuple(slice(0, shape[i]) for i in order)] = view.permute(*order)
    assert torch.equal(ours.reshape(out_shape).view(torch.int16 if dtype is torch.bfloat16 else torch.int32), want.view(torch.int16 if dtype is torch.bfloat16 else torch.int32))


class _Fn(nn.Module):
    def __init__(self, fn):
        super().__init__()
        self.fn = fn

    def forward(self, *args):
        return self.fn(*args)


class _GemmaNorm(nn.Module):
    """Gemma's RMSNorm: computed in fp32, scaled by ``1 + weight``, cast back last."""

    def __init__(self, dim: int):
        super().__init__()
        self.weight = nn.Parameter(0.1 * torch.randn(dim))

    def forward(self, t):
        f = t.float()
        out = f * torch.rsqrt(f.pow(2).mean(-1, keepdim=True) + 1e-6)
        return (out * (1.0 + self.weight.float())).type_as(t)


def _op_cases():
    Fn = torch.nn.functional
    x = lambda *s: torch.randn(*s)  # noqa: E731
    return {
        # element-wise ops of the reference's tracer (emmy/compiler/trace/torch.py:489-503)
        "gelu": (_Fn(Fn.gelu), lambda: (x(4, 33, 250),)),
        "gelu_tanh": (_Fn(lambda t: Fn.gelu(t, approximate="tanh")), lambda: (x(4, 33, 250),)),
        "erf": (_Fn(torch.erf), lambda: (x(3, 100),)),
        "relu": (_Fn(Fn.relu), lambda: (x(3, 100),)),
        "pow3": (_Fn(lambda t: t.pow(3)), lambda: (x(3, 100),)),
        "pow2_5": (_Fn(lambda t: t.abs().pow(2.5)), lambda: (x(3, 100),)),
        "addmm": (_Fn(lambda b, a, w: torch.addmm(b, a, w)), lambda: (x(64), x(40, 128), 0.2 * x(128, 64))),
        "t": (_Fn(lambda a, w: a @ w.t()), lambda: (x(32, 128), 0.2 * x(64, 128))),
        # reductions over any axis, amax
        "amax": (_Fn(lambda t: t.amax(-1)), lambda: (x(4, 32, 300),)),
        "amax_keep": (_Fn(lambda t: t.amax(-1, keepdim=True)), lambda: (x(4, 32, 300),)),
        "amax_axis1": (_Fn(lambda t: t.amax(1)), lambda: (x(4, 70, 36),)),
        "sum_axis1": (_Fn(lambda t: t.sum(1)), lambda: (x(4, 70, 36),)),
        "mean_axis0_keep": (_Fn(lambda t: t.mean(0, keepdim=True)), lambda: (x(5, 9, 40),)),
        "softmax_axis1": (_Fn(lambda t: torch.softmax(t, 1) * 2), lambda: (x(4, 70, 36),)),
        "softmax_axis0": (_Fn(lambda t: torch.softmax(t, 0)), lambda: (x(6, 9, 40),)),
        # layer norm, embedding, index_select, cat
        "layer_norm": (nn.LayerNorm(256), lambda: (3 + 2 * x(4, 33, 256),)),
        "layer_norm_plain": (nn.LayerNorm(200, elementwise_affine=False), lambda: (x(7, 200),)),
        "layer_norm_no_bias": (nn.LayerNorm(96, bias=False), lambda: (x(2, 5, 96),)),
        "embedding": (nn.Embedding(100, 64), lambda: (torch.randint(0, 100, (4, 16)),)),
        "index_select": (_Fn(lambda t, i: t.index_select(1, i)), lambda: (x(4, 32, 24), torch.tensor([1, 31, 7, 7, 0]))),
        "cat_last": (_Fn(lambda a, b: torch.cat([a, b], -1)), lambda: (x(4, 32, 24), x(4, 32, 40))),
        "cat_first": (_Fn(lambda a, b: torch.cat([a, b * 2], 0)), lambda: (x(3, 8, 24), x(5, 8, 24))),
        "cat_three_slices": (_Fn(lambda a, b: torch.cat([a[..., :10], b, a[..., 5:9]], -1)), lambda: (x(4, 32, 24), x(4, 32, 7))),
        "rotate_half": (_Fn(lambda t: torch.cat((-t[..., 64:], t[..., :64]), -1)), lambda: (x(2, 8, 50, 128),)),
        # normalisations spelled out with keepdim reductions: one fused row kernel each
        "gemma_rms_norm": (_GemmaNorm(256), lambda: (x(4, 33, 256),)),
        "manual_layer_norm": (_Fn(lambda t: (t - t.mean(-1, keepdim=True)) * torch.rsqrt((t - t.mean(-1, keepdim=True)).pow(2).mean(-1, keepdim=True) + 1e-5)), lambda: (2 + x(5, 40, 200),)),
        "shift_by_row_max": (_Fn(lambda t: torch.exp(t - t.amax(-1, keepdim=True))), lambda: (3 * x(6, 300),)),
        "residual_plus_norm": (_Fn(lambda t, r: r + t * torch.rsqrt(t.pow(2).mean(-1, keepdim=True) + 1e-6)), lambda: (x(4, 33, 256), x(4, 33, 256))),
        # what an embedding model does after its last layer: pick the last token, normalise to unit length
        "normalize": (_Fn(lambda t: Fn.normalize(t, p=2, dim=-1)), lambda: (x(4, 33, 256),)),
        "last_token_normalize": (_Fn(lambda t: Fn.normalize(t[:, -1], p=2, dim=1)), lambda: (x(4, 33, 256),)),
        "select": (_Fn(lambda t: t[:, 5] * 2), lambda: (x(4, 33, 40),)),
        "clamp": (_Fn(lambda t: t.clamp(-0.5, 0.7)), lambda: (x(3, 100),)),
        "clamp_min": (_Fn(lambda t: t.clamp_min(0.1) * 2), lambda: (x(3, 100),)),
        "vector_norm_axis1": (_Fn(lambda t: torch.linalg.vector_norm(t, dim=1)), lambda: (x(4, 33, 40),)),
        # an output width that is not whole runs of four columns (a 151 669-word vocabulary in small): padded weight, windowed result
        "linear_odd_width": (nn.Linear(64, 37, bias=False), lambda: (x(5, 9, 64),)),
        "linear_odd_width_then_softmax": (nn.Sequential(nn.Linear(64, 37, bias=False), nn.Softmax(-1)), lambda: (x(21, 64),)),
        # a transformer MLP of the GELU family, and a pre-norm projection
        "gelu_mlp": (nn.Sequential(nn.Linear(256, 512), nn.GELU(), nn.Linear(512, 256)), lambda: (x(2, 48, 256),)),
        "layer_norm_linear": (nn.Sequential(nn.LayerNorm(256), nn.Linear(256, 128)), lambda: (x(4, 33, 256),)),
    }


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", sorted(_op_cases()))
def test_frontend_op_coverage(device, case, dtype):
    """Every op the reference's tracer accepts that is not part of the five benchmark configurations, through trace
    -> compile -> run, against the module in float64 (fp32: 1e-4 of the output's RMS; bf16: rtol 2e-2)."""
    import copy

    torch.manual_seed(61)
    mod, make = _op_cases()[case]
    args = tuple(t.to(dtype) if t.is_floating_point() else t for t in make())
    mod = copy.deepcopy(mod).to(dtype).eval()
    be = HipBackend()
    compiled = be.compile(trace_module(mod, args))
    prog = be.program(compiled, dict(zip(compiled.inputs, (t.to(device) for t in args))))
    try:
        prog.run()
        torch.cuda.synchronize()
        ours = prog.output_tensors()[compiled.outputs[0]].clone().cpu()
    finally:
        prog.close()
    with torch.no_grad():
        want = copy.deepcopy(mod).double()(*(t.double() if t.is_floating_point() else t for t in args)).float()
    rms = float(want.pow(2).mean().sqrt())
    rtol, atol = (1e-4, 1e-4 * max(rms, 1e-3)) if dtype is torch.float32 else (2e-2, 2e-2 * max(rms, 1.0))
    if case in ("embedding", "index_select", "cat_last", "cat_first", "rotate_half") and dtype is torch.float32:
        assert torch.equal(ours.reshape(want.shape), want) or case == "cat_first"  # pure data movement is exact
    eager.assert_close(ours.reshape(want.shape).float(), want, rtol, atol, f"{case} {dtype}")


class _FirstOutput(nn.Module):
    def __init__(self, inner):
        super().__init__()
        self.inner = inner

    def forward(self, x):
        out = self.inner(x)
        return out[0] if isinstance(out, tuple) else out


def _gpt2_block():
    from transformers import GPT2Config
    from transformers.models.gpt2.modeling_gpt2 import GPT2Block

    cfg = GPT2Config(n_embd=256, n_head=4, n_layer=1, n_positions=128)
    cfg._attn_implementation = "sdpa"
    return _FirstOutput(GPT2Block(cfg, 0))


def _bert_layer():
    from transformers import BertConfig
    from transformers.models.bert.modeling_bert import BertLayer

    cfg = BertConfig(hidden_size=256, num_attention_heads=4, intermediate_size=1024, num_hidden_layers=1)
    cfg._attn_implementation = "sdpa"
    return _FirstOutput(BertLayer(cfg))


class _RotaryLayer(nn.Module):
    def __init__(self, layer):
        super().__init__()
        self.layer = layer

    def forward(self, x, cos, sin):
        out = self.layer(x, position_embeddings=(cos, sin), attention_mask=None)
        return out[0] if isinstance(out, tuple) else out


_DECODER_FAMILIES = {
    "llama": ("LlamaConfig", "LlamaDecoderLayer", "LlamaRotaryEmbedding", {}),
    "mistral": ("MistralConfig", "MistralDecoderLayer", "MistralRotaryEmbedding", {}),
    "qwen2": ("Qwen2Config", "Qwen2DecoderLayer", "Qwen2RotaryEmbedding", {}),
    "gemma": ("GemmaConfig", "GemmaDecoderLayer", "GemmaRotaryEmbedding", {"head_dim": 64}),
    "gemma2": ("Gemma2Config", "Gemma2DecoderLayer", "Gemma2RotaryEmbedding", {"head_dim": 64}),
    "phi3": ("Phi3Config", "Phi3DecoderLayer", "Phi3RotaryEmbedding", {}),
    "olmo2": ("Olmo2Config", "Olmo2DecoderLayer", "Olmo2RotaryEmbedding", {}),
}


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("family", sorted(_DECODER_FAMILIES))
def test_decoder_layers_of_other_families(device, family, dtype):
    """One decoder layer of each family as ``transformers`` builds it (hidden 512, 8 query / 4 KV heads, 64 tokens,
    random weights): the norm variants (Gemma's ``1 + w`` in fp32, OLMo-2's norm after the projection and on q / k),
    fused qkv + ``chunk`` (Phi-3), biased projections (Qwen-2), GeGLU — against the module in float64."""
    import copy
    import importlib

    cfg_name, layer_name, rotary_name, extra = _DECODER_FAMILIES[family]
    modeling = importlib.import_module(f"transformers.models.{family}.modeling_{family}")
    cfg = getattr(importlib.import_module(f"transformers.models.{family}.configuration_{family}"), cfg_name)(
        hidden_size=512, num_attention_heads=8, num_key_value_heads=4, intermediate_size=1024, num_hidden_layers=1, vocab_size=1000, pad_token_id=0, eos_token_id=1, bos_token_id=2, **extra)  # fmt: skip
    cfg._attn_implementation = "sdpa"
    torch.manual_seed(72)
    layer = getattr(modeling, layer_name)(cfg, 0)
    with torch.no_grad():
        for name, p in layer.named_parameters():
            p.copy_((0.1 if "gemma" in family else 1.0) + 0.1 * torch.randn_like(p) if "norm" in name else 0.04 * torch.randn_like(p))
    x = torch.randn(1, 64, 512)
    cos, sin = getattr(modeling, rotary_name)(cfg)(x, torch.arange(64)[None])
    mod = _RotaryLayer(layer).to(dtype).eval()
    args = tuple(t.to(dtype) for t in (x, cos, sin))
    be = HipBackend()
    compiled = be.compile(trace_module(mod, args))
    prog = be.program(compiled, dict(zip(compiled.inputs, (t.to(device) for t in args))))
    try:
        prog.run()
        torch.cuda.synchronize()
        ours = prog.output_tensors()[compiled.outputs[0]].clone().cpu()
    finally:
        prog.close()
    with torch.no_grad():
        want = copy.deepcopy(mod).double()(*(t.double() for t in args)).float()
        half = copy.deepcopy(mod)(*args).float()
    rms = float(want.pow(2).mean().sqrt())
    if dtype is torch.float32:
        eager.assert_close(ours.reshape(want.shape), want, 1e-4, 1e-4 * rms, f"{family} layer fp32 vs float64")
    else:
        eager.assert_close(ours.reshape(want.shape).float(), want, 2e-2, 4e-2 * max(rms, 1.0), f"{family} layer bf16 vs float64")
        eager.assert_mean_error_within_baseline(ours.reshape(want.shape).float(), half, want, 1.5, f"{family} layer bf16: mean error against eager bf16's")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("family", ["gpt2", "bert"])
def test_layers_of_other_model_families(device, family, dtype):
    """A GPT-2 block (LayerNorm, Conv1D = ``addmm`` over ``[K, N]`` parameters, ``split``, tanh-GELU spelled out,
    causal attention) and a BERT layer (LayerNorm after the residual, erf-GELU, biased projections, inference
    dropout) as ``transformers`` builds them: against the module in float64."""
    import copy

    torch.manual_seed(71)
    mod = (_gpt2_block if family == "gpt2" else _bert_layer)()
    with torch.no_grad():
        for name, p in mod.named_parameters():
            p.copy_(1 + 0.1 * torch.randn_like(p) if ("ln" in name.lower() or "norm" in name.lower()) and name.endswith("weight") else 0.05 * torch.randn_like(p))
    mod = mod.to(dtype).eval()
    x = torch.randn(2, 64, 256).to(dtype)
    be = HipBackend()
    compiled = be.compile(trace_module(mod, (x,)))
    names = [n.op.kernel_name.rsplit("_", 1)[0] for n in compiled.nodes.values() if isinstance(n.op, HipOp)]
    assert "k_layer_norm_reduce" in names
    if family == "gpt2":
        assert names[1].startswith("k_linear")  # the Conv1D weight is transposed at bind time: no copy kernel in front of the projection
    if dtype is torch.bfloat16:
        assert names.count("k_sdpa_reduce") == 1 and names.count("k_linear_add") == 2
    prog = be.program(compiled, {compiled.inputs[0]: x.to(device)})
    try:
        prog.run()
        torch.cuda.synchronize()
        ours = prog.output_tensors()[compiled.outputs[0]].clone().cpu()
    finally:
        prog.close()
    with torch.no_grad():
        want = copy.deepcopy(mod).double()(x.double()).float()
        half = copy.deepcopy(mod)(x).float()  # what eager makes of it in the same precision
    rms = float(want.pow(2).mean().sqrt())
    if dtype is torch.float32:
        eager.assert_close(ours.reshape(want.shape), want, 1e-4, 1e-4 * rms, f"{family} fp32 vs float64")
    else:
        eager.assert_close(ours.reshape(want.shape).float(), want, 2e-2, 4e-2 * max(rms, 1.0), f"{family} bf16 vs float64")
        eager.assert_mean_error_within_baseline(ours.reshape(want.shape).float(), half, want, 1.5, f"{family} bf16: mean error against eager bf16's")


class _Logits(nn.Module):
    def __init__(self, model):
        super().__init__()
        self.model = model

    def forward(self, ids):
        out = self.model(input_ids=ids)
        return out.logits if hasattr(out, "logits") else out.last_hidden_state


def _small_model(family: str):
    import transformers as tf

    common = dict(vocab_size=1000, pad_token_id=0, eos_token_id=1, bos_token_id=2)
    if family == "llama":
        cfg, cls = tf.LlamaConfig(hidden_size=256, num_attention_heads=4, num_key_value_heads=2, intermediate_size=512, num_hidden_layers=2, **common), tf.LlamaForCausalLM
    elif family == "qwen3":
        cfg, cls = tf.Qwen3Config(hidden_size=256, num_attention_heads=4, num_key_value_heads=2, head_dim=64, intermediate_size=512, num_hidden_layers=2, **common), tf.Qwen3Model
    elif family == "gpt2":
        cfg, cls = tf.GPT2Config(n_embd=256, n_head=4, n_layer=2, n_positions=128, vocab_size=1000, bos_token_id=2, eos_token_id=1), tf.GPT2LMHeadModel
    elif family == "bert":
        cfg, cls = tf.BertConfig(hidden_size=256, num_attention_heads=4, intermediate_size=1024, num_hidden_layers=2, vocab_size=1000, pad_token_id=0), (lambda c_: tf.BertModel(c_, add_pooling_layer=False))
    else:
        cfg_name, cls_name, extra = _MORE_CAUSAL_LMS[family]
        cfg = getattr(tf, cfg_name)(hidden_size=256, num_attention_heads=4, num_key_value_heads=2, intermediate_size=512, num_hidden_layers=2, **extra, **common)
        cls = getattr(tf, cls_name)
    cfg._attn_implementation = "sdpa"
    return cls(cfg)


_MORE_CAUSAL_LMS = {
    "mistral": ("MistralConfig", "MistralForCausalLM", {}),
    "qwen2": ("Qwen2Config", "Qwen2ForCausalLM", {}),
    "gemma": ("GemmaConfig", "GemmaForCausalLM", {"head_dim": 64}),
    "gemma2": ("Gemma2Config", "Gemma2ForCausalLM", {"head_dim": 64}),
    "phi3": ("Phi3Config", "Phi3ForCausalLM", {}),
    "olmo2": ("Olmo2Config", "Olmo2ForCausalLM", {}),
}


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("family", ["llama", "qwen3", "gpt2", "bert", *sorted(_MORE_CAUSAL_LMS)])
def test_whole_small_models(device, family, dtype):
    """Token ids in, logits (or the last hidden state) out: two-layer models as ``transformers`` builds them — a Llama
    and a GPT-2 causal LM, a Qwen-3 base model (the architecture of the reference's flagship embedding model), a BERT
    encoder.  Embeddings are gather kernels; position ids, rotary tables, the causal mask and an empty key / value
    cache depend on no input, so the trace computes them once (a boolean lower-triangle mask becomes the attention
    kernel's own causal form); against the model in float64, and for the causal LMs the greedy next token of every
    position must agree wherever float64's top two are clearly apart."""
    import copy

    torch.manual_seed(81)
    model = _small_model(family).eval()
    ids = torch.randint(3, 1000, (2, 48))
    mod = _Logits(model).to(dtype).eval()
    be = HipBackend()
    compiled = be.compile(trace_module(mod, (ids,)))
    ops = [n.op for n in compiled.nodes.values() if isinstance(n.op, HipOp)]
    names = [op.kernel_name.rsplit("_", 1)[0] for op in ops]
    assert "k_index_rows" in names[:2]
    if dtype is torch.bfloat16:
        assert names.count("k_sdpa_reduce") == 2
        if family not in ("bert", "gemma2"):
            assert all("#define HAS_MASK 0" in op.kernel_source and "#define CAUSAL 1" in op.kernel_source for op in ops if "sdpa" in op.kernel_name)
    prog = be.program(compiled, {compiled.inputs[0]: ids.to(device)})
    try:
        prog.run()
        torch.cuda.synchronize()
        ours = prog.output_tensors()[compiled.outputs[0]].clone().cpu().float()
    finally:
        prog.close()
    with torch.no_grad():
        want = copy.deepcopy(mod).double()(ids).float()
    ours = ours.reshape(want.shape)
    rms = float(want.pow(2).mean().sqrt())
    if dtype is torch.float32:
        eager.assert_close(ours, want, 1e-4, 2e-4 * rms, f"{family} fp32 vs float64")
    else:
        eager.assert_close(ours, want, 2e-2, 4e-2 * max(rms, 1.0), f"{family} bf16 vs float64")
    if family != "bert" and family != "qwen3":
        top2 = want.topk(2, -1).values
        clear = (top2[..., 0] - top2[..., 1]) > (1e-3 if dtype is torch.float32 else 0.1) * rms
        assert bool(clear.any()) and bool((ours.argmax(-1) == want.argmax(-1))[clear].all())


@pytest.mark.gpu
def test_full_width_model_a_few_layers_deep(device):
    """The bench's whole-model workload at four layers and 128 tokens (full width: hidden 1024, 16 / 8 heads of 128,
    vocabulary 151 669): five launches per layer plus the embedding gather and the final norm, and a mean distance
    from the fp32 run of the same model no larger than 1.5 x bf16 eager's own."""
    from deplodock_amd import workloads as wl

    case = wl.qwen3_model_case(seq=128, layers=4)
    be = HipBackend()
    compiled = be.compile(trace_module(case.module, case.inputs))
    names = [n.op.kernel_name.rsplit("_", 1)[0] for n in compiled.nodes.values() if isinstance(n.op, HipOp)]
    assert len(names) == 1 + 4 * 5 + 1 and names[0] == "k_index_rows" and names.count("k_sdpa_reduce") == 4
    prog = be.program(compiled, {compiled.inputs[0]: case.inputs[0].to(device)})
    try:
        prog.run()
        torch.cuda.synchronize()
        ours = prog.output_tensors()[compiled.outputs[0]].clone().float()
    finally:
        prog.close()
    gm = case.module.to(device)
    with torch.no_grad():
        half = gm(case.inputs[0].to(device)).float()
        exact = gm.float()(case.inputs[0].to(device))
    eager.assert_mean_error_within_baseline(ours.reshape(exact.shape), half, exact, 1.5, "four-layer full-width model vs fp32 eager")
    eager.assert_rows_within_baseline(ours.reshape(exact.shape), half, exact, 2.0, "four-layer full-width model rows vs fp32 eager")


@pytest.mark.gpu
def test_whole_model_is_one_set_of_runtime_int_kernels_over_the_sequence_length(device):
    """Token ids in, last hidden state out, with the sequence length symbolic: the embedding gather takes its row count
    at run time like every other kernel of the model, so one compilation serves every length (the rotary table rows
    and the attention lengths follow the same ``int``)."""
    from deplodock_amd import workloads as wl

    case = wl.qwen3_model_case(seq=64, layers=2)
    be = HipBackend()
    compiled = be.compile(trace_module(case.module, case.inputs, dynamic_shapes={"ids": {1: "seq_len"}}))
    assert compiled.symbolic == "seq_len"
    ops = [n.op for n in compiled.nodes.values() if isinstance(n.op, HipOp)]
    assert len(ops) == 1 + 2 * 5 + 1 and all(op.runtime_args == ("seq_len",) for op in ops)
    gm = copy.deepcopy(case.module).to(device)
    for seq in (64, 200, 5):
        torch.manual_seed(seq)
        ids = torch.randint(3, 151000, (1, seq))
        prog = be.program(compiled, {compiled.inputs[0]: ids.to(device)})
        try:
            prog.run()
            torch.cuda.synchronize()
            ours = prog.output_tensors()[compiled.outputs[0]].clone().float()
        finally:
            prog.close()
        with torch.no_grad():
            half = gm(ids.to(device)).float()
            exact = copy.deepcopy(gm).float()(ids.to(device))
        eager.assert_mean_error_within_baseline(ours.reshape(exact.shape), half, exact, 1.5, f"two-layer model at {seq} tokens vs fp32 eager")


@pytest.mark.gpu
@pytest.mark.parametrize("seq", [2048, 4096])
def test_c5_block_at_long_sequences(device, seq):
    """At 2048 tokens the heuristic 128x256 tile of the q/k/v projection spills under its head-norm + rotary output
    stage, and at 4096 the attention schedule spills with its key steps unrolled in pairs: both are rendered again
    in a form that builds clean (a kernel that waits for loads by count must not spill), and the block still matches."""
    from deplodock_amd.backend.hip import hiprtc

    case = eager.qwen3_block_case(seq=seq, norm_std=0.1, seed=7)
    ours, want, compiled = run_case(case, device)
    for n in compiled.nodes.values():
        if isinstance(n.op, HipOp):
            assert hiprtc.spilled_vgprs(n.op.kernel_source, n.op.kernel_name) == 0, n.op.kernel_name
    exact = eager.run_eager_fp32(case, device)
    x = case.inputs[0].to(device).float()
    eager.assert_mean_error_within_baseline(ours.float() - x, want.float() - x, exact - x, 1.5, f"block S={seq} (out - x) vs fp32 eager")
    eager.assert_rows_within_baseline(ours.float() - x, want.float() - x, exact - x, 1.5, f"block S={seq} rows vs fp32 eager")


@pytest.mark.gpu
def test_c4_sdpa_at_4096_tokens(device):
    case = eager.sdpa_case(s=4096)
    ours, want, _ = run_case(case, device)
    q, k, v = (t.to(device).float() for t in case.inputs)
    exact = nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True, enable_gqa=True)
    eager.assert_close(ours, want, 2e-2, 2e-2, "sdpa S=4096 vs eager")
    eager.assert_rows_within_baseline(ours, want, exact, 1.5, "sdpa S=4096 rows vs fp32 eager")


@pytest.mark.gpu
@pytest.mark.parametrize("head_dim", [40, 24])
def test_rotary_embedding_on_heads_that_are_not_whole_16_byte_pairs(device, head_dim):
    """head_dim 40 in bf16 is five 16-byte chunks: the rotate-half kernel keeps both halves of a row in one lane, so
    it narrows its vectors until each half is whole vectors (ten chunks of four); attention at that head_dim runs on the
    flash kernel at its next width (64), the columns past the row's end counting as zeros."""
    case = eager.normed_rope_attention_case(hidden=256, q_heads=4, kv_heads=2, head_dim=head_dim, seq=50)
    ours, want, compiled = run_case(case, device)
    names = [n.op.kernel_name.rsplit("_", 1)[0] for n in compiled.nodes.values() if isinstance(n.op, HipOp)]
    assert any("rope" in n for n in names) and names.count("k_sdpa_reduce") == 1 and "k_batched_linear" not in names, names
    eager.assert_close(ours, want, case.rtol, case.atol, f"rope + attention head_dim={head_dim} vs eager")
