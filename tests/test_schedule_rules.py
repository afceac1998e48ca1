"""Scheduling rules that came out of tuner sweeps of the decoder layer (``tune arch:qwen3-0.6b --layer 0 --seq-len S``,
1 - 1024 tokens): what ``passes/schedule.py`` picks with nothing pinned, checked on the host through the whole lowering
(every kernel here also has to build)."""

from __future__ import annotations

import re

import torch
from torch import nn

from deplodock_amd import HipBackend, trace_module
from deplodock_amd import workloads as wl
from deplodock_amd.ir.hip import HipOp
from oracle import eager


def kernels(case_or_module, inputs=None) -> dict[str, HipOp]:
    module, inputs = (case_or_module.module, case_or_module.inputs) if inputs is None else (case_or_module, inputs)
    compiled = HipBackend().compile(trace_module(module, inputs))
    return {re.sub(r"_[0-9a-f]{6}$", "", n.op.kernel_name): n.op for n in compiled.nodes.values() if isinstance(n.op, HipOp)}


def test_two_waves_on_16x32_tiles_down_to_a_quarter_of_the_cus(launcher_lib):
    """32 rows x 1024 columns: 64 workgroups of two waves (4.70 us at K = 3072), not 128 one-wave 16x16 tiles (7.04)."""
    op = kernels(eager.linear_case(m=32, k=3072, n=1024))["k_linear"]
    assert op.knobs["TILE"].endswith("/w1x2/f1x1/k8") and op.knobs["STAGE"] == "d3/dl" and op.grid[0] == (64,) and op.block[0] == (128,)


def test_decoder_block_at_32_tokens(launcher_lib):
    """Up to 32 tokens the head norms + rotary embedding are a launch of their own behind a few-row q/k/v projection; the
    few-row form splits K = 1024 over four waves and owns whole 16-column tiles (192 workgroups for the gate / up pair);
    the 32-row o / down projections (more than 16 rows of K > 1024) take the two-wave 16x32 tile."""
    ks = kernels(eager.qwen3_block_case(seq=32))
    assert set(ks) == {"k_rms_norm_linear", "k_rms_norm_rope", "k_sdpa_reduce", "k_linear_add", "k_rms_norm_linear_silu_mul"}
    assert ks["k_rms_norm_linear"].knobs["STAGE"] == "d4/ks" and ks["k_rms_norm_linear"].grid[0] == (4096 // 16,)
    assert ks["k_rms_norm_linear_silu_mul"].knobs["STAGE"] == "d4/ks" and ks["k_rms_norm_linear_silu_mul"].grid[0] == (3072 // 16,)
    assert ks["k_linear_add"].knobs["TILE"].endswith("/w1x2/f1x1/k8") and ks["k_linear_add"].knobs["STAGE"] == "d3/dl"


def test_decoder_block_at_96_tokens(launcher_lib):
    """No second round of workgroups for a few stragglers (288 tiles of 32x32 -> 144 eight-wave tiles of 32x64), 128-deep
    slabs where only those leave the LDS for a third ring slot, and four key-split groups for three key blocks."""
    ks = kernels(eager.qwen3_block_case(seq=96))
    gate_up, qkv = ks["k_rms_norm_linear_silu_mul"], ks["k_rms_norm_linear_rope"]
    assert gate_up.knobs["TILE"].endswith("/w2x4/f1x1/k4") and gate_up.knobs["STAGE"] == "d3/dl" and gate_up.grid[0] == (144,)
    assert qkv.knobs["TILE"].endswith("/w1x4/f1x2/k4") and qkv.knobs["STAGE"] == "d3/dl"
    assert ks["k_sdpa_reduce"].knobs["FLASH"] == "w1/kv32/s4"


def test_gate_up_pair_takes_its_64x96_tile_as_a_three_quarter_cover(launcher_lib):
    ks = kernels(eager.qwen3_block_case(seq=384))
    assert ks["k_rms_norm_linear_silu_mul"].knobs["TILE"].endswith("/w4x2/f1x3/k2") and ks["k_rms_norm_linear_silu_mul"].grid[0] == (192,)
    assert ks["k_sdpa_reduce"].knobs["FLASH"] == "w2/kv32/s4"  # two row groups a workgroup from three 64-row blocks on


def test_decode_attention_slices_keep_256_keys(launcher_lib):
    for kv, slices in ((2048, 8), (4096, 16), (32768, 16)):
        ks = kernels(wl.sdpa_decode_case(q_len=1, kv_len=kv))
        assert ks["k_sdpa_reduce_partial"].knobs["REDUCE"] == f"g{slices}k", (kv, ks["k_sdpa_reduce_partial"].knobs)


def test_fp32_tier_prefers_even_rounds_and_splits_few_rows(launcher_lib):
    torch.manual_seed(0)
    # 256 x 3072: 192 tiles of 64x64 fill three quarters of one round; 768 four-wave 32x32 tiles are three even rounds
    op = kernels(nn.Linear(1024, 3072, bias=False).eval(), (torch.randn(256, 1024),))["k_linear"]
    assert op.knobs["TILE"] == "a:mfma_16x16x4_f32/w2x2/f1x1/k16" and op.knobs["STAGE"] == "d2/dl" and op.grid[0] == (768,)
    # 16 rows over a 12 MiB weight: the reduction axis split across workgroups, as for 17 - 128 rows
    ks = kernels(nn.Linear(3072, 1024, bias=False).eval(), (torch.randn(16, 3072),))
    assert set(ks) == {"k_linear_partial", "k_linear_combine"} and ks["k_linear_partial"].knobs["REDUCE"] == "g8k"
