"""Compile-only checks (no GPU): tracing, kernel boundaries, knob pins, source structure,
and hipRTC cross-compilation of every kernel the five configurations need."""

from __future__ import annotations

import re

import pytest
import torch
from torch import nn

from deplodock_amd import HipBackend, trace_module
from deplodock_amd.ir.sym import Affine as Affine_
from deplodock_amd.backend.hip import hiprtc
from deplodock_amd.ir.hip import HipOp
from deplodock_amd.dtype import F32
from deplodock_amd.ir import expr as E
from deplodock_amd.ir.tile import TileOp
from deplodock_amd.passes.fuse import fuse
from oracle import eager


def kernels(compiled):
    return [compiled.nodes[n].op for n in compiled.topological_order() if isinstance(compiled.nodes[n].op, HipOp)]


def compile_case(case):
    return HipBackend().compile(trace_module(case.module, case.inputs))


def test_rms_norm_is_one_fused_reduce_kernel(launcher_lib):
    ks = kernels(compile_case(eager.rms_norm_case()))
    assert len(ks) == 1
    k = ks[0]
    assert re.fullmatch(r"k_rms_norm_reduce_[0-9a-f]{6}", k.kernel_name)
    assert k.knobs["REDUCE"] == "b256" and k.grid[0] == (32,) and k.block[0] == (256,)
    src = k.kernel_source
    assert "emh_wave_reduce<EmhSum, 64>" in src and "rsqrtf" in src
    assert "__shfl" not in src  # wave combine is DPP / swizzle, not a bpermute butterfly
    assert src.count("__syncthreads") == 1  # one LDS hand-off for the 4 waves of a row, no tree
    assert k.algo_bytes == 532480
    hiprtc.compile_to_hsaco(src, k.kernel_name)


def test_softmax_is_one_kernel_with_row_resident_single_read(launcher_lib):
    ks = kernels(compile_case(eager.softmax_case()))
    assert len(ks) == 1
    k = ks[0]
    assert k.kernel_name.startswith("k_softmax_reduce_")
    assert k.algo_bytes == 939524096
    src = k.kernel_source
    assert src.count("expf(") == len(re.findall(r"xv\[\d+\]\[\d+\] = expf", src))  # exp evaluated once per element, kept resident
    assert "EmhMax" in src and "EmhSum" in src
    hiprtc.compile_to_hsaco(src, k.kernel_name)


@pytest.mark.parametrize("m", [1, 16, 128, 2048])
def test_linear_is_one_mfma_kernel(launcher_lib, m):
    ks = kernels(compile_case(eager.linear_case(m=m)))
    assert len(ks) == 1
    k = ks[0]
    assert k.kernel_name.startswith("k_linear_")
    assert "__builtin_amdgcn_mfma_f32_" in k.kernel_source
    assert k.algo_flops == 2 * m * 3072 * 1024
    # decode sizes are one pass over the weight: the reduction axis split over the four waves of a workgroup (256 values each),
    # every fragment requested at once, no slab loop (a shape that does not fit that form goes through two
    # register sets); from 128 rows on direct-to-LDS loads (three 48 KiB slabs
    # of the 32x64x256 tile); at 2048 rows the 128x192 tile's eight waves alternate in two groups behind four
    # staging waves (twelve waves, a ring of four 40 KiB slabs)
    assert k.knobs["STAGE"] == {1: "d4/ks", 16: "d4/ks", 128: "d3/dl", 2048: "d4/pp"}[m]
    assert ("wave * 256 + lk * 8" in k.kernel_source) == (m < 128) and ("#define EMH_DLOAD" in k.kernel_source) == (m >= 128)
    if m == 2048:
        assert k.block[0] == (768,) and k.lds_bytes == 4 * (128 + 192) * 64 * 2 and "role == 2" in k.kernel_source
    if m == 16:
        odd = kernels(compile_case(eager.linear_case(m=16, k=1000, n=712)))[0]  # K is not a multiple of 32
        assert odd.knobs["STAGE"].startswith("d2/sync") and "ra[RS][A_PER_T]" in odd.kernel_source
    hiprtc.compile_to_hsaco(k.kernel_source, k.kernel_name)


def test_sdpa_is_one_flash_kernel(launcher_lib):
    ks = kernels(compile_case(eager.sdpa_case()))
    assert len(ks) == 1
    k = ks[0]
    assert k.kernel_name.startswith("k_sdpa_reduce_")
    assert k.algo_flops == 17188257792
    assert "#define GROUP 2" in k.kernel_source and "#define CAUSAL 1" in k.kernel_source
    assert "flash_pv_smem" not in k.kernel_source  # P stays in registers
    hiprtc.compile_to_hsaco(k.kernel_source, k.kernel_name)


def test_sdpa_with_an_additive_mask_is_the_same_flash_kernel(launcher_lib):
    """The mask is a fourth operand of the one attention kernel: added to the scores (over the scale, so the
    exponent's fma sees ``s * scale + mask``) before the running maximum."""
    torch.manual_seed(0)
    q, k, v = torch.randn(2, 4, 96, 128).bfloat16(), torch.randn(2, 2, 160, 128).bfloat16(), torch.randn(2, 2, 160, 128).bfloat16()
    for mask, strides, vec in ((torch.zeros(1, 1, 96, 160).bfloat16(), (0, 0, 160), 1), (torch.zeros(2, 4, 1, 160), (640, 160, 0), 1), (torch.zeros(2, 1, 96, 160)[..., 1:], None, 0)):
        kk, vv = (k, v) if mask.shape[-1] == 160 else (k[:, :, 1:], v[:, :, 1:])
        ks = kernels(compile_case(eager.Case("m", eager.MaskedSdpa().eval(), (q, kk, vv, mask), 2e-2, 2e-2)))
        assert len(ks) == 1 and ks[0].kernel_name.startswith("k_sdpa_reduce_") and len(ks[0].arg_order) == 5
        src = ks[0].kernel_source
        assert "#define HAS_MASK 1" in src and "#define CAUSAL 0" in src and f"#define MASK_VEC {vec}" in src
        if strides:
            assert all(f"#define {n} {v_}" in src for n, v_ in zip(("M_SB", "M_SH", "M_SS"), strides))
        hiprtc.compile_to_hsaco(src, ks[0].kernel_name)
    with pytest.raises(Exception, match="bool"):
        compile_case(eager.Case("m", eager.MaskedSdpa().eval(), (q, k, v, torch.ones(1, 1, 96, 160, dtype=torch.bool)), 2e-2, 2e-2))


def test_masked_block_repeats_kv_heads_without_a_copy(launcher_lib):
    """Called with an attention mask the layer repeats its KV heads itself (``x[:, :, None].expand(..).reshape(..)``,
    not a view) and hands the bias to attention: still the five kernels of the unmasked block, the attention kernel
    reading the projection's KV windows with grouped heads and the mask as a fourth operand."""
    compiled = compile_case(eager.masked_qwen3_block_case(seq=64))
    ks = kernels(compiled)
    assert [re.sub(r"_[0-9a-f]{6}$", "", k.kernel_name) for k in ks] == ["k_rms_norm_linear_rope", "k_sdpa_reduce", "k_linear_add", "k_rms_norm_linear_silu_mul", "k_linear_add"]
    flash = ks[1].kernel_source
    assert "#define GROUP 2" in flash and "#define HAS_MASK 1" in flash and "#define CAUSAL 0" in flash and "#define M_SS 64" in flash
    assert ks[1].arg_order[:3] == (ks[0].arg_order[-1],) * 3 and ks[1].arg_order[3] == compiled.inputs[3]


def test_expanded_operands_are_broadcast_reads(launcher_lib):
    class ColTimes(nn.Module):
        def forward(self, x, b):
            return x * b[None, :].expand(x.shape[0], -1)

    class RowTimes(nn.Module):
        def forward(self, x, b):
            return x * b[:, None].expand(-1, x.shape[1])

    for mod, b, kind in ((ColTimes(), torch.randn(2048), "col"), (RowTimes(), torch.randn(64), "row")):
        g = trace_module(mod, (torch.randn(64, 2048), b))
        tile = [n.op.body for n in fuse(g).nodes.values() if isinstance(n.op, TileOp)]
        assert len(tile) == 1 and [o.index for o in tile[0].operands] == ["flat", kind]


def test_qwen3_block_kernel_boundaries(launcher_lib):
    compiled = compile_case(eager.qwen3_block_case(seq=64))
    names = [re.sub(r"_[0-9a-f]{6}$", "", k.kernel_name) for k in kernels(compiled)]
    assert names == [
        "k_rms_norm_linear_rope",
        "k_sdpa_reduce", "k_linear_add", "k_rms_norm_linear_silu_mul", "k_linear_add",
    ]  # fmt: skip
    # the two layer norms ride in the contractions that read them, deferred: the norm weight is
    # folded into the stacked projection weights at bind time, the rows are staged as they are
    # while their sum of squares is accumulated, and the accumulators take the row's scale factor
    first = kernels(compiled)[0]
    assert "a=row-scaled-after" in first.comment and first.arg_order[0] == compiled.inputs[0] and first.knobs["STAGE"] == "d3/dl"
    # 16 tokens (as many as heads) and fewer: the projection takes the few-row form with the deferred norm (the row
    # statistic from the fragments a lane holds, the accumulators scaled), and the head norms + rotary embedding of q
    # and k are one small row kernel behind it; one token, whose token dim is a unit dim, pairs q and k the same way
    for seq in (16, 1):
        few = kernels(compile_case(eager.qwen3_block_case(seq=seq)))
        assert [re.sub(r"_[0-9a-f]{6}$", "", k.kernel_name) for k in few] == ["k_rms_norm_linear", "k_rms_norm_rope", "k_sdpa_reduce", "k_linear_add", "k_rms_norm_linear_silu_mul", "k_linear_add"]
        decode, rope = few[0], few[1]
        assert decode.knobs["STAGE"] == "d4/ks" and "ss[t] += emh_xor16(ss[t])" in decode.kernel_source and "* rs_)" in decode.kernel_source
        assert decode.arg_order[1].endswith("__k*p_l_input_layernorm_weight") and rope.arg_order[0] == decode.arg_order[-1]
        for k in few[:2]:
            hiprtc.compile_to_hsaco(k.kernel_source, k.kernel_name)
    assert "__shfl_xor(ss[i], msk, 64)" in first.kernel_source and "* rs_)" in first.kernel_source
    assert "p_l_input_layernorm_weight" not in first.arg_order and first.arg_order[1].endswith("__k*p_l_input_layernorm_weight")
    # q, k and v projections are one contraction over the stacked weights; each
    # projection is a column window of its [tokens, 2048 + 1024 + 1024] result
    qkv = kernels(compiled)[0]
    assert "N=4096" in qkv.comment and qkv.algo_flops == 2 * 64 * 4096 * 1024
    for k in kernels(compiled):
        hiprtc.compile_to_hsaco(k.kernel_source, k.kernel_name)
    # layout ops produced no kernels and no buffers
    assert not any("transpose" in n or "view" in n or "slice" in n for n in compiled.nodes)
    # the query and key head norms + rotary embeddings ride in the projection's
    # output stage: its 128-column tiles are whole heads, the first 16 + 8 of which
    # are normalised (two norm weights stacked per head) and rotated before the store
    assert "row-epilogue=24x128" in qkv.comment and "if (n0 < 3072)" in qkv.kernel_source
    assert qkv.arg_order[-3:-1] == ("cos", "sin") and "emh_wave_reduce<EmhSum, 16>(ss)" in qkv.kernel_source
    # q/k/v and gate/up weights are stacked into constants the runtime assembles
    stacked = sorted((n for n in compiled.nodes.values() if n.hints.get("stacked") and len(n.output.shape) == 2), key=lambda n: n.output.shape[0])
    assert [n.output.shape for n in stacked] == [(4096, 1024), (6144, 1024)]
    data = HipBackend.bind(compiled, {})
    assert [tuple(data[n.id].shape) for n in stacked] == [(4096, 1024), (6144, 1024)]
    traced = compiled.constant_values
    (norm_w,) = [n for n in compiled.nodes.values() if n.hints.get("stacked") and len(n.output.shape) == 1]
    assert tuple(data[norm_w.id].shape) == (24 * 128,)
    assert (data[norm_w.id][15 * 128 : 16 * 128] == traced["p_l_self_attn_q_norm_weight"]).all()
    assert (data[norm_w.id][16 * 128 : 17 * 128] == traced["p_l_self_attn_k_norm_weight"]).all()
    parts = stacked[0].hints["stacked"].parts
    assert [p.split("_proj")[0][-1] for p in parts] == ["q", "k", "v"]
    assert (data[stacked[0].id][2048:3072] == traced[parts[1]]).all()


def test_head_norm_and_rope_fold_into_the_projection(launcher_lib, monkeypatch):
    ks = kernels(compile_case(eager.normed_rope_attention_case()))
    assert [re.sub(r"_[0-9a-f]{6}$", "", k.kernel_name) for k in ks] == ["k_linear_rope", "k_sdpa_reduce"]
    k = ks[0]
    assert "row-epilogue=6x64" in k.comment and "emh_wave_reduce<EmhSum, 8>(ss)" in k.kernel_source
    assert "#define TN 64" in k.kernel_source  # output tiles are whole heads
    hiprtc.compile_to_hsaco(k.kernel_source, k.kernel_name)
    # a pinned tile that splits a head degrades to the heuristic pick for this kernel
    monkeypatch.setenv("EMMY_TILE", "a:mfma_16x16x32_bf16/w1x2/f1x1/k4")
    assert "#define TN 64" in kernels(compile_case(eager.normed_rope_attention_case()))[0].kernel_source


def test_deferred_norm_takes_the_direct_to_lds_ring_at_prefill_sizes(launcher_lib):
    ks = kernels(compile_case(eager.qwen3_block_case(seq=512)))
    qkv, gate_up = ks[0], ks[3]
    assert all(k.knobs["STAGE"] == "d3/dl" for k in (ks[0], ks[2], ks[3], ks[4]))  # four to six MFMAs a step: the request burst stays
    # eight and more MFMAs a step per wave (2 048 tokens: the q/k/v projection's 128x256 tile): the next slab's requests and the
    # next step's fragment reads go out one at a time between the MFMAs
    big = kernels(compile_case(eager.qwen3_block_case(seq=2048)))[0]
    assert big.knobs["STAGE"].endswith("/dlm") and "EMH_DPART_A((kt) + DEPTH, cur," in big.kernel_source and "EMH_DLOAD((kt) + DEPTH, cur);" not in big.kernel_source
    assert "EMH_READ_W(" in big.kernel_source and "EMH_READ_X(" in big.kernel_source
    assert gate_up.knobs["TILE"].endswith("/w4x2/f1x3/k2") and gate_up.grid[0][0] == 256  # 64x96 tiles: one workgroup per CU
    for k in (qkv, gate_up):
        assert "a=row-scaled-after" in k.comment and "#define EMH_SUMSQ_READ(buf)" in k.kernel_source and "EMH_SUMSQ_ADD();" in k.kernel_source
        hiprtc.compile_to_hsaco(k.kernel_source, k.kernel_name)


def test_reduce_pin_is_authoritative_and_bad_pin_degrades(launcher_lib, monkeypatch):
    case = eager.rms_norm_case()
    monkeypatch.setenv("EMMY_REDUCE", "b64")
    k = kernels(compile_case(case))[0]
    assert k.knobs["REDUCE"] == "b64" and k.block[0] == (256,) and k.grid[0] == (8,)
    assert "__syncthreads" not in k.kernel_source  # one wave per row: no LDS at all
    monkeypatch.setenv("EMMY_REDUCE", "b100")
    assert kernels(compile_case(case))[0].knobs["REDUCE"] == "b256"  # resolved spelling is stamped
    monkeypatch.setenv("EMMY_REDUCE", "b16")  # 2048 columns over 16 lanes cannot stay register-resident
    assert kernels(compile_case(case))[0].knobs["REDUCE"] == "b256"


def test_split_k_pin_makes_a_partial_kernel_and_a_combine(launcher_lib, monkeypatch):
    """``REDUCE=g<n>k``: a partial kernel over slices of k (grid y = the split) writing fp32 planes of a workspace,
    and a combine kernel that folds them and owns bias / rounding; ``g<n>a``: one plane, cleared before the launch,
    atomic adds.  A split that does not divide the reduction extent into whole slabs degrades to the unsplit kernel."""
    from deplodock_amd.dtype import F32

    case = eager.linear_case(m=128)
    monkeypatch.setenv("EMMY_REDUCE", "g2k")
    g = compile_case(case)
    ks = {k.kernel_name.rsplit("_", 1)[0]: k for k in kernels(g)}
    assert set(ks) == {"k_linear_partial", "k_linear_combine"}
    part, comb = ks["k_linear_partial"], ks["k_linear_combine"]
    assert part.grid[1] == (2,) and part.knobs["REDUCE"] == "g2k" and comb.knobs["REDUCE"] == "g2k" and part.zero_outputs == ()
    ws = part.arg_order[-1]
    assert comb.arg_order[0] == ws and g.nodes[ws].output.shape == (2, 128, 3072) and g.nodes[ws].output.dtype is F32 and g.node_role(ws) == "scratch"
    assert "blockIdx.y * K" in part.kernel_source and "#define K 512" in part.kernel_source
    order = g.topological_order()
    assert order.index(ws) < order.index(g.outputs[0])
    for k in (part, comb):
        hiprtc.compile_to_hsaco(k.kernel_source, k.kernel_name)
    monkeypatch.setenv("EMMY_REDUCE", "g4a")
    g = compile_case(case)
    part = next(k for k in kernels(g) if "partial" in k.kernel_name)
    assert part.grid[1] == (4,) and part.zero_outputs == (part.arg_order[-1],) and "global_atomic_fadd_f32" in part.kernel_source
    assert g.nodes[part.arg_order[-1]].output.shape == (1, 128, 3072)
    hiprtc.compile_to_hsaco(part.kernel_source, part.kernel_name)
    monkeypatch.setenv("EMMY_REDUCE", "g3k")  # 1024 is not three slices of whole slabs
    (k,) = kernels(compile_case(case))
    assert "REDUCE" not in k.knobs and k.grid[1] == (1,)
    monkeypatch.setenv("EMMY_REDUCE", "g2k")  # few rows: the k-split-over-waves form gives way to slab staging
    part = next(k for k in kernels(compile_case(eager.linear_case(m=16))) if "partial" in k.kernel_name)
    assert part.knobs["STAGE"].startswith("d2/sync")


def test_fp32_linear_takes_the_fp32_mfma_tier(launcher_lib, monkeypatch):
    """An fp32 ``nn.Linear`` (what the reference's own perf suite runs, tests/perf/cases.py:20-23) lowers to the same
    tiled kernel on ``v_mfma_f32_16x16x4_f32`` / ``32x32x2``: 16-byte chunks hold four k-values, one per MFMA."""
    torch.manual_seed(0)
    lin = torch.nn.Linear(1024, 3072).eval()
    x = torch.randn(2048, 1024)
    (k,) = kernels(HipBackend().compile(trace_module(lin, (x,))))
    assert k.knobs["TILE"].startswith("a:mfma_16x16x4_f32/") and "__builtin_amdgcn_mfma_f32_16x16x4f32" in k.kernel_source
    assert "#define EPCK 4" in k.kernel_source and "#define MPF 4" in k.kernel_source and "f32x4 fw[2]" in k.kernel_source
    assert k.algo_flops == 2 * 2048 * 1024 * 3072 and k.algo_bytes == (2048 * 1024 + 3072 * 1024 + 2048 * 3072 + 3072) * 4
    assert hiprtc.vgpr_spill_counts(hiprtc.compile_to_hsaco(k.kernel_source, k.kernel_name).read_bytes()) == [0]
    monkeypatch.setenv("EMMY_TILE", "a:mfma_32x32x2_f32/w2x2/f2x2/k16")
    monkeypatch.setenv("EMMY_STAGE", "d2/sync")
    (k,) = kernels(HipBackend().compile(trace_module(lin, (x,))))
    assert k.knobs["TILE"] == "a:mfma_32x32x2_f32/w2x2/f2x2/k16" and "mfma_f32_32x32x2f32" in k.kernel_source
    monkeypatch.setenv("EMMY_TILE", "a:mfma_32x32x16_bf16/w2x2/f2x2/k2")  # a 16-bit atom on fp32 operands degrades
    (k,) = kernels(HipBackend().compile(trace_module(lin, (x,))))
    assert "_f32/" in k.knobs["TILE"]


def test_tile_and_stage_pins(launcher_lib, monkeypatch):
    case = eager.linear_case()
    monkeypatch.setenv("EMMY_TILE", "a:mfma_32x32x16_bf16/w2x2/f2x3/k4")
    monkeypatch.setenv("EMMY_STAGE", "d3/cp")
    k = kernels(compile_case(case))[0]
    assert k.knobs["TILE"] == "a:mfma_32x32x16_bf16/w2x2/f2x3/k4" and k.knobs["STAGE"] == "d3/dl"
    assert "emh_dma16(" in k.kernel_source and "global_load_lds_dwordx4" in k.kernel_source and k.lds_bytes == 3 * (128 + 192) * 64 * 2
    assert k.grid[0] == (256,)
    hiprtc.compile_to_hsaco(k.kernel_source, k.kernel_name)
    monkeypatch.setenv("EMMY_TILE", "a:mma_m16n8k16_bf16/w2x2/f4x8/k2")  # an NVIDIA pin degrades to the gfx950 pick
    monkeypatch.setenv("EMMY_STAGE", "d2/tma")
    k = kernels(compile_case(case))[0]
    assert "mfma" in k.knobs["TILE"] and k.knobs["STAGE"] == "d4/pp"  # the default staging of this shape


def test_uniform_pointer_halves_are_widened_unsigned(launcher_lib):
    """``emh_uniform`` rebuilds a 64-bit pointer from two ``readfirstlane`` results, which the builtin returns as
    signed ints: widened as they are, a low half with bit 31 set sign-extends over the high half and the requests
    built on that base fault.  The flash kernel's code object must not hold the 32 -> 64 bit sign extension."""
    import subprocess
    import tempfile

    from deplodock_amd.emit import prelude

    assert prelude.DMA.count("(unsigned)__builtin_amdgcn_readfirstlane(") >= 3
    k = kernels(compile_case(eager.sdpa_case()))[0]
    assert "emh_uniform(" in k.kernel_source
    blob = hiprtc.compile_to_hsaco(k.kernel_source, k.kernel_name)
    blob = blob if isinstance(blob, (bytes, bytearray)) else open(blob, "rb").read()
    with tempfile.NamedTemporaryFile(suffix=".hsaco") as fh:
        fh.write(blob)
        fh.flush()
        asm = subprocess.run(["/opt/rocm/llvm/bin/llvm-objdump", "-d", fh.name], capture_output=True, text=True, check=True).stdout
    assert "global_load_lds_dwordx4" in asm and "s_bfe_i64" not in asm


def test_flash_pin_grammar_and_degrade(launcher_lib, monkeypatch):
    case = eager.sdpa_case(1, 8, 4, 320, 128)
    default = kernels(compile_case(case))[0].knobs["FLASH"]
    assert default == "w2/kv32/s4"  # few heads, short sequence: two 32-row groups share each K / V block, four key-split groups
    # long causal self-attention: mirrored query-block pairs, so every workgroup streams the same number of keys
    big = kernels(compile_case(eager.sdpa_case()))[0]
    assert big.knobs["FLASH"] == "w2/kv32/s4/p" and big.grid[0] == (16 * 32 // 2,) and "#define PAIR 1" in big.kernel_source
    monkeypatch.setenv("EMMY_FLASH", "w4/kv64/s2/p")  # 320 rows = 3 blocks of 128: no mirror for the middle one
    assert kernels(compile_case(case))[0].knobs["FLASH"] == default
    monkeypatch.setenv("EMMY_FLASH", "w2/kv32/s4")
    k = kernels(compile_case(case))[0]
    assert k.knobs["FLASH"] == "w2/kv32/s4" and k.block[0] == (512,)
    assert k.lds_bytes == 4 * 4 * 32 * 128 * 2 + 64 * 128 * 2  # four groups' blocks a slot, K and V rings of two slots, then the Q tile
    monkeypatch.setenv("EMMY_FLASH", "w2/kv32/s4/k3")
    k = kernels(compile_case(case))[0]
    # a K ring of three slots beside the V ring of two fills the LDS (the Q fragments then come from global memory)
    assert k.knobs["FLASH"] == "w2/kv32/s4/k3" and k.lds_bytes == 5 * 4 * 32 * 128 * 2 == 160 * 1024 and "#define DEEP 1" in k.kernel_source and "#define Q_LDS 0" in k.kernel_source
    monkeypatch.setenv("EMMY_FLASH", "w2/kv64/s4")  # 256 KiB of staging does not fit: degrade to the default pick
    assert kernels(compile_case(case))[0].knobs["FLASH"] == default
    monkeypatch.setenv("EMMY_FLASH", "w3/zz")
    assert kernels(compile_case(case))[0].knobs["FLASH"] == default


def test_unsupported_op_raises_not_silently_falls_back():
    class Weird(nn.Module):
        def forward(self, x):
            return torch.cumsum(x, -1)

    with pytest.raises(NotImplementedError):
        trace_module(Weird(), (torch.randn(4, 4),))


def test_cache_is_content_addressed(launcher_lib, tmp_path, monkeypatch):
    monkeypatch.setenv("EMMY_HSACO_CACHE", str(tmp_path))
    src = 'extern "C" __global__ void k(float* x) { x[threadIdx.x] = 2.0f; }'
    p1 = hiprtc.compile_to_hsaco(src, "k")
    assert p1.parent == tmp_path and hiprtc.compile_to_hsaco(src, "k") == p1
    monkeypatch.setenv("EMMY_HIPRTC_FLAGS", "-O1")
    assert hiprtc.compile_to_hsaco(src, "k") != p1  # flags are part of the key
    assert not list(tmp_path.glob("*.tmp"))


def test_a_symbolic_axis_lowers_to_kernels_that_take_it_as_a_runtime_int(launcher_lib):
    """``dynamic_shapes`` marks axes.  With one symbolic axis the module lowers once: every kernel whose work
    follows the axis takes the extent as a trailing ``int`` parameter (``emh_n_seq_len``: a name no local of a kernel has), guards its rows / key blocks at run time and is
    launched on a grid the runtime sizes per launch (the reference's form: ir/kernel/ir.py:258-276,
    ir/cuda/ir.py:66-112).  One code object per kernel then serves every length."""
    from deplodock_amd.ir.sym import Affine, CeilDiv, XcdRounds

    case = eager.qwen3_block_case(seq=64)
    g = trace_module(case.module, case.inputs, dynamic_shapes={"x": {1: "seq_len"}, "cos": {1: "seq_len"}, "sin": {1: "seq_len"}})
    assert g.dynamic.hints == {"seq_len": 64} and g.dynamic.input_axes == [{1: "seq_len"}] * 3
    be = HipBackend()
    compiled = be.compile(g)
    assert compiled.symbolic == "seq_len" and not hasattr(compiled, "variants")
    ks = kernels(compiled)
    assert len(ks) == 5
    for k in ks:
        assert k.runtime_args == ("seq_len",) and k.kernel_source.count("int emh_n_seq_len") == 1
        hiprtc.compile_to_hsaco(k.kernel_source, k.kernel_name)
    flash = next(k for k in ks if k.kernel_name.startswith("k_sdpa"))
    assert flash.grid[0] == (CeilDiv(Affine("seq_len", 1, 0), 32 * int(flash.knobs["FLASH"].split("/")[0][1:])), 16) and "/p" not in flash.knobs["FLASH"]
    assert "#define SQ (emh_n_seq_len)" in flash.kernel_source and "#define GRID ((int)gridDim.x)" in flash.kernel_source
    lin = next(k for k in ks if k.kernel_name.startswith("k_linear_add"))
    assert isinstance(lin.grid[0][0], XcdRounds) and "#define M (emh_n_seq_len)" in lin.kernel_source and "/ks" not in lin.knobs["STAGE"]
    assert lin.grid[0][0]({"seq_len": 200}) >= -(-200 // lin.grid[0][0].tile_m) * lin.grid[0][0].blocks_n * lin.grid[0][0].per_block
    assert compiled.nodes["x"].output.shape == (1, "seq_len", 1024) and compiled.nodes[compiled.outputs[0]].output.shape == (1, "seq_len", 1024)

    def inputs_at(s):
        return {n: torch.zeros([s if i == 1 else d for i, d in enumerate(t.shape)], dtype=t.dtype) for n, t in zip(compiled.inputs, case.inputs)}

    assert be.variant(compiled, inputs_at(96)) is compiled and be.variant(compiled, None) is compiled  # no per-size lowering
    with pytest.raises(NotImplementedError, match="not arguments"):
        trace_module(case.module, case.inputs, dynamic_shapes={"nope": {1: "s"}})


def test_a_symbolic_fp32_linear_never_takes_the_cross_workgroup_split(launcher_lib, monkeypatch):
    """A split contraction is a kernel pair with the row count baked in (partial grid, combine extent).  A module
    traced with a symbolic row count must therefore either come out as runtime-int kernels on every launch (the
    fp32 tier's automatic split stands down) or not be marked symbolic at all (a pinned split: per-size lowering)."""
    import torch.nn as nn

    mod = nn.Linear(1024, 1024).eval()
    g = trace_module(mod, (torch.randn(64, 1024),), dynamic_shapes={"input": {0: "seq"}})
    be = HipBackend()
    compiled = be.compile(g)
    assert compiled.symbolic == "seq"
    ks = kernels(compiled)
    assert ks and all(k.runtime_args == ("seq",) for k in ks), [(k.kernel_name, k.runtime_args) for k in ks]
    assert not any("partial" in k.kernel_name or "combine" in k.kernel_name for k in ks)
    # the static lowering of the same shape does split (so the case above is the one the guard is for)
    static = be.compile(trace_module(mod, (torch.randn(64, 1024),)))
    assert any("partial" in k.kernel_name for k in kernels(static))
    # a pinned split cannot be symbolic: the backend falls back to lowering per size
    monkeypatch.setenv("EMMY_REDUCE", "g4k")
    pinned = HipBackend().compile(trace_module(mod, (torch.randn(64, 1024),), dynamic_shapes={"input": {0: "seq"}}))
    assert getattr(pinned, "symbolic", None) is None and hasattr(pinned, "variants")


def test_position_tables_folded_at_trace_time_follow_a_symbolic_length_as_prefixes(launcher_lib):
    """Token ids in: the rotary cos / sin tables are constants computed from the positions when the model is traced,
    so their row count follows the symbolic length.  Rows at one length are the leading rows at any longer one: the
    lowering stays one set of runtime-int kernels (embedding gather included), and binding hands out the leading rows
    of the largest table held, re-tracing once for a length beyond it."""
    from deplodock_amd import workloads as wl
    from deplodock_amd.passes.symbolic import SymbolicError, _prefix_table

    case = wl.qwen3_model_case(seq=64, layers=1)
    g = trace_module(case.module, case.inputs, dynamic_shapes={"ids": {1: "seq_len"}})
    be = HipBackend()
    compiled = be.compile(g)
    assert compiled.symbolic == "seq_len"
    ks = kernels(compiled)
    assert ks[0].kernel_name.startswith("k_index_rows_") and all(k.runtime_args == ("seq_len",) for k in ks)
    tables = [nid for nid, n in compiled.nodes.items() if "prefix_table" in n.hints]
    assert len(tables) == 2 and all(compiled.nodes[t].output.shape == (1, 1, "seq_len", 128) for t in tables)
    for size, held in ((5, None), (64, None), (200, 200), (130, 200), (500, 500)):
        data = be.bind(compiled, {compiled.inputs[0]: torch.randint(3, 1000, (1, size))})
        want = fuse(g.dynamic.retrace({"seq_len": size})).constant_values
        assert all(torch.equal(data[t], want[t]) for t in tables), size
        assert getattr(compiled, "prefix_table_size", None) == held
    # what is not such a table is refused: values that change on the common rows, or an inner dim that follows the axis
    a = Affine_("s", 1, 0)
    with pytest.raises(SymbolicError, match="leading rows"):
        _prefix_table("c", (1, a, 4), [torch.zeros(1, 3, 4), torch.ones(1, 5, 4), torch.zeros(1, 9, 4)], "s")
    with pytest.raises(SymbolicError, match="leading dim"):
        _prefix_table("c", (2, a, 4), [torch.zeros(2, 3, 4), torch.zeros(2, 5, 4), torch.zeros(2, 9, 4)], "s")
    assert _prefix_table("c", (1, a, 4), [torch.arange(12.0).reshape(1, 3, 4), torch.arange(20.0).reshape(1, 5, 4), torch.arange(36.0).reshape(1, 9, 4)], "s") == 1


def test_per_size_specialisation_remains_for_what_does_not_symbolise(launcher_lib):
    """With runtime-int kernels switched off (or a module whose kernel boundaries change with the size) the backend
    re-traces and re-lowers per distinct size and keeps an LRU of the results."""
    case = eager.qwen3_block_case(seq=64)
    g = trace_module(case.module, case.inputs, dynamic_shapes={"x": {1: "seq_len"}, "cos": {1: "seq_len"}, "sin": {1: "seq_len"}})
    be = HipBackend()
    be.symbolic_kernels = False
    compiled = be.compile(g)
    assert getattr(compiled, "symbolic", None) is None and be.variant(compiled, None) is compiled

    def inputs_at(s):
        return {n: torch.zeros([s if i == 1 else d for i, d in enumerate(t.shape)], dtype=t.dtype) for n, t in zip(compiled.inputs, case.inputs)}

    assert be.variant(compiled, inputs_at(64)) is compiled
    v96 = be.variant(compiled, inputs_at(96))
    assert v96 is not compiled and be.variant(compiled, inputs_at(96)) is v96
    assert 96 in v96.nodes[v96.outputs[0]].output.shape and v96.inputs == compiled.inputs and v96.outputs == compiled.outputs
    for s in range(1, 12):
        be.variant(compiled, inputs_at(32 * s + 32))
    assert len(compiled.variants) == HipBackend.VARIANT_CACHE
    bad = inputs_at(96)
    bad[compiled.inputs[1]] = torch.zeros(1, 80, 128, dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="disagree"):
        be.variant(compiled, bad)


def test_symbolize_refuses_what_a_runtime_int_cannot_express():
    from deplodock_amd.graph import Graph, Tensor
    from deplodock_amd.ir.tile import RowReduce, Stat, TileOp
    from deplodock_amd.passes.symbolic import SymbolicError, symbolize

    def tile(rows, cols):
        g = Graph()
        g.add_input("X", (rows, cols))
        body = RowReduce(rows=rows, cols=cols, x="X", x_dtype=F32, out="y", out_dtype=F32, stats=(Stat("s", "sum", E.Var("x")),), project=E.Var("x") / E.Var("s"))
        g.add_node(TileOp(name="k_n", body=body), ["X"], Tensor("y", (rows, cols), F32))
        g.outputs = ["y"]
        return g

    ok = symbolize([tile(8, 64), tile(15, 64), tile(104, 64)], "rows", [8, 15, 104])
    assert ok.nodes["y"].op.body.sym.fields == {"rows": Affine_("rows", 1, 0)}
    with pytest.raises(SymbolicError, match="cols"):  # the reduced extent is baked into the kernel
        symbolize([tile(8, 64), tile(8, 71), tile(8, 160)], "cols", [64, 71, 160])
    with pytest.raises(SymbolicError, match="not affine"):
        symbolize([tile(8, 64), tile(16, 64), tile(100, 64)], "rows", [8, 15, 104])


def test_elementwise_trees_fold_into_one_map_kernel(launcher_lib):
    class Tree(nn.Module):
        def forward(self, x, y, w):
            return torch.exp(torch.neg(x)) * y + w  # w: a vector along the last axis

    g = trace_module(Tree(), (torch.randn(8, 64), torch.randn(8, 64), torch.randn(64)))
    (k,) = kernels(HipBackend().compile(g))
    assert k.kernel_name.startswith("k_pointwise_fused4") and k.kernel_source.count("expf(") >= 1
    assert len(k.arg_order) == 4  # x, y, w, out

    class Shared(nn.Module):
        def forward(self, x):
            t = torch.exp(x)  # two readers: stays a kernel of its own
            return t * 2.0, t + 1.0

    names = [k.kernel_name.rsplit("_", 1)[0] for k in kernels(HipBackend().compile(trace_module(Shared(), (torch.randn(4, 32),))))]
    assert names == ["k_pointwise_elementwise"] * 3


def test_row_sum_and_mean_are_row_reductions(launcher_lib):
    class M(nn.Module):
        def forward(self, x):
            return x - x.mean(-1, keepdim=True)

    # centring rows is one row kernel (the mean a statistic of the resident row) ...
    ks = kernels(HipBackend().compile(trace_module(M(), (torch.randn(16, 256),))))
    assert [k.kernel_name.rsplit("_", 1)[0] for k in ks] == ["k_row_fused_reduce"] and ks[0].algo_bytes == 2 * 16 * 256 * 4
    # ... and a mean that is a result of its own is a row reduction with one value per row
    ks = kernels(HipBackend().compile(trace_module(type("Mean", (nn.Module,), {"forward": lambda self, x: x.mean(-1, keepdim=True)})(), (torch.randn(16, 256),))))
    assert [k.kernel_name.rsplit("_", 1)[0] for k in ks] == ["k_mean_reduce"]
    assert "one value per row" in ks[0].comment and ks[0].algo_bytes == 16 * 256 * 4 + 16 * 4
    # any other axis is moved last by a dense copy first
    ks = kernels(HipBackend().compile(trace_module(type("S", (nn.Module,), {"forward": lambda self, x: x.sum(0)})(), (torch.randn(4, 8),))))
    assert [k.kernel_name.rsplit("_", 1)[0] for k in ks] == ["k_gather", "k_sum_reduce"]


def test_short_last_slab_takes_the_register_staged_path(launcher_lib):
    """K = 200 is 6 MFMA steps and 8 elements: the slabs are 64 deep, the fourth one is mostly zeros."""
    k = kernels(compile_case(eager.linear_case(m=64, k=200, n=712)))[0]
    assert k.knobs["STAGE"] == "d2/sync" and k.knobs["TILE"].endswith("/k2")
    assert "if ((kt) * BK + ka[i] < K)" in k.kernel_source and "if ((kt) * BK + kb[i] < K)" in k.kernel_source
    hiprtc.compile_to_hsaco(k.kernel_source, k.kernel_name)
    with pytest.raises(Exception):  # rows that are not whole 16-byte chunks stay unsupported
        compile_case(eager.linear_case(m=64, k=100, n=712))


def test_direct_to_lds_ring_kernels_must_not_spill(launcher_lib, monkeypatch):
    """The slab ring waits for part of its outstanding loads by count; spill stores share that counter and
    complete out of order with loads.  A tile whose accumulators fill the registers degrades to register
    staging at schedule time, and a ring kernel that spills anyway is refused by the compile step."""
    from deplodock_amd.backend.hip import launcher as L

    assert hiprtc.vgpr_spill_counts(b"xx.vgpr_spill_count\xcd\x01\xa1yy.vgpr_spill_count\x05") == [417, 5]
    default = kernels(compile_case(eager.linear_case(m=2048)))[0]
    assert default.knobs["STAGE"].endswith(("/dl", "/pp")) and hiprtc.NO_SPILL_CONTRACT in default.kernel_source
    monkeypatch.setenv("EMMY_TILE", "a:mfma_32x32x16_bf16/w1x1/f3x4/k8")
    monkeypatch.setenv("EMMY_STAGE", "d2/dl")
    k = kernels(compile_case(eager.linear_case(m=2048, k=3072, n=3072)))[0]
    # 56 request addresses beside 192 accumulators: this tile sits at the edge of the register file; whatever the
    # compiler makes of it, what the pipeline hands on does not spill
    assert hiprtc.spilled_vgprs(k.kernel_source, k.kernel_name) == 0
    # a ring kernel (it carries the contract's marker) that needs more registers than its launch bounds leave
    live = "\n".join(f"  float v{i} = x[t + {i} * 1024];" for i in range(160)) + "\n  __syncthreads();\n" + "\n".join(f"  x[t + {i} * 1024] = v{(i * 7) % 160} * v{(i * 13) % 160};" for i in range(160))
    src = f'{hiprtc.NO_SPILL_CONTRACT} {{}}\nextern "C" __global__ __launch_bounds__(1024) void k_spilling_ring(float* x) {{\n  const int t = threadIdx.x;\n{live}\n}}\n'
    with pytest.raises(L.CompileError, match="spilled"):
        hiprtc.compile_to_hsaco(src, "k_spilling_ring")


def test_a_pinned_tile_that_only_builds_with_spills_degrades(launcher_lib, monkeypatch):
    """The code object decides: register sets that overflow first give way to plain register staging, and a
    tile that still spills to the heuristic one; the stamped knobs name what was built."""
    monkeypatch.setenv("EMMY_TILE", "a:mfma_32x32x16_bf16/w2x1/f4x4/k4")
    monkeypatch.setenv("EMMY_STAGE", "d2/sync/p3")
    k = kernels(compile_case(eager.linear_case(m=256, k=1024, n=1024)))[0]
    assert hiprtc.spilled_vgprs(k.kernel_source, k.kernel_name) == 0
    assert k.knobs["STAGE"] != "d2/sync/p3"
    monkeypatch.setenv("EMMY_TILE", "a:mfma_32x32x16_bf16/w1x1/f3x6/k2")  # 288 accumulators per lane
    k = kernels(compile_case(eager.linear_case(m=256, k=1024, n=1024)))[0]
    assert "f3x6" not in k.knobs["TILE"]


def test_matmul_spelled_attention_lowers_to_batched_contractions(launcher_lib):
    """``torch.matmul`` / ``@`` trace to ``MatmulOp``: ``q @ k.T`` reads ``k`` in place (the transposed view's reduction
    axis is the contiguous one), ``p @ v`` gets ``v`` transposed by a copy nest; each product is one launch whose
    second grid dimension is batch x heads.  A ragged reduction extent is padded."""
    import torch
    from torch import nn

    from deplodock_amd import HipBackend, trace_module
    from deplodock_amd.backend.hip import hiprtc
    from deplodock_amd.ir import frontend as F
    from deplodock_amd.ir.hip import HipOp
    class Attn(nn.Module):
        def forward(self, q, k, v):
            return torch.softmax(torch.matmul(q, k.transpose(-1, -2)) * 0.125, -1) @ v

    q = torch.randn(2, 4, 104, 64)  # (fp32: 16-bit operands are raised to the fused attention kernel instead)
    traced = trace_module(Attn().eval(), (q, q.clone(), q.clone()))
    assert sum(isinstance(n.op, F.MatmulOp) for n in traced.nodes.values()) == 2
    compiled = HipBackend().compile(traced)
    ks = [n.op for n in compiled.nodes.values() if isinstance(n.op, HipOp)]
    assert [k.kernel_name.rsplit("_", 1)[0] for k in ks] == ["k_matmul", "k_pointwise_elementwise", "k_softmax_reduce", "k_gather", "k_matmul"]
    assert [k.grid[1] for k in ks if k.kernel_name.startswith("k_matmul")] == [(8,), (8,)]
    for k in ks:
        hiprtc.compile_to_hsaco(k.kernel_source, k.kernel_name)
    # 16-bit operands: the same module is one attention kernel
    qb = torch.randn(2, 4, 104, 64).bfloat16()
    kb = [n.op.kernel_name.rsplit("_", 1)[0] for n in HipBackend().compile(trace_module(Attn().eval(), (qb, qb.clone(), qb.clone()))).nodes.values() if isinstance(n.op, HipOp)]
    assert kb == ["k_sdpa_reduce"]
    # a key count that is not whole 16-byte chunks: the second product's operands are copied with their reduction axis
    # padded with zeros (both, so that nothing undefined meets a zero)
    q = torch.randn(2, 4, 100, 64)
    ks = [n.op for n in HipBackend().compile(trace_module(Attn().eval(), (q, q.clone(), q.clone()))).nodes.values() if isinstance(n.op, HipOp)]
    assert [k.kernel_name.rsplit("_", 1)[0] for k in ks] == ["k_matmul", "k_pointwise_elementwise", "k_softmax_reduce", "k_gather", "k_gather", "k_matmul"]
    assert "K=104" in ks[-1].comment
    for k in ks:
        hiprtc.compile_to_hsaco(k.kernel_source, k.kernel_name)


@pytest.mark.parametrize("mode", [1, 2])
def test_stamped_measurement_builds_of_the_attention_and_ring_contraction_kernels_compile(launcher_lib, mode, monkeypatch):
    """``-DEMH_STAMP=1|2`` among the compiler options builds the same kernels with shader-clock stamps at their phase
    boundaries (``microbench --stamps`` reads them): the stamped sources of the default attention kernel, the burst and
    spread direct-to-LDS rings and the wave-specialised ring build without spills; without the define the statements are
    compiled out (same source text, the define decides)."""
    monkeypatch.setenv("EMMY_HIPRTC_FLAGS", f"-DEMH_STAMP={mode}")
    cases = [eager.sdpa_case(), eager.sdpa_case(s=512), eager.linear_case(m=4096, k=4096, n=4096), eager.linear_case(m=2048), eager.linear_case(m=512)]
    stages = []
    for case in cases:
        (k,) = kernels(compile_case(case))
        assert "EMH_STAMP_AT(" in k.kernel_source and "EMH_PHASE_AT(" in k.kernel_source and "#ifndef EMH_STAMP" in k.kernel_source
        assert hiprtc.spilled_vgprs(k.kernel_source, k.kernel_name) == 0, k.kernel_name
        stages.append(k.knobs.get("STAGE"))
    assert stages[2:] == ["d2/dlm", "d4/pp", "d3/dl"]
