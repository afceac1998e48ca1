"""Attention no streaming kernel takes (16-bit rows that are not whole 16-byte chunks, head dims beyond 256) is decomposed into the two loop nests
the reference's own pipeline reaches (masked scores; softmax times v).  Pinned on the host: the two nests,
evaluated by the Loop-IR restatement in float64, equal ``F.scaled_dot_product_attention`` in float64 — a wrong
head-group index, mask predicate, scale or broadcast is an error of order one."""

import numpy as np
import pytest
import torch
import torch.nn.functional as Fn
from torch import nn

from deplodock_amd import HipBackend, trace_module
from deplodock_amd.ir.hip import HipOp
from deplodock_amd.ir import frontend as F
from deplodock_amd.passes.decompose_attention import decompose_attention
from deplodock_amd.passes.fuse import FusionError, _undo_repeat_kv
from oracle import loop_ir


class _Sdpa(nn.Module):
    def __init__(self, **kw):
        super().__init__()
        self.kw = kw

    def forward(self, q, k, v, mask=None):
        return Fn.scaled_dot_product_attention(q, k, v, attn_mask=mask, **self.kw)


class _RepeatedKv(nn.Module):
    """Grouped heads the materialising way (``repeat_kv`` of the Llama family)."""

    def forward(self, q, k, v):
        b, h, s, d = k.shape
        g = q.shape[1] // h
        k = k[:, :, None].expand(b, h, g, s, d).reshape(b, h * g, s, d)
        v = v[:, :, None].expand(b, h, g, s, d).reshape(b, h * g, s, d)
        return Fn.scaled_dot_product_attention(q, k, v, is_causal=True)


def _causal_bias(sq, skv):
    return torch.zeros(sq, skv).masked_fill(torch.arange(skv)[None, :] > torch.arange(sq)[:, None], float("-inf"))


CASES = {
    "causal_gqa": (_Sdpa(is_causal=True, enable_gqa=True), [(1, 4, 12, 8), (1, 2, 12, 8), (1, 2, 12, 8)], None),
    "plain_batch2": (_Sdpa(), [(2, 3, 9, 8), (2, 3, 9, 8), (2, 3, 9, 8)], None),
    "cross_lengths_scale": (_Sdpa(scale=0.3), [(2, 2, 5, 4), (2, 2, 11, 4), (2, 2, 11, 6)], None),
    "mask_1_1_s_s": (_Sdpa(), [(2, 3, 7, 4), (2, 3, 7, 4), (2, 3, 7, 4)], lambda: _causal_bias(7, 7)[None, None]),
    "mask_b_1_1_s": (_Sdpa(enable_gqa=True), [(2, 4, 6, 4), (2, 2, 10, 4), (2, 2, 10, 4)], lambda: torch.randn(2, 1, 1, 10)),
    "mask_s_s": (_Sdpa(), [(1, 2, 6, 4), (1, 2, 6, 4), (1, 2, 6, 4)], lambda: torch.randn(6, 6)),
    "two_lead_dims": (_Sdpa(is_causal=True), [(2, 3, 2, 6, 4), (2, 3, 2, 6, 4), (2, 3, 2, 6, 4)], None),
    "repeat_kv": (_RepeatedKv(), [(2, 6, 8, 4), (2, 2, 8, 4), (2, 2, 8, 4)], None),
}


@pytest.mark.parametrize("case", sorted(CASES))
def test_decomposed_nests_equal_eager_attention(case):
    mod, shapes, mask = CASES[case]
    torch.manual_seed(5)
    args = [torch.randn(*s) for s in shapes] + ([mask()] if mask else [])
    g = trace_module(mod.eval(), tuple(args))
    d = decompose_attention(g, _undo_repeat_kv, streamed=lambda node: False)  # (fp32 operands of these sizes would stay fused)
    assert not any(isinstance(n.op, F.SdpaOp) for n in d.nodes.values())
    nests = [n for n in d.nodes.values() if isinstance(n.op, F.LoopNestOp)]
    assert [n.op.label for n in nests] == ["sdpa_scores", "sdpa_softmax_v"]
    if case == "repeat_kv":  # the repeat is the head // group index, not a copy
        assert [d.nodes[i].output.shape[1] for i in nests[0].inputs] == [6, 2]
    values = {nid: a.double().numpy() for nid, a in zip(g.inputs, args)}
    for n in nests:
        ins = {name: values[src] for name, src in zip(n.op.loads, n.inputs)}
        ins.update({name: np.array([val]) for name, val in (n.op.scalars or {}).items()})
        shape = tuple(int(x) for x in n.output.shape)
        values[n.id] = loop_ir.run_vectorised(n.op.stmts, ins, shape)
        if n.output.numel <= 2048:  # the literal python-loop reading of the same statements
            np.testing.assert_allclose(loop_ir.run_loops(n.op.stmts, ins, shape), values[n.id], rtol=1e-12, atol=1e-12)
    want = mod(*(a.double() for a in args)).numpy()
    np.testing.assert_allclose(values[nests[1].id], want, rtol=1e-9, atol=1e-9)


def _kernel_names(compiled):
    return [n.op.kernel_name.rsplit("_", 1)[0] for n in compiled.nodes.values() if isinstance(n.op, HipOp)]


def test_which_attention_is_decomposed():
    """16-bit rows that are not whole 16-byte chunks, fp32 head dims beyond 256 and value rows of another length than the
    keys' become two batched contractions with loop-nest operand / output stages; fp32 up to head_dim 256 is one streaming
    kernel on fp32 atoms, 16-bit head_dim 128 the one fused kernel, and a 16-bit head_dim between the kernel's widths
    (32: padded to 64 with columns that count as zeros) takes it too."""
    be = HipBackend()
    q, k = torch.randn(1, 16, 128, 128), torch.randn(1, 8, 128, 128)
    compiled = be.compile(trace_module(_Sdpa(is_causal=True, enable_gqa=True).eval(), (q, k, k)))
    assert _kernel_names(compiled) == ["k_sdpa_reduce"]
    (op,) = [n.op for n in compiled.nodes.values() if isinstance(n.op, HipOp)]
    assert "mfma_f32_32x32x2f32" in op.kernel_source and op.knobs["FLASH"].startswith("f32/")
    for shapes in ([(1, 2, 40, 320)] * 3, [(1, 2, 40, 16), (1, 2, 40, 16), (1, 2, 40, 24)]):
        names = _kernel_names(be.compile(trace_module(_Sdpa().eval(), tuple(torch.randn(*s) for s in shapes))))
        assert names.count("k_batched_linear") == 2 and "k_sdpa_reduce" not in names
        assert names.count("k_operand_a") == 1  # q is read in place; only the softmax is an operand stage of its own
    names = _kernel_names(be.compile(trace_module(_Sdpa(is_causal=True, enable_gqa=True).eval(), (q.bfloat16(), k.bfloat16(), k.bfloat16()))))
    assert names == ["k_sdpa_reduce"]
    q32 = torch.randn(2, 4, 64, 32).bfloat16()
    compiled = be.compile(trace_module(_Sdpa().eval(), (q32, q32, q32)))
    assert _kernel_names(compiled) == ["k_sdpa_reduce"]
    (op,) = [n.op for n in compiled.nodes.values() if isinstance(n.op, HipOp)]
    assert "#define D 64\n" in op.kernel_source and "#define DR 32\n" in op.kernel_source
    q36 = torch.randn(2, 4, 64, 36).bfloat16()  # rows that are not whole 16-byte chunks: the kernel on fp32 atoms, converting as it stages
    compiled = be.compile(trace_module(_Sdpa().eval(), (q36, q36, q36)))
    assert _kernel_names(compiled) == ["k_sdpa_reduce"]
    (op,) = [n.op for n in compiled.nodes.values() if isinstance(n.op, HipOp)]
    assert "mfma_f32_32x32x2f32" in op.kernel_source and "#define ELT __bf16\n" in op.kernel_source
    q320 = torch.randn(1, 2, 40, 320).bfloat16()
    names = _kernel_names(be.compile(trace_module(_Sdpa().eval(), (q320, q320, q320))))
    assert names.count("k_batched_linear") == 2 and "k_sdpa_reduce" not in names


def test_grouped_heads_without_the_flag_are_refused():
    q, k = torch.randn(1, 4, 8, 8), torch.randn(1, 2, 8, 8)
    g = trace_module(_Sdpa(enable_gqa=True).eval(), (q, k, k))
    for n in g.nodes.values():
        if isinstance(n.op, F.SdpaOp):
            n.op.enable_gqa = False
    with pytest.raises(FusionError, match="enable_gqa"):
        HipBackend().compile(g)


def test_a_scores_tensor_beyond_the_limit_is_refused_with_a_message():
    """The decomposed route writes the scores to device memory; a shape whose scores exceed the limit is refused when
    the module is compiled, not when the runtime asks for the memory."""
    from deplodock_amd.passes.fuse import FusionError

    q = torch.zeros(1, 32, 16384, 264).bfloat16()
    with pytest.raises(FusionError, match="16.0 GiB of scores"):
        HipBackend().compile(trace_module(_Sdpa(is_causal=True).eval(), (q, q, q)))


@pytest.mark.parametrize("head_dim, form", [(3, "w1"), (21, "w4"), (40, "s4"), (64, "s8"), (128, "s4"), (128, "s2"), (128, "s8/o"), (128, "s4/o"), (64, "s2/o"), (128, "s4/sp"), (128, "w4"), (200, "w2"), (256, "w1")])
def test_fp32_streaming_attention_builds_without_spills(head_dim, form, monkeypatch):
    """Every head_dim up to 256 and both forms of the fp32 streaming kernel build within a wave's registers (the
    key-split form counts its outstanding direct-to-LDS requests, which spill traffic would disturb); the key-split
    form is refused — and the shared form taken — for rows that are not whole 16-byte chunks or wider than 128 values."""
    from deplodock_amd.backend.hip import hiprtc, launcher

    monkeypatch.setenv("EMMY_FLASH", f"f32/{form}")
    q = torch.randn(1, 4, 70, head_dim)
    k = torch.randn(1, 2, 90, head_dim)
    compiled = HipBackend().compile(trace_module(_Sdpa(enable_gqa=True).eval(), (q, k, k, torch.randn(70, 90))))
    (op,) = [n.op for n in compiled.nodes.values() if isinstance(n.op, HipOp)]
    assert op.knobs["FLASH"] == f"f32/{form}" and "mfma_f32_32x32x2f32" in op.kernel_source
    assert op.block[0] == ((64 * int(form.split("/")[0][1:]),) if form[0] == "s" else (256,))
    try:
        assert hiprtc.spilled_vgprs(op.kernel_source, op.kernel_name) == 0
    except launcher.CompileError:
        raise
    except launcher.LauncherError:
        pytest.skip("no launcher library: the code object is not built here")


def test_fp32_streaming_attention_default_forms(monkeypatch):
    monkeypatch.delenv("EMMY_FLASH", raising=False)

    def form(q_shape, kv_shape):
        q, k = torch.randn(*q_shape), torch.randn(*kv_shape)
        (op,) = [n.op for n in HipBackend().compile(trace_module(_Sdpa(is_causal=True, enable_gqa=True).eval(), (q, k, k))).nodes.values() if isinstance(n.op, HipOp)]
        return op.knobs["FLASH"]

    assert form((1, 16, 32, 128), (1, 8, 32, 128)) == "f32/w1"  # one key block: nothing to split
    assert form((1, 16, 128, 128), (1, 8, 128, 128)) == "f32/s4/o"  # four key blocks: four waves
    assert form((1, 16, 512, 128), (1, 8, 512, 128)) == "f32/s8/o"
    assert form((1, 16, 2048, 128), (1, 8, 2048, 128)) == "f32/s4/o"  # four workgroups per CU and more
    assert form((1, 2, 40, 21), (1, 2, 40, 21)) == "f32/w1"  # rows that are not whole 16-byte chunks
    assert form((1, 2, 40, 256), (1, 2, 40, 256)) == "f32/w1"  # beyond 128 columns
    # a pin the shape cannot take is ignored
    monkeypatch.setenv("EMMY_FLASH", "f32/s4")
    assert form((1, 2, 40, 21), (1, 2, 40, 21)) == "f32/w1"
