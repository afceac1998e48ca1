"""Reading the reference's own traced-graph fixtures (``Graph.to_dict`` JSON) and driving this backend with them.

``tests/golden/tinyllama_layer0.json`` and ``qwen25_7b_layer0.json`` are the data files of the reference's
tests/compiler/fixtures (traced decoder blocks, fp32, 8 tokens; tests/compiler/ir/test_real_trace.py checks their
op census).  The oracle is PyTorch eager evaluating the same node list (``oracle.ref_graph.evaluate_torch``) and the
numpy restatement of the reference's ``Op.forward`` definitions; both are pinned here against ``transformers``'
decoder layers."""

from __future__ import annotations

import json
from pathlib import Path

import numpy as np
import pytest
import torch

from deplodock_amd import HipBackend
from deplodock_amd.dtype import BF16, F32
from deplodock_amd.ingest import IngestError, graph_from_reference_dict, load_reference_graph
from deplodock_amd.ir import frontend as F
from deplodock_amd.ir.base import ConstantOp, InputOp
from deplodock_amd.ir.hip import HipOp
from oracle import eager, ref_graph

GOLDEN = Path(__file__).resolve().parent / "golden"
TINYLLAMA = GOLDEN / "tinyllama_layer0.json"
QWEN25 = GOLDEN / "qwen25_7b_layer0.json"


def _census(g) -> dict[str, int]:
    out: dict[str, int] = {}
    for n in g.nodes.values():
        out[type(n.op).__name__] = out.get(type(n.op).__name__, 0) + 1
    return out


def test_tinyllama_fixture_reads_as_a_traced_graph():
    """Same census the reference asserts on this file (test_real_trace.py:33-70: 3 inputs, 7 linears, 1 attention,
    means kept, one silu), with the format's scalar-constant nodes folded into the ops that take them."""
    g = load_reference_graph(TINYLLAMA)
    ops = _census(g)
    assert g.inputs == ["hidden_states", "position_embeddings_0", "position_embeddings_1"] and g.outputs == ["add_5"]
    assert ops["InputOp"] == 3 and ops["LinearOp"] == 7 and ops["SdpaOp"] == 1 and ops["MeanOp"] == 2 and ops["ConstantOp"] == 9
    assert sum(1 for n in g.nodes.values() if isinstance(n.op, F.ElementwiseOp) and n.op.fn == "silu") == 1
    assert all(not (isinstance(n.op, ConstantOp) and n.output.shape == (1,)) for n in g.nodes.values())  # scalars are not tensors here
    assert g.nodes["pow_1"].op.scalar == 2.0 and g.nodes["add"].op.scalar == pytest.approx(1e-5) and g.nodes["mean"].op == F.MeanOp(axis=2, keepdim=True)
    assert g.nodes["slice_2"].op == F.SliceOp(dim=3, start=32, end=64, step=1) and g.nodes["cat"].op == F.CatOp(dim=3)  # legacy [tensor, dim, start, end] inputs
    assert g.nodes["transpose"].op == F.TransposeOp(dim0=1, dim1=2) and g.nodes["view"].op == F.ViewOp(shape=(1, 8, 32, 64))
    sd = g.nodes["scaled_dot_product_attention"]
    assert sd.op.is_causal is False and sd.op.enable_gqa and sd.output.shape == (1, 1, 32, 8, 64)  # traced with [1, 1, S, D] rotary tables
    assert all(n.output.dtype is F32 for n in g.nodes.values())
    assert all(n.output.dtype is BF16 for n in load_reference_graph(TINYLLAMA, cast=BF16).nodes.values())
    assert isinstance(g.nodes["hidden_states"].op, InputOp)


def test_later_stage_or_foreign_json_is_refused():
    with pytest.raises(IngestError, match="not a reference graph"):
        graph_from_reference_dict({"format": 1, "nodes": []})
    data = json.loads(TINYLLAMA.read_text())
    data["nodes"]["linear"]["op"] = "TileOp"
    with pytest.raises(IngestError, match="only the frontend"):
        graph_from_reference_dict(data)
    data = json.loads(TINYLLAMA.read_text())
    data["nodes"]["silu"]["op_fields"]["op"] = "erfinv"
    with pytest.raises(IngestError, match="not traced"):
        graph_from_reference_dict(data)


def _masked_attention_json(b=1, hq=4, hkv=2, sq=24, skv=40, d=64) -> dict:
    """A frontend graph in the reference's JSON form whose ``SdpaOp`` takes a fourth, additive-mask input
    (emmy/compiler/trace/torch.py:559-583)."""
    def t(name, shape):
        return {"name": name, "shape": list(shape), "dtype": "f32"}

    nodes = {n: {"op": "InputOp", "op_fields": {}, "inputs": [], "output": t(n, shp)}
             for n, shp in (("q", (b, hq, sq, d)), ("k", (b, hkv, skv, d)), ("v", (b, hkv, skv, d)), ("mask", (1, 1, sq, skv)))}  # fmt: skip
    nodes["attn"] = {"op": "SdpaOp", "op_fields": {"is_causal": True}, "inputs": ["q", "k", "v", "mask"], "output": t("attn", (b, hq, sq, d))}
    return {"inputs": ["q", "k", "v", "mask"], "outputs": ["attn"], "nodes": nodes}


def test_masked_attention_graph_reads_with_the_mask_as_an_operand(launcher_lib):
    data = _masked_attention_json()
    g = graph_from_reference_dict(data, cast=BF16)
    op = g.nodes["attn"].op
    assert isinstance(op, F.SdpaOp) and op.has_mask and not op.is_causal and g.nodes["attn"].inputs == ["q", "k", "v", "mask"]
    compiled = HipBackend().compile(g)
    ks = [n.op for n in compiled.nodes.values() if isinstance(n.op, HipOp)]
    assert len(ks) == 1 and "#define HAS_MASK 1" in ks[0].kernel_source
    # the two interpreters agree on the masked node, and the mask is what makes the difference
    vals = ref_graph.random_values(data, seed=3)
    vals["mask"] = torch.where(torch.rand(vals["mask"].shape, generator=torch.Generator().manual_seed(4)) < 0.3, -float("inf"), 1.0) * torch.ones_like(vals["mask"])
    vals["mask"][..., 0] = 0.0
    want = ref_graph.evaluate_torch(data, vals)["attn"].numpy()
    got = ref_graph.evaluate_numpy(data, {k: v.numpy() for k, v in vals.items()})["attn"]
    np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-5)
    unmasked = ref_graph.evaluate_numpy(data, {**{k: v.numpy() for k, v in vals.items()}, "mask": np.zeros_like(vals["mask"].numpy())})["attn"]
    assert np.abs(unmasked - got).max() > 1e-2


@pytest.mark.gpu
def test_masked_attention_graph_runs_on_the_gpu(device):
    data = _masked_attention_json(b=2, hq=4, hkv=2, sq=100, skv=164, d=128)
    vals = {k: v.bfloat16() for k, v in ref_graph.random_values(data, seed=5).items()}
    hole = torch.rand(vals["mask"].shape, generator=torch.Generator().manual_seed(6)) < 0.4
    vals["mask"] = vals["mask"].masked_fill(hole, -float("inf"))
    vals["mask"][..., 0] = 0.0
    be = HipBackend()
    compiled = be.compile(graph_from_reference_dict(data, cast=BF16))
    prog = be.program(compiled, {n: vals[n].to(device) for n in compiled.inputs})
    try:
        prog.run()
        torch.cuda.synchronize()
        ours = prog.output_tensors()["attn"].clone()
    finally:
        prog.close()
    want = ref_graph.evaluate_torch(data, {k: v.to(device) for k, v in vals.items()})["attn"]
    eager.assert_close(ours.reshape(want.shape), want, 2e-2, 2e-2, "ingested masked attention vs eager")


@pytest.mark.parametrize("path,launches", [(TINYLLAMA, 7), (QWEN25, 7)])
def test_fixtures_lower_to_fused_kernels(launcher_lib, path, launches):
    """The ingested block compiles to the same kind of kernels a traced module does (norms folded into the
    projections that read them, rotary embedding as row kernels, one attention kernel, residual adds in the
    projections' output stage); Qwen2.5's biased q/k/v projections are merged over stacked weights and a stacked bias."""
    compiled = HipBackend().compile(load_reference_graph(path, cast=BF16))
    ks = [n.op for n in compiled.nodes.values() if isinstance(n.op, HipOp)]
    assert len(ks) == launches
    names = " ".join(k.kernel_name for k in ks)
    assert names.count("k_sdpa_reduce") == 1 and names.count("k_rope") == 2 and names.count("k_linear_add") == 2 and "k_rms_norm_linear_silu_mul" in names


def _llama_layer(values: dict, kind: str):
    """A ``transformers`` decoder layer carrying the fixture's weights (no download: built from a local config)."""
    if kind == "llama":
        from transformers import LlamaConfig as Cfg
        from transformers.models.llama.modeling_llama import LlamaDecoderLayer as Layer

        cfg = Cfg(hidden_size=2048, num_attention_heads=32, num_key_value_heads=4, head_dim=64, intermediate_size=5632, rms_norm_eps=1e-5, num_hidden_layers=1, vocab_size=64)
    else:
        from transformers import Qwen2Config as Cfg
        from transformers.models.qwen2.modeling_qwen2 import Qwen2DecoderLayer as Layer

        cfg = Cfg(hidden_size=3584, num_attention_heads=28, num_key_value_heads=4, intermediate_size=18944, rms_norm_eps=1e-6, num_hidden_layers=1, vocab_size=64)
    cfg._attn_implementation = "sdpa"
    layer = Layer(cfg, 0).eval()
    sd = layer.state_dict()
    with torch.no_grad():
        for name, t in values.items():
            if not name.startswith("p_"):
                continue
            key = name[2:].replace("attn_", "self_attn.").replace("mlp_", "mlp.").replace("_proj_", "_proj.").replace("layernorm_", "layernorm.")
            assert key in sd and sd[key].shape == t.shape, (name, key)
            sd[key].copy_(t)
    return layer


@pytest.mark.parametrize("path,kind,eps", [(TINYLLAMA, "llama", 1e-5), (QWEN25, "qwen2", 1e-6)])
def test_graph_interpreters_are_pinned_by_the_library_decoder_layer(path, kind, eps):
    """Fed ordinary ``[1, S, D]`` rotary tables the fixture's node list is the library's decoder layer with full
    (non-causal) attention: PyTorch eager on the nodes and the numpy restatement must both reproduce
    ``LlamaDecoderLayer`` / ``Qwen2DecoderLayer`` carrying the same weights.  A wrong slice order in the rotation,
    a swapped cat, a missing bias, a mean taken as a sum or a wrong GQA head mapping fails this."""
    data = json.loads(path.read_text())
    if kind == "qwen2":
        assert data["nodes"]["add_c1"]["op_fields"]["value"] == pytest.approx(eps)
    d = data["nodes"]["position_embeddings_0"]["output"]["shape"][-1]
    values = ref_graph.random_values(data, seed=4, shapes={"position_embeddings_0": (1, 8, d), "position_embeddings_1": (1, 8, d)})
    layer = _llama_layer(values, kind)
    x, cos, sin = values["hidden_states"], values["position_embeddings_0"], values["position_embeddings_1"]
    with torch.no_grad():
        out = layer(x, position_embeddings=(cos, sin), attention_mask=torch.zeros(1, 1, 8, 8))  # an all-zero additive mask: full attention
    want = out[0] if isinstance(out, tuple) else out
    got_t = ref_graph.evaluate_torch(data, values)[data["outputs"][0]]
    eager.assert_close(got_t, want, 1e-4, 1e-4, f"{path.name}: eager on the node list vs the library layer")
    got_n = ref_graph.evaluate_numpy(data, {k: v.numpy() for k, v in values.items()})[data["outputs"][0]]
    np.testing.assert_allclose(got_n, want.double().numpy(), rtol=1e-4, atol=1e-4)
    # and at the recorded (five-dimensional) operand shapes the two interpreters agree with each other
    rec = ref_graph.random_values(data, seed=5)
    a = ref_graph.evaluate_torch(data, rec)[data["outputs"][0]]
    b = ref_graph.evaluate_numpy(data, {k: v.numpy() for k, v in rec.items()})[data["outputs"][0]]
    assert tuple(a.shape) == tuple(data["nodes"][data["outputs"][0]]["output"]["shape"])
    np.testing.assert_allclose(a.double().numpy(), b, rtol=1e-4, atol=1e-4)


@pytest.mark.gpu
@pytest.mark.parametrize("path", [TINYLLAMA, QWEN25])
def test_reference_fixture_runs_on_the_gpu_and_matches_eager(device, path):
    """A graph the reference wrote drives this backend: read the JSON (as a bf16 module: the attention kernel
    takes 16-bit operands), lower, run, and compare with PyTorch eager evaluating the same node list in bf16 —
    within the bf16 tolerance of the fp32 evaluation, and no further from it (mean, and worst row) than 1.5 x what bf16 eager is."""
    data = json.loads(path.read_text())
    values = ref_graph.random_values(data, seed=6)
    be = HipBackend()
    compiled = be.compile(load_reference_graph(path, cast=BF16))
    on_dev = {k: v.to(device).bfloat16() for k, v in values.items()}
    res_prog = be.program(compiled, {k: on_dev[k] for k in on_dev if k in compiled.nodes or k in values})
    try:
        res_prog.run()
        torch.cuda.synchronize()
        ours = res_prog.output_tensors()[compiled.outputs[0]].clone()
    finally:
        res_prog.close()
    out_id = data["outputs"][0]
    want = ref_graph.evaluate_torch(data, on_dev)[out_id]
    exact = ref_graph.evaluate_torch(data, {k: v.float() for k, v in on_dev.items()})[out_id]
    ours = ours.reshape(want.shape)
    # Outputs here are O(1)..O(10) (hidden sizes 2048 / 3584, an 18944-deep down projection), so the absolute floor
    # scales with the output: bf16 rtol 2e-2 plus 3 % of the output's RMS, against the fp32 evaluation.
    rms = float(exact.pow(2).mean().sqrt())
    eager.assert_close(ours, exact, 2e-2, 3e-2 * rms, f"{path.name} vs fp32 eager on the node list")
    x = on_dev["hidden_states"].float()
    eager.assert_mean_error_within_baseline(ours.float() - x, want.float() - x, exact - x, 1.5, f"{path.name} (out - x) vs fp32 eager")
    eager.assert_rows_within_baseline(ours.float() - x, want.float() - x, exact - x, 1.5, f"{path.name} rows of (out - x) vs fp32 eager")
