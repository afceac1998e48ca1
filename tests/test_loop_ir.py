"""The Loop-IR reader and its CPU restatement, pinned without the reference:

* the parser accepts the eleven kernel reproducers the reference ships (``kernels/*.json``, copied as data under
  ``tests/golden/loop_ir/``) and refuses text that is not a statement constructor;
* the vectorised interpreter equals the literal python-loop interpreter on small nests that exercise every
  statement kind, floor division / modulo of negative index values included;
* the eleven reproducers are the kernels of one TinyLlama decoder layer at 128 tokens (fp32): chained by their
  node names and evaluated in float64 they reproduce ``transformers``' ``LlamaDecoderLayer`` in float64 to 1e-5 of
  the largest output (the layer's own RMSNorm squares its rows in float32 whatever the module's dtype, which is
  the 1e-7 that remains) — a wrong rotary index, head mapping, mask predicate or fold is an error of order one.
"""

import json
from pathlib import Path

import numpy as np
import pytest

from deplodock_amd.ir import loopnest as L
from oracle import loop_ir

CORPUS = Path(__file__).parent / "golden" / "loop_ir"


def corpus() -> dict[str, dict]:
    return {p.stem: json.loads(p.read_text()) for p in sorted(CORPUS.glob("*.json"))}


def loop_node(doc: dict) -> tuple[str, dict]:
    (nid, node), = [(n, v) for n, v in doc["nodes"].items() if v["op"] == "LoopOp"]
    return nid, node


def test_the_shipped_reproducers_parse():
    docs = corpus()
    assert len(docs) == 11
    kinds = set()
    for doc in docs.values():
        nid, node = loop_node(doc)
        stmts = L.parse_body(node["op_fields"]["body"])
        kinds |= {type(s).__name__ for s in L.walk(stmts)}
        assert loop_ir.infer_write_shape(stmts) == tuple(node["output"]["shape"])
    assert kinds == {"Loop", "Load", "Assign", "Accum", "Select", "Write"}


@pytest.mark.parametrize(
    "text, message",
    [
        ("__import__('os').system('true')", "constructor call"),
        ("Loop(axis=Axis(name='a', extent=4), body=(exec('1'),))", "not read"),
        ("Load(name='x', input='X', index=(Var(name='a').__class__,))", "constructor call"),
        ("Loop(axis=Axis(name='a', extent=Dim('s')), body=())", "symbolic extent"),
        ("Load(name='x', input='X', index=(Var(name='a'),))", "outside their loops"),
        ("Loop(axis=Axis(name='a', extent=4), body=(Accum(name='s', value='y'),))", "before it is bound"),
        ("Assign(name='y', op=ElementwiseImpl('frobnicate'), args=('x',))", "not read"),
        ("Accum(name='s', value='x', base='t')", "later stage"),
        ("StridedLoop(axis=Axis(name='a', extent=4), body=())", "not read"),
        ("1 +", "not a statement expression"),
    ],
)
def test_text_that_is_not_a_loop_ir_statement_is_refused(text, message):
    with pytest.raises(L.LoopNestError, match=message):
        L.parse_body([text])


SMALL = [
    # statistics of a row (two folds in one loop), a rotated read with a negative intermediate index, a Select
    # between a per-element value and a row value
    (
        ["Load(name='c', input='cnt', index=(Literal(value=0, dtype='int'),))",
         "Loop(axis=Axis(name='a0', extent=3), body=(Loop(axis=Axis(name='a1', extent=5), body=(Load(name='x', input='X', index=(Var(name='a0'), Var(name='a1'))), "
         "Assign(name='sq', op=ElementwiseImpl('multiply'), args=('x','x')), Accum(name='acc', value='sq', op=ElementwiseImpl('add')), Accum(name='mx', value='x', op=ElementwiseImpl('maximum')))), "
         "Assign(name='m', op=ElementwiseImpl('divide'), args=('acc','c')), Assign(name='r', op=ElementwiseImpl('rsqrt'), args=('m',)), "
         "Loop(axis=Axis(name='a2', extent=5), body=(Load(name='y', input='X', index=(Var(name='a0'), BinaryExpr(op='%', left=BinaryExpr(op='-', left=Var(name='a2'), right=Literal(value=2, dtype='int')), right=Literal(value=5, dtype='int')))), "
         "Assign(name='z', op=ElementwiseImpl('multiply'), args=('y','r')), Select(name='w', branches=(SelectBranch(value='z', select=BinaryExpr(op='<', left=Var(name='a2'), right=Literal(value=2, dtype='int'))), "
         "SelectBranch(value='mx', select=Literal(value=1, dtype='int')))), Write(output='O', index=(Var(name='a0'), Var(name='a2')), value='w')))))"],
        {"X": (3, 5), "cnt": (1,)},
        lambda a: np.where(np.arange(5)[None] < 2, a["X"][:, (np.arange(5) - 2) % 5] / np.sqrt((a["X"] ** 2).sum(1) / a["cnt"][0])[:, None], a["X"].max(1)[:, None]),
    ),
    # a contraction with a residual, written through a permuted index; the flat index is taken apart with / and %
    (
        ["Loop(axis=Axis(name='m', extent=4), body=(Loop(axis=Axis(name='n', extent=6), body=(Loop(axis=Axis(name='k', extent=7), body=("
         "Load(name='a', input='A', index=(Var(name='m'), Var(name='k'))), Load(name='b', input='B', index=(BinaryExpr(op='/', left=BinaryExpr(op='+', left=BinaryExpr(op='*', left=Var(name='n'), right=Literal(value=7, dtype='int')), right=Var(name='k')), right=Literal(value=7, dtype='int')), "
         "BinaryExpr(op='%', left=BinaryExpr(op='+', left=BinaryExpr(op='*', left=Var(name='n'), right=Literal(value=7, dtype='int')), right=Var(name='k')), right=Literal(value=7, dtype='int')))), "
         "Assign(name='p', op=ElementwiseImpl('multiply'), args=('a','b')), Accum(name='s', value='p'))), Load(name='r', input='R', index=(Var(name='n'), Var(name='m'))), "
         "Assign(name='o', op=ElementwiseImpl('add'), args=('s','r')), Write(output='O', index=(Var(name='n'), Literal(value=0, dtype='int'), Var(name='m')), value='o'))),))"],
        {"A": (4, 7), "B": (6, 7), "R": (6, 4)},
        lambda a: (a["A"] @ a["B"].T + a["R"].T).T[:, None, :],
    ),
    # a softmax-weighted sum: two folds feeding a nested fold (loops that hold loops), sibling loops reusing an axis name
    (
        ["Loop(axis=Axis(name='q', extent=3), body=(Loop(axis=Axis(name='j', extent=4), body=(Load(name='s', input='S', index=(Var(name='q'), Var(name='j'))), Accum(name='mx', value='s', op=ElementwiseImpl('maximum')))), "
         "Loop(axis=Axis(name='j', extent=4), body=(Load(name='s2', input='S', index=(Var(name='q'), Var(name='j'))), Assign(name='d', op=ElementwiseImpl('subtract'), args=('s2','mx')), Assign(name='e', op=ElementwiseImpl('exp'), args=('d',)), Accum(name='l', value='e'))), "
         "Loop(axis=Axis(name='c', extent=2), body=(Loop(axis=Axis(name='j2', extent=4), body=(Load(name='s3', input='S', index=(Var(name='q'), Var(name='j2'))), Assign(name='d2', op=ElementwiseImpl('subtract'), args=('s3','mx')), Assign(name='e2', op=ElementwiseImpl('exp'), args=('d2',)), "
         "Load(name='v', input='V', index=(Var(name='j2'), Var(name='c'))), Assign(name='p', op=ElementwiseImpl('divide'), args=('e2','l')), Assign(name='pv', op=ElementwiseImpl('multiply'), args=('p','v')), Accum(name='o', value='pv'))), "
         "Write(output='O', index=(Var(name='q'), Var(name='c')), value='o')))))"],
        {"S": (3, 4), "V": (4, 2)},
        lambda a: (np.exp(a["S"] - a["S"].max(1, keepdims=True)) / np.exp(a["S"] - a["S"].max(1, keepdims=True)).sum(1, keepdims=True)) @ a["V"],
    ),
]  # fmt: skip


@pytest.mark.parametrize("case", range(len(SMALL)))
def test_vectorised_interpreter_equals_the_literal_loops_and_the_closed_form(case):
    body, shapes, closed = SMALL[case]
    stmts = L.parse_body(body)
    rng = np.random.default_rng(case)
    arrays = {k: (rng.standard_normal(s) if k != "cnt" else np.array([5.0])) for k, s in shapes.items()}
    shape = loop_ir.infer_write_shape(stmts)
    want = closed(arrays)
    assert shape == want.shape
    literal = loop_ir.run_loops(stmts, arrays, shape)
    np.testing.assert_allclose(literal, want, rtol=1e-12, atol=1e-12)
    for budget in (1 << 24, 8, 1):  # all axes as array axes / outer loops one iteration at a time
        np.testing.assert_allclose(loop_ir.run_vectorised(stmts, arrays, shape, budget=budget), literal, rtol=1e-12, atol=1e-12)


def llama_layer(seed: int = 0):
    """The decoder layer the corpus was cut from (TinyLlama-1.1B architecture), random weights, float64."""
    import torch
    from transformers import LlamaConfig
    from transformers.models.llama.modeling_llama import LlamaDecoderLayer, LlamaRotaryEmbedding

    cfg = LlamaConfig(hidden_size=2048, num_attention_heads=32, num_key_value_heads=4, head_dim=64, intermediate_size=5632, rms_norm_eps=1e-5,
                      num_hidden_layers=1, vocab_size=64, max_position_embeddings=2048, rope_theta=10000.0)  # fmt: skip
    cfg._attn_implementation = "eager"
    torch.manual_seed(seed)
    layer = LlamaDecoderLayer(cfg, 0)
    with torch.no_grad():
        for name, p in layer.named_parameters():
            p.copy_(1 + 0.1 * torch.randn_like(p) if "norm" in name else 0.02 * torch.randn_like(p))
    return cfg, layer.double().eval(), LlamaRotaryEmbedding(cfg)


WEIGHT_NAMES = {
    "p_input_layernorm_weight": "input_layernorm.weight", "p_post_attention_layernorm_weight": "post_attention_layernorm.weight",
    "p_attn_q_proj_weight": "self_attn.q_proj.weight", "p_attn_k_proj_weight": "self_attn.k_proj.weight", "p_attn_v_proj_weight": "self_attn.v_proj.weight",
    "p_attn_o_proj_weight": "self_attn.o_proj.weight", "p_mlp_gate_proj_weight": "mlp.gate_proj.weight", "p_mlp_up_proj_weight": "mlp.up_proj.weight",
    "p_mlp_down_proj_weight": "mlp.down_proj.weight",
}  # fmt: skip


def corpus_layer_case(seed: int = 0, seq: int = 128):
    """``(values by node name, expected output)``: the layer's inputs and weights under the corpus' node names, and
    the eager float64 output."""
    import torch

    cfg, layer, rotary = llama_layer(seed)
    torch.manual_seed(seed + 1)
    x = torch.randn(1, seq, cfg.hidden_size, dtype=torch.float64)
    cos, sin = rotary(x.float(), torch.arange(seq)[None])
    cos, sin = cos.double(), sin.double()
    mask = torch.zeros(1, 1, seq, seq, dtype=torch.float64).masked_fill(torch.arange(seq)[None, :] > torch.arange(seq)[:, None], float("-inf"))
    with torch.no_grad():
        out = layer(x, position_embeddings=(cos, sin), attention_mask=mask)
    out = out[0] if isinstance(out, tuple) else out
    sd = layer.state_dict()
    values = {"hidden_states": x.numpy(), "position_embeddings_0": cos.numpy(), "position_embeddings_1": sin.numpy()}
    values.update({k: sd[v].numpy() for k, v in WEIGHT_NAMES.items()})
    return values, out.numpy()


def run_corpus_chain(values: dict[str, np.ndarray], run) -> dict[str, np.ndarray]:
    """Evaluate the eleven kernels in dependency order; ``run(stmts, operands, node, doc)`` evaluates one."""
    docs = corpus()
    values = dict(values)
    pending = dict(docs)
    while pending:
        ready = [k for k, d in pending.items() if all(i in values for i in d["inputs"])]
        assert ready, f"kernels {sorted(pending)} wait for inputs nobody produces"
        for k in ready:
            doc = pending.pop(k)
            nid, node = loop_node(doc)
            operands = {}
            for name in node["inputs"]:
                src = doc["nodes"][name]
                if src["op"] == "ConstantOp" and src["op_fields"].get("value") is not None:
                    operands[name] = np.full(tuple(src["output"]["shape"]), src["op_fields"]["value"])
                else:
                    operands[name] = values[name].reshape(tuple(src["output"]["shape"]))
            values[nid] = run(L.parse_body(node["op_fields"]["body"]), operands, node, doc)
    return values


def test_the_corpus_chained_is_the_decoder_layer_it_was_cut_from():
    values, want = corpus_layer_case()
    got = run_corpus_chain(values, lambda stmts, operands, node, doc: loop_ir.run_vectorised(stmts, operands, tuple(node["output"]["shape"])))
    out = got["merged_merged_lift_add_5"]
    assert out.shape == want.shape
    err = np.abs(out - want).max()
    assert err < 1e-5 * np.abs(want).max(), err


# ---------------------------------------------------------------------------------------------------------------
# the product side: ingest -> lower -> run on the GPU


def _kernels(compiled):
    from deplodock_amd.ir.hip import HipOp

    return [compiled.nodes[n].op for n in compiled.topological_order() if isinstance(compiled.nodes[n].op, HipOp)]


RAISED = {  # what each reproducer becomes when nests with a tiled form are raised (kernel labels, in launch order)
    "k_add_3_reduce": ["k_gather", "k_linear_add"],  # the attention output is read through a permuted index: copied to a plain matrix first
    "k_add_5_reduce": ["k_linear_add"],
    # the k / v projections (128 x 2048 x 256 in fp32) would put 32 tiles on 256 CUs: the reduction axis is split across workgroups
    "k_linear_1_reduce_reduce": ["k_linear_partial", "k_linear_combine"],
    "k_linear_2_reduce_reduce": ["k_linear_partial", "k_linear_combine"],
    "k_linear_4_reduce": ["k_linear"],
    "k_linear_reduce_reduce": ["k_linear"],
    "k_mul_1_reduce": ["k_rms_norm_reduce"],
    "k_mul_7_reduce": ["k_rms_norm_reduce"],
    "k_mul_8_reduce": ["k_linear", "k_pointwise_fused6"],
    # scores: the rotary embedding is applied while each operand is written out, the per-head products are one batched
    # contraction, scale and causal mask run over its result
    "k_scaled_dot_product_attention_masked_reduce": ["k_operand_a", "k_operand_b", "k_batched_linear", "k_output_stage"],
    # softmax-weighted sum: the probabilities (two folds and the division) and the transposed values are written out,
    # then one batched contraction
    "k_scaled_dot_product_attention_reduce_reduce": ["k_operand_a", "k_operand_b", "k_batched_linear"],
}


@pytest.mark.parametrize("mode", ["raised", "loops"])
def test_every_reproducer_lowers_to_kernels_that_build_for_gfx950(launcher_lib, monkeypatch, mode):
    """By default a nest that is a contraction (+ element-wise output stage) or a row RMS normalisation is raised
    to the tiled kernels (fp32 MFMA contraction, register-resident row kernel); ``EMMY_NEST=loops`` renders every
    nest loop for loop."""
    import re

    from deplodock_amd import HipBackend
    from deplodock_amd.backend.hip import hiprtc
    from deplodock_amd.ingest import load_reference_graph

    if mode == "loops":
        monkeypatch.setenv("EMMY_NEST", "loops")
    be = HipBackend()
    for path in sorted(CORPUS.glob("*.json")):
        ks = _kernels(be.compile(load_reference_graph(path)))
        labels = [re.sub(r"_[0-9a-f]{6}$", "", k.kernel_name) for k in ks]
        if mode == "loops":
            assert len(ks) == 1 and "NEST" in ks[0].knobs, (path.name, labels)
        else:
            assert labels == RAISED[path.stem], (path.name, labels)
            assert [("NEST" in k.knobs) for k in ks] == [lab in ("k_gather", "k_operand_a", "k_operand_b", "k_output_stage") for lab in labels]
        for k in ks:
            hiprtc.compile_to_hsaco(k.kernel_source, k.kernel_name)
            assert hiprtc.spilled_vgprs(k.kernel_source, k.kernel_name) == 0


def test_a_body_that_would_leave_its_operand_is_refused_on_the_host():
    """Nothing is left to fault on the GPU: an index that leaves its tensor anywhere in the iteration space stops
    the lowering."""
    from deplodock_amd import HipBackend
    from deplodock_amd.emit.errors import LoweringError
    from deplodock_amd.ingest import graph_from_reference_dict

    doc = json.loads((CORPUS / "k_mul_1_reduce.json").read_text())
    nid, node = loop_node(doc)
    node["op_fields"]["body"] = [b.replace("Var(name='a2')", "BinaryExpr(op='+', left=Var(name='a2'), right=Literal(value=1, dtype='int'))") for b in node["op_fields"]["body"]]
    with pytest.raises(LoweringError, match=r"spans \[1, 2048\] outside \[0, 2048\)"):
        HipBackend().compile(graph_from_reference_dict(doc))


def _random_operands(doc: dict, seed: int) -> dict[str, np.ndarray]:
    rng = np.random.default_rng(seed)
    vals = {}
    for name, nd in doc["nodes"].items():
        if nd["op"] == "InputOp" or (nd["op"] == "ConstantOp" and nd["op_fields"].get("value") is None):
            scale = 0.03 if name.startswith("p_") and "norm" not in name else 1.0
            vals[name] = (scale * rng.standard_normal(tuple(nd["output"]["shape"]))).astype(np.float32)
    return vals


@pytest.mark.gpu
@pytest.mark.parametrize("mode", ["raised", "loops"])
@pytest.mark.parametrize("kernel", sorted(p.stem for p in CORPUS.glob("*.json")))
def test_reproducer_on_the_gpu_equals_the_interpreter(device, monkeypatch, kernel, mode):
    """One kernel of the corpus, read from the reference's JSON, lowered (raised to the tiled kernels where it has
    a tiled form, or loop for loop) and run through the launcher library, against the float64 interpretation of
    the same statements on the same fp32 operands."""
    import torch

    if mode == "loops":
        monkeypatch.setenv("EMMY_NEST", "loops")

    from deplodock_amd import HipBackend
    from deplodock_amd.ingest import graph_from_reference_dict
    from oracle import eager

    doc = json.loads((CORPUS / f"{kernel}.json").read_text())
    nid, node = loop_node(doc)
    vals = _random_operands(doc, seed=11)
    operands = {}
    for name in node["inputs"]:
        src = doc["nodes"][name]
        value = src["op_fields"].get("value") if src["op"] == "ConstantOp" else None
        operands[name] = np.full(tuple(src["output"]["shape"]), value) if value is not None else vals[name]
    want = loop_ir.run_vectorised(L.parse_body(node["op_fields"]["body"]), operands, tuple(node["output"]["shape"]))
    be = HipBackend()
    compiled = be.compile(graph_from_reference_dict(doc))
    prog = be.program(compiled, {k: torch.from_numpy(v).to(device) for k, v in vals.items()})
    try:
        prog.run()
        torch.cuda.synchronize()
        ours = prog.output_tensors()[compiled.outputs[0]].clone()
    finally:
        prog.close()
    want_t = torch.from_numpy(want).float()
    rms = float(want_t.pow(2).mean().sqrt())
    eager.assert_close(ours.reshape(want_t.shape), want_t, 1e-4, 1e-4 * max(rms, 1e-30), f"{kernel} vs the float64 interpretation")


@pytest.mark.gpu
@pytest.mark.parametrize("mode", ["raised", "loops"])
def test_the_corpus_chained_on_the_gpu_is_the_decoder_layer(device, monkeypatch, mode):
    """The eleven kernels run in dependency order on the GPU, each feeding the next, reproduce the decoder layer
    they were cut from (PyTorch eager in float64 on the host)."""
    import torch

    if mode == "loops":
        monkeypatch.setenv("EMMY_NEST", "loops")

    from deplodock_amd import HipBackend
    from deplodock_amd.ingest import graph_from_reference_dict
    from oracle import eager

    values, want = corpus_layer_case(seed=3)
    be = HipBackend()

    def run(stmts, operands, node, doc):
        compiled = be.compile(graph_from_reference_dict(doc))
        feed = {k: torch.from_numpy(np.ascontiguousarray(v, dtype=np.float32)).to(device) for k, v in operands.items() if k in compiled.nodes and compiled.nodes[k].op.__class__.__name__ in ("InputOp", "ConstantOp")}
        prog = be.program(compiled, feed)
        try:
            prog.run()
            torch.cuda.synchronize()
            return prog.output_tensors()[compiled.outputs[0]].cpu().numpy().reshape(tuple(node["output"]["shape"]))
        finally:
            prog.close()

    got = run_corpus_chain(values, run)["merged_merged_lift_add_5"]
    want_t = torch.from_numpy(want).float()
    rms = float(want_t.pow(2).mean().sqrt())
    eager.assert_close(torch.from_numpy(got).float(), want_t, 1e-4, 2e-4 * rms, "corpus chain on the GPU vs the eager decoder layer")


# ---------------------------------------------------------------------------------------------------------------
# hand-written nests: the branches of the raise (bias vector, row vector, scalar operands, a k-major weight) and
# nests that must stay loop nests


def _doc(body: list[str], tensors: dict[str, tuple], out: tuple[str, tuple], scalars: dict[str, float] | None = None) -> dict:
    """A reference-format graph around one ``LoopOp``."""
    name, shape = out
    nodes = {}
    for k, shp in tensors.items():
        nodes[k] = {"op": "InputOp", "op_fields": {}, "inputs": [], "output": {"name": k, "shape": list(shp), "dtype": "float32"}}
    for k, v in (scalars or {}).items():
        nodes[k] = {"op": "ConstantOp", "op_fields": {"name": k, "value": v}, "inputs": [], "output": {"name": k, "shape": [1], "dtype": "float32"}}
    nodes[name] = {"op": "LoopOp", "op_fields": {"body": body}, "inputs": [*tensors, *(scalars or {})], "output": {"name": name, "shape": list(shape), "dtype": "float32"}}
    return {"inputs": list(tensors), "outputs": [name], "nodes": nodes}


def _V(n):
    return f"Var(name='{n}')"


_ZERO = "Literal(value=0, dtype='int')"
HAND = {
    # y = max(x @ W.T + bias[n], 0.5) * rowscale[m] - 2.0 : bias vector, scalar operands on either side, row vector
    "bias_clamp_rowscale": (
        _doc(
            ["Load(name='half', input='c_half', index=(" + _ZERO + ",))", "Load(name='two', input='c_two', index=(" + _ZERO + ",))",
             f"Loop(axis=Axis(name='m', extent=70), body=(Loop(axis=Axis(name='n', extent=96), body=(Load(name='bb', input='bias', index=({_V('n')},)), "
             f"Loop(axis=Axis(name='k', extent=200), body=(Load(name='a', input='X', index=({_ZERO}, {_V('m')}, {_V('k')})), Load(name='w', input='W', index=({_V('n')}, {_V('k')})), "
             "Assign(name='p', op=ElementwiseImpl('multiply'), args=('w','a')), Accum(name='s', value='p'))), "
             "Assign(name='t', op=ElementwiseImpl('add'), args=('s','bb')), Assign(name='u', op=ElementwiseImpl('maximum'), args=('half','t')), "
             f"Load(name='r', input='rows', index=({_V('m')}, {_ZERO})), Assign(name='v', op=ElementwiseImpl('multiply'), args=('u','r')), "
             f"Assign(name='y', op=ElementwiseImpl('subtract'), args=('v','two')), Write(output='Y', index=({_ZERO}, {_V('m')}, {_V('n')}), value='y'))),))"],
            {"X": (1, 70, 200), "W": (96, 200), "bias": (96,), "rows": (70, 1)}, ("Y", (1, 70, 96)), {"c_half": 0.5, "c_two": 2.0}),
        ["k_linear", "k_pointwise_fused4"],
    ),
    # the weight stored k-major ([K, N]): read through a transposing index, so it is copied to [N, K] first
    "k_major_weight": (
        _doc(
            [f"Loop(axis=Axis(name='m', extent=64), body=(Loop(axis=Axis(name='n', extent=48), body=(Loop(axis=Axis(name='k', extent=128), body=("
             f"Load(name='a', input='X', index=({_V('m')}, {_V('k')})), Load(name='w', input='Wt', index=({_V('k')}, {_V('n')})), "
             "Assign(name='p', op=ElementwiseImpl('multiply'), args=('a','w')), Accum(name='s', value='p'))), "
             f"Write(output='Y', index=({_V('m')}, {_V('n')}), value='s'))),))"],
            {"X": (64, 128), "Wt": (128, 48)}, ("Y", (64, 48))),
        ["k_gather", "k_linear"],
    ),
    # a batch of products whose first operand is computed in the reduction loop (scaled), whose second is shared by
    # every product, with a bias in the output stage: operand nests + one batched contraction + an output-stage nest
    "batched_computed_operand": (
        _doc(
            ["Load(name='two', input='c_two', index=(" + _ZERO + ",))",
             f"Loop(axis=Axis(name='h', extent=3), body=(Loop(axis=Axis(name='m', extent=40), body=(Loop(axis=Axis(name='n', extent=24), body=("
             f"Loop(axis=Axis(name='k', extent=32), body=(Load(name='a', input='X', index=({_V('h')}, {_V('m')}, {_V('k')})), Assign(name='u', op=ElementwiseImpl('multiply'), args=('a','two')), "
             f"Load(name='w', input='W', index=({_V('n')}, {_V('k')})), Assign(name='p', op=ElementwiseImpl('multiply'), args=('u','w')), Accum(name='s', value='p'))), "
             f"Load(name='bb', input='bias', index=({_V('n')},)), Assign(name='y', op=ElementwiseImpl('add'), args=('s','bb')), "
             f"Write(output='Y', index=({_V('h')}, {_V('m')}, {_V('n')}), value='y'))),)),))"],
            {"X": (3, 40, 32), "W": (24, 32), "bias": (24,)}, ("Y", (3, 40, 24)), {"c_two": 2.0}),
        ["k_operand_a", "k_batched_linear", "k_output_stage"],  # W is one plain load over (n, k): read in place
    ),
    # RMS normalisation with the row element loaded once and squared (the 512-token corpus spells it this way)
    "rms_single_load": (
        _doc(
            ["Load(name='cnt', input='c_cnt', index=(" + _ZERO + ",))", "Load(name='eps', input='c_eps', index=(" + _ZERO + ",))",
             f"Loop(axis=Axis(name='r', extent=50), body=(Loop(axis=Axis(name='c', extent=256), body=(Load(name='x', input='X', index=({_ZERO}, {_V('r')}, {_V('c')})), "
             "Assign(name='sq', op=ElementwiseImpl('multiply'), args=('x','x')), Accum(name='ss', value='sq'))), "
             "Assign(name='mean', op=ElementwiseImpl('divide'), args=('ss','cnt')), Assign(name='me', op=ElementwiseImpl('add'), args=('mean','eps')), Assign(name='rs', op=ElementwiseImpl('rsqrt'), args=('me',)), "
             f"Loop(axis=Axis(name='c2', extent=256), body=(Load(name='x2', input='X', index=({_ZERO}, {_V('r')}, {_V('c2')})), Assign(name='xn', op=ElementwiseImpl('multiply'), args=('x2','rs')), "
             f"Load(name='w', input='W', index=({_V('c2')},)), Assign(name='y', op=ElementwiseImpl('multiply'), args=('w','xn')), Write(output='Y', index=({_ZERO}, {_V('r')}, {_V('c2')}), value='y')))))"],
            {"X": (1, 50, 256), "W": (256,)}, ("Y", (1, 50, 256)), {"c_cnt": 256.0, "c_eps": 1e-5}),
        ["k_rms_norm_reduce"],
    ),
    # a normalisation without a weight and with a maximum instead of a sum: neither tiled form, stays a loop nest
    "max_normalise": (
        _doc(
            [f"Loop(axis=Axis(name='r', extent=37), body=(Loop(axis=Axis(name='c', extent=300), body=(Load(name='x', input='X', index=({_V('r')}, {_V('c')})), "
             "Assign(name='ab', op=ElementwiseImpl('abs'), args=('x',)), Accum(name='mx', value='ab', op=ElementwiseImpl('maximum')))), "
             f"Loop(axis=Axis(name='c2', extent=300), body=(Load(name='x2', input='X', index=({_V('r')}, {_V('c2')})), Assign(name='y', op=ElementwiseImpl('divide'), args=('x2','mx')), "
             f"Write(output='Y', index=({_V('r')}, {_V('c2')}), value='y')))))"],
            {"X": (37, 300)}, ("Y", (37, 300))),
        ["k_Y"],
    ),
}  # fmt: skip


@pytest.mark.parametrize("case", sorted(HAND))
def test_hand_written_nests_take_the_expected_route(launcher_lib, case):
    import re

    from deplodock_amd import HipBackend
    from deplodock_amd.backend.hip import hiprtc
    from deplodock_amd.ingest import graph_from_reference_dict

    doc, labels = HAND[case]
    ks = _kernels(HipBackend().compile(graph_from_reference_dict(doc)))
    assert [re.sub(r"_[0-9a-f]{6}$", "", k.kernel_name) for k in ks] == labels
    for k in ks:
        hiprtc.compile_to_hsaco(k.kernel_source, k.kernel_name)


@pytest.mark.gpu
@pytest.mark.parametrize("mode", ["raised", "loops"])
@pytest.mark.parametrize("case", sorted(HAND))
def test_hand_written_nests_on_the_gpu_equal_the_interpreter(device, monkeypatch, case, mode):
    import torch

    from deplodock_amd import HipBackend
    from deplodock_amd.ingest import graph_from_reference_dict
    from oracle import eager

    if mode == "loops":
        monkeypatch.setenv("EMMY_NEST", "loops")
    doc, _ = HAND[case]
    nid, node = loop_node(doc)
    rng = np.random.default_rng(5)
    vals = {k: rng.standard_normal(tuple(nd["output"]["shape"])).astype(np.float32) for k, nd in doc["nodes"].items() if nd["op"] == "InputOp"}
    operands = {**vals, **{k: np.full((1,), nd["op_fields"]["value"]) for k, nd in doc["nodes"].items() if nd["op"] == "ConstantOp"}}
    stmts = L.parse_body(node["op_fields"]["body"])
    want = loop_ir.run_vectorised(stmts, operands, tuple(node["output"]["shape"]))
    be = HipBackend()
    compiled = be.compile(graph_from_reference_dict(doc))
    prog = be.program(compiled, {k: torch.from_numpy(v).to(device) for k, v in vals.items()})
    try:
        prog.run()
        torch.cuda.synchronize()
        ours = prog.output_tensors()[compiled.outputs[0]].clone()
    finally:
        prog.close()
    want_t = torch.from_numpy(want).float()
    eager.assert_close(ours.reshape(want_t.shape), want_t, 1e-4, 1e-4 * float(want_t.pow(2).mean().sqrt()), f"{case} ({mode}) vs the float64 interpretation")
