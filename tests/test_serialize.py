"""JSON form of traced and lowered graphs."""

import json

import pytest
import torch

from deplodock_amd import HipBackend, serialize, trace_module
from deplodock_amd.cli import main
from deplodock_amd.ir.hip import HipOp
from deplodock_amd.passes.fuse import fuse
from oracle import eager


def hip_ops(g):
    return [g.nodes[n].op for n in g.topological_order() if isinstance(g.nodes[n].op, HipOp)]


def test_traced_graph_round_trips_and_lowers_to_the_same_kernels(launcher_lib):
    case = eager.qwen3_block_case(seq=64)
    g = trace_module(case.module, case.inputs)
    d = json.loads(json.dumps(serialize.graph_to_dict(g)))
    assert d["stage"] == "torch" and d["format"] == serialize.FORMAT
    g2 = serialize.graph_from_dict(d)
    assert g2.pretty_print() == g.pretty_print() and g2.inputs == g.inputs and g2.outputs == g.outputs
    a, b = hip_ops(HipBackend().compile(g)), hip_ops(HipBackend().compile(g2))
    assert [k.kernel_name for k in a] == [k.kernel_name for k in b]  # names hash the source: identical kernels


def test_lowered_graph_round_trips_field_for_field(launcher_lib, tmp_path):
    case = eager.qwen3_block_case(seq=64)
    c = HipBackend().compile(trace_module(case.module, case.inputs))
    path = tmp_path / "block.json"
    serialize.save(c, path)
    c2 = serialize.load(path)
    assert c2.stage == "hip"
    for x, y in zip(hip_ops(c), hip_ops(c2)):
        for f in ("kernel_source", "kernel_name", "arg_order", "grid", "block", "lds_bytes", "zero_outputs", "runtime_args", "algo_bytes", "algo_flops", "knobs"):
            assert getattr(x, f) == getattr(y, f), f
    stacked = [n for n in c2.nodes.values() if n.hints.get("stacked")]
    assert len(stacked) == 3 and all(isinstance(n.hints["stacked"].parts, tuple) for n in stacked)
    data = serialize.random_inputs(c2, seed=1)
    need = {n.id for n in c2.nodes.values() if type(n.op).__name__ in ("InputOp", "ConstantOp")}
    assert set(data) == need and all(tuple(data[k].shape) == tuple(c2.nodes[k].output.shape) for k in data)
    again = serialize.random_inputs(c2, seed=1)
    assert all(torch.equal(data[k], again[k]) for k in data)


def test_runtime_int_graph_round_trips_with_its_symbolic_parts(launcher_lib, tmp_path):
    """A lowering with a symbolic axis keeps, through JSON: ``seq_len`` / affine dims in shapes, launch-time grid
    factors, the trailing int arguments and the traced size."""
    from deplodock_amd.ir.sym import resolve
    from deplodock_amd.ir.hip import resolve_dim
    from deplodock_amd.ir.sym import Affine, CeilDiv, XcdRounds

    case = eager.qwen3_block_case(seq=64)
    dyn = {"x": {1: "seq_len"}, "cos": {1: "seq_len"}, "sin": {1: "seq_len"}}
    c = HipBackend().compile(trace_module(case.module, case.inputs, dynamic_shapes=dyn))
    assert c.symbolic == "seq_len"
    serialize.save(c, tmp_path / "sym.json")
    c2 = serialize.load(tmp_path / "sym.json")
    assert c2.symbolic == "seq_len" and c2.dynamic.hints == {"seq_len": 64}
    kinds = set()
    for x, y in zip(hip_ops(c), hip_ops(c2)):
        assert x.grid == y.grid and x.runtime_args == y.runtime_args == ("seq_len",) and x.kernel_source == y.kernel_source
        kinds |= {type(f) for dim in y.grid for f in (dim if isinstance(dim, tuple) else (dim,))}
        for s_ in (7, 64, 513):
            assert [resolve_dim(d, {"seq_len": s_}) for d in x.grid] == [resolve_dim(d, {"seq_len": s_}) for d in y.grid]
    assert {CeilDiv, XcdRounds} <= kinds
    for nid in c.nodes:
        assert c.nodes[nid].output.shape == c2.nodes[nid].output.shape
        assert [resolve(d, {"seq_len": 200}) for d in c2.nodes[nid].output.shape] == [resolve(d, {"seq_len": 200}) for d in c.nodes[nid].output.shape]
    assert any(isinstance(d, (str, Affine)) for n in c2.nodes.values() for d in n.output.shape)
    assert tuple(serialize.random_inputs(c2)["x"].shape) == (1, 64, 1024)
    assert tuple(serialize.random_inputs(c2, sizes={"seq_len": 200})["cos"].shape)[1] == 200
    assert HipBackend().variant(c2, {"x": torch.zeros(1, 200, 1024)}) is c2  # one lowering serves every size


def test_tile_stage_has_no_json_form():
    case = eager.rms_norm_case()
    with pytest.raises(serialize.SerializeError, match="TileOp"):
        serialize.graph_to_dict(fuse(trace_module(case.module, case.inputs)))
    with pytest.raises(serialize.SerializeError, match="format"):
        serialize.graph_from_dict({"format": 99})


def test_compile_writes_a_reproducer(tmp_path, capsys):
    path = tmp_path / "k.json"
    main(["compile", "--json", str(path), "-c", "nn.RMSNorm(2048)(torch.randn(1,32,2048))"])
    capsys.readouterr()
    d = json.loads(path.read_text())
    assert d["stage"] == "hip" and [n["op"]["type"] for n in d["nodes"]] == ["InputOp", "ConstantOp", "HipOp"]
    main(["compile", "--ir", "torch", "--json", str(path), "-c", "nn.RMSNorm(2048)(torch.randn(1,32,2048))"])
    assert json.loads(path.read_text())["stage"] == "torch"


@pytest.mark.gpu
def test_run_ir_replays_both_stages(tmp_path, capsys):
    hip, traced = tmp_path / "hip.json", tmp_path / "torch.json"
    expr = "x = torch.randn(64, 512); torch.softmax(x * 0.5, -1)"
    main(["compile", "--json", str(hip), "-c", expr])
    main(["compile", "--ir", "torch", "--json", str(traced), "-c", expr])
    capsys.readouterr()
    main(["run", "--ir", str(hip), "--bench", "--iters", "5", "--warmup", "1"])
    out = capsys.readouterr().out
    assert out.startswith("RAN ") and "k_softmax_reduce" in out and "program:" in out
    main(["run", "--ir", str(traced)])
    assert capsys.readouterr().out.startswith("RAN ")


@pytest.mark.gpu
def test_reloaded_runtime_int_graph_runs_at_other_sizes(device, tmp_path, capsys):
    """The reloaded symbolic lowering against eager at sizes it was not traced at, and ``run --ir --at``."""
    case = eager.qwen3_block_case(seq=64)
    dyn = {"x": {1: "seq_len"}, "cos": {1: "seq_len"}, "sin": {1: "seq_len"}}
    be = HipBackend()
    c = be.compile(trace_module(case.module, case.inputs, dynamic_shapes=dyn))
    serialize.save(c, tmp_path / "sym.json")
    c2 = serialize.load(tmp_path / "sym.json")
    weights = {k: v.to(device) for k, v in be.bind(c, {}).items()}
    for seq in (200, 33):
        other = eager.qwen3_block_case(seq=seq)
        data = {**weights, **{n: t.to(device) for n, t in zip(c2.inputs, other.inputs)}}
        prog = be.program(c2, data)
        try:
            prog.run()
            torch.cuda.synchronize()
            ours = prog.output_tensors()[c2.outputs[0]].clone()
        finally:
            prog.close()
        want = eager.run_eager(other, device)
        exact = eager.run_eager_fp32(other, device)
        eager.assert_mean_error_within_baseline(ours.reshape(want.shape), want, exact, 1.5, f"reloaded runtime-int block S={seq}")
    main(["run", "--ir", str(tmp_path / "sym.json"), "--at", "seq_len=100"])
    out = capsys.readouterr().out
    assert out.startswith("RAN ") and "(1, 100, 1024)" in out


@pytest.mark.gpu
def test_reloaded_lowered_graph_computes_what_the_original_does(device, tmp_path):
    case = eager.linear_case(m=128)
    be = HipBackend()
    c = be.compile(trace_module(case.module, case.inputs))
    serialize.save(c, tmp_path / "lin.json")
    c2 = serialize.load(tmp_path / "lin.json")
    x = case.inputs[0].to(device)
    w = case.module.weight.detach().to(device)
    (wid,) = [nid for nid, _ in c2.constant_ops()]
    prog = be.program(c2, {c2.inputs[0]: x, wid: w})
    try:
        prog.run()
        torch.cuda.synchronize()
        ours = prog.output_tensors()[c2.outputs[0]]
        eager.assert_close(ours, eager.run_eager(case, device), case.rtol, case.atol, "reloaded linear vs eager")
    finally:
        prog.close()


def test_loop_ir_and_matmul_graphs_round_trip(launcher_lib):
    """A graph read from the reference's Loop-IR JSON (its statements are nested dataclasses) and a traced graph with
    ``MatmulOp`` keep their JSON form: the reloaded graph lowers to the same kernels, name for name."""
    import json
    from pathlib import Path

    import torch
    from torch import nn

    from deplodock_amd import HipBackend, serialize, trace_module
    from deplodock_amd.ingest import load_reference_graph
    from deplodock_amd.ir.hip import HipOp

    class Mm(nn.Module):
        def forward(self, a, b):
            return a @ b

    def kernels(g):
        return [n.op.kernel_name for n in HipBackend().compile(g).nodes.values() if isinstance(n.op, HipOp)]

    corpus = Path(__file__).parent / "golden" / "loop_ir"
    graphs = [load_reference_graph(corpus / f"{k}.json") for k in ("k_mul_1_reduce", "k_scaled_dot_product_attention_masked_reduce", "k_add_3_reduce")]
    graphs.append(trace_module(Mm().eval(), (torch.randn(4, 8, 16), torch.randn(16, 12))))
    for g in graphs:
        again = serialize.graph_from_dict(json.loads(json.dumps(serialize.graph_to_dict(g))))
        assert kernels(again) == kernels(g)
    with pytest.raises(serialize.SerializeError, match="unknown Loop-IR statement"):
        serialize._dec({"$loop": ["Exec", "x"]})
