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
