"""Tune database, shape keys and the way the schedule consults them."""

import pytest
import torch
from torch import nn

from deplodock_amd import HipBackend, trace_module
from deplodock_amd.ir.hip import HipOp
from deplodock_amd.tune import FAMILY_KNOBS, TuneDB, candidate_rounds, pinned, shape_key
from oracle import eager


def kernels(compiled):
    return [n.op for n in compiled.nodes.values() if isinstance(n.op, HipOp)]


def test_db_keeps_the_fastest_entry_per_key(tmp_path):
    db = TuneDB(tmp_path / "t.db")
    assert db.lookup("contraction/x") == {} and db.lookup(None) == {}
    db.store("contraction/x", {"TILE": "a", "STAGE": "d2/sync"}, 10.0, 12.0)
    db.store("contraction/x", {"TILE": "b"}, 11.0, 12.0)  # slower: ignored
    assert db.lookup("contraction/x") == {"TILE": "a", "STAGE": "d2/sync"}
    db.store("contraction/x", {"TILE": "c"}, 9.0, 12.0)
    assert db.lookup("contraction/x") == {"TILE": "c"}
    db.close()
    again = TuneDB(tmp_path / "t.db")
    assert again.rows() == [("contraction/x", {"TILE": "c"}, 9.0, 12.0)]
    assert TuneDB(tmp_path / "t.db", arch="gfx942").lookup("contraction/x") == {}


def test_shape_keys_separate_what_the_schedule_depends_on(launcher_lib):
    from deplodock_amd.passes.fuse import fuse

    block = fuse(trace_module(*(lambda c: (c.module, c.inputs))(eager.qwen3_block_case(seq=64))))
    keys = [shape_key(n.op.body) for n in block.nodes.values() if hasattr(n.op, "body")]
    assert len(keys) == 5 and len(set(keys)) == 5
    norm = fuse(trace_module(*(lambda c: (c.module, c.inputs))(eager.rms_norm_case())))
    keys += [shape_key(n.op.body) for n in norm.nodes.values() if hasattr(n.op, "body")]
    assert keys[-1] == "row_reduce/r32/c2048/f32>f32/s1/rot0"
    fams = {k.split("/")[0] for k in keys}
    assert fams == set(FAMILY_KNOBS)
    # the merged q/k/v projection carries the head norm + rotary epilogue over 128-column groups: its own key
    assert "contraction/m64/n4096/k1024/bf16>bf16/g0/p0/a1/e128" in keys and "contraction/m64/n3072/k1024/bf16>bf16/g1/p0/a1" in keys
    assert "contraction/m64/n1024/k2048/bf16>bf16/g0/p1/a0" in keys
    assert any(k.startswith("flash/b1/hq16/hkv8/sq64/skv64/d128/c1") for k in keys)


def test_schedule_takes_pins_from_the_db_and_env_wins(tmp_path, monkeypatch, launcher_lib):
    for var in ("EMMY_TILE", "EMMY_STAGE", "EMMY_KNOBS", "EMMY_REDUCE"):
        monkeypatch.delenv(var, raising=False)
    case = eager.linear_case(m=128)
    graph = trace_module(case.module, case.inputs)
    default = kernels(HipBackend().compile(graph))[0].knobs["TILE"]
    db = TuneDB(tmp_path / "t.db")
    tuned = "a:mfma_16x16x32_bf16/w2x2/f2x2/k4"
    assert tuned != default
    db.store("contraction/m128/n3072/k1024/bf16>bf16/g0/p0/a0", {"TILE": tuned, "STAGE": "d3/dl"}, 1.0)
    k = kernels(HipBackend(tune_db=db).compile(graph))[0]
    assert k.knobs["TILE"] == tuned and k.knobs["STAGE"] == "d3/dl"
    # another shape is not affected
    other = eager.linear_case(m=16)
    assert kernels(HipBackend(tune_db=db).compile(trace_module(other.module, other.inputs)))[0].knobs["TILE"] != tuned
    # an environment pin is authoritative over the database
    monkeypatch.setenv("EMMY_TILE", "a:mfma_16x16x32_bf16/w1x2/f2x2/k4")
    assert kernels(HipBackend(tune_db=db).compile(graph))[0].knobs["TILE"] == "a:mfma_16x16x32_bf16/w1x2/f2x2/k4"
    monkeypatch.delenv("EMMY_TILE")
    # a stored pin the emitter could not realise degrades to the heuristic pick
    db.store("contraction/m128/n3072/k1024/bf16>bf16/g0/p0/a0", {"TILE": "a:mfma_32x32x16_bf16/w4x4/f8x8/k4"}, 0.5)
    assert kernels(HipBackend(tune_db=db).compile(graph))[0].knobs["TILE"] == default
    # path form of the constructor argument
    assert kernels(HipBackend(tune_db=str(tmp_path / "t.db")).compile(graph))[0].knobs["TILE"] == default


def test_unrealisable_tile_pin_degrades_per_kernel(monkeypatch, launcher_lib):
    """A pin that fits one contraction of a graph and not another must not fail the lowering."""
    monkeypatch.setenv("EMMY_TILE", "a:mfma_32x32x16_bf16/w2x4/f4x2/k4")  # 256x256 tile, 8 waves, 64-deep slabs
    monkeypatch.setenv("EMMY_STAGE", "d4/dl")  # 4 x 64 KiB of slabs: does not fit
    k = kernels(HipBackend().compile(trace_module(*(lambda c: (c.module, c.inputs))(eager.linear_case(m=2048)))))[0]
    assert k.knobs["TILE"] == "a:mfma_32x32x16_bf16/w2x4/f4x2/k4" and k.knobs["STAGE"] == "d2/dlm"  # two slabs of it do (eight MFMAs a step: requests spread among the last step's)


def test_candidate_rounds_cover_every_family_once():
    rounds = candidate_rounds({"contraction", "row_reduce", "flash"})
    assert len(rounds) == 79  # the longest family: 23 tiles x 3 stagings + the ten tile-less few-row forms (waves x columns)
    assert {"TILE", "STAGE", "REDUCE", "NT", "FLASH"} <= set(rounds[0])
    assert "FLASH" not in rounds[-1] and "TILE" in rounds[-1]
    assert candidate_rounds({"row_reduce"}) and all(set(r) == {"REDUCE", "NT"} for r in candidate_rounds({"row_reduce"}))


def test_fp32_contractions_sweep_fp32_atoms_in_rounds_of_their_own():
    from deplodock_amd.ir.schedule import TilePlan
    from deplodock_amd.tune import STAGE_SWEEP_F32, TILE_SWEEP_F32, _family

    assert _family("contraction/m512/n3072/k1024/f32>f32/g0/p0/a0") == "contraction_f32" and _family("contraction/m512/n3072/k1024/bf16>bf16/g0/p0/a0") == "contraction"
    only = candidate_rounds({"contraction_f32"})
    assert len(only) == len(TILE_SWEEP_F32) * len(STAGE_SWEEP_F32) and all(set(r) == {"TILE", "STAGE"} for r in only)
    assert all(TilePlan.parse(r["TILE"]).atom.dtype == "f32" for r in only)
    mixed = candidate_rounds({"contraction", "contraction_f32"})
    assert len(mixed) == 79 + len(only) and mixed[79:] == only  # appended, never merged with the 16-bit pins of a round
    # attention on fp32 atoms likewise sweeps its own forms
    assert _family("flash/b1/hq16/hkv8/sq512/skv512/d128/c1/f32") == "flash_f32" and _family("flash/b1/hq16/hkv8/sq512/skv512/d128/c1/bf16") == "flash"
    f32_flash = candidate_rounds({"flash_f32"})
    assert f32_flash and all(set(r) == {"FLASH"} and r["FLASH"].startswith("f32/") for r in f32_flash)


@pytest.mark.gpu
def test_tuning_an_fp32_contraction_keeps_fp32_pins(device, tmp_path):
    """The sweep over an fp32 matmul: candidates keep their pins (fp32 atoms), outputs stay equal, and whatever wins is
    at least as fast as the default."""
    import torch

    from deplodock_amd.tune import tune_graph

    class Mm(torch.nn.Module):
        def forward(self, a, b):
            return a @ b.transpose(-1, -2)

    torch.manual_seed(3)
    a, b = torch.randn(512, 512), torch.randn(768, 512)  # (enough 32x32 tiles to cover the CUs: the launch is not split)
    be = HipBackend()
    graph = trace_module(Mm().eval(), (a, b))
    base = be.compile(graph)
    data = dict(zip(base.inputs, (a.to(device), b.to(device))))
    db = TuneDB(tmp_path / "tune.db")
    try:
        (res,) = tune_graph(graph, be, db, input_data=data, warmup=1, num_iters=3, max_rounds=12)
    finally:
        db.close()
    assert res.tried >= 4 and not res.rejected and res.best_us <= res.baseline_us
    assert "_f32/" in res.best_knobs["TILE"]


def test_pinned_context_restores_the_environment(monkeypatch):
    monkeypatch.setenv("EMMY_TILE", "x")
    monkeypatch.setenv("EMMY_KNOBS", "REDUCE=b64")
    with pinned({"TILE": "y"}):
        import os

        assert "EMMY_TILE" not in os.environ and os.environ["EMMY_KNOBS"] == "TILE=y"
    import os

    assert os.environ["EMMY_TILE"] == "x" and os.environ["EMMY_KNOBS"] == "REDUCE=b64"


@pytest.mark.gpu
def test_tune_graph_finds_and_stores_pins_the_next_compile_uses(tmp_path):
    from deplodock_amd.tune import tune_graph

    class TwoOps(nn.Module):
        def __init__(self):
            super().__init__()
            self.lin = nn.Linear(512, 768, bias=False)
            self.norm = nn.RMSNorm(768)

        def forward(self, x):
            return self.norm(self.lin(x))

    torch.manual_seed(0)
    mod = TwoOps().bfloat16().eval()
    x = torch.randn(256, 512).bfloat16()
    graph = trace_module(mod, (x,))
    db = TuneDB(tmp_path / "t.db")
    be = HipBackend()
    report = tune_graph(graph, be, db, input_data={graph.inputs[0]: x.cuda()}, warmup=1, num_iters=3, max_rounds=6)
    assert {r.key.split("/")[0] for r in report} == {"contraction", "row_reduce"}
    assert all(r.tried >= 1 and r.best_us <= r.baseline_us and not r.rejected for r in report)
    stored = dict((k, knobs) for k, knobs, _, _ in db.rows())
    tuned = HipBackend(tune_db=db).compile(graph)
    for op in kernels(tuned):
        key = shape_key(op.source.body)
        for knob, value in stored.get(key, {}).items():
            assert str(op.knobs[knob]) == value
    want = mod.cuda()(x.cuda()).float()
    res, _ = HipBackend(tune_db=db).run(tuned, input_data={graph.inputs[0]: x.cuda()})
    got = torch.from_numpy(res.outputs[tuned.outputs[0]].view("int16").copy()).view(torch.bfloat16).float().cuda()
    eager.assert_close(got.reshape(want.shape), want, 2e-2, 2e-2, "tuned program vs eager")
