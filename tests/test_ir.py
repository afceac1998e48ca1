"""Host logic: knob codecs, expressions, strided views, the scratch planner, HipOp geometry."""

from __future__ import annotations

import numpy as np
import pytest

from deplodock_amd.ir import expr as E
from deplodock_amd.ir import frontend as F
from deplodock_amd.ir.hip import resolve_dim
from deplodock_amd.ir.schedule import ATOMS, ReducePlan, ScheduleError, Stage, TilePlan
from deplodock_amd.passes import views as V


def test_reduce_codec_roundtrip():
    for spec in ("b256", "g4a/b64/r2", "g2k", "r4", "b8"):
        assert ReducePlan.parse(spec).spell() == spec
    assert ReducePlan.parse("") == ReducePlan()
    assert ReducePlan.parse("g4").finalize == "kernel"
    for bad in ("b100", "x3", "b", "b2048"):
        with pytest.raises(ScheduleError):
            ReducePlan.parse(bad)


def test_tile_codec_and_geometry():
    p = TilePlan.parse("a:mfma_32x32x16_bf16/w2x2/f2x3/k4")
    assert (p.tile_m, p.tile_n, p.bk_elems, p.block_threads, p.acc_regs_per_lane) == (128, 192, 64, 256, 96)
    assert p.spell() == "a:mfma_32x32x16_bf16/w2x2/f2x3/k4"
    q = TilePlan.parse("a:mfma_16x16x32_bf16/w4x2/f2x6")
    assert (q.tile_m, q.tile_n, q.bk_elems, q.block_threads) == (128, 192, 32, 512)
    assert q.spell().endswith("f2x6")  # k omitted at 1
    with pytest.raises(ScheduleError):
        TilePlan.parse("n16x16/f4x4")  # scalar tier does not exist on gfx950
    with pytest.raises(ScheduleError):
        TilePlan.parse("a:mma_m16n8k16_bf16/w2x2/f4x8")  # NVIDIA atom
    with pytest.raises(ScheduleError):
        TilePlan.parse("a:mfma_32x32x16_bf16/w8x4/f1x1")  # 2048 threads
    assert all(a.lanes == 64 for a in ATOMS.values())
    assert ATOMS["mfma_32x32x16_bf16"].k_per_lane == 8 and ATOMS["mfma_16x16x32_bf16"].acc_per_lane == 4


def test_stage_codec():
    assert Stage.parse("d2/sync").spell() == "d2/sync"
    assert Stage.parse("d3/cp/ring").spell() == "d3/dl/ring"  # the reference's cp token maps to direct-to-LDS
    assert Stage.parse("d2/dl/p2").reg_depth == 2
    assert Stage.parse("") is None
    with pytest.raises(ScheduleError):
        Stage.parse("d2/tma")
    with pytest.raises(ScheduleError):
        Stage.parse("d9/sync")


def test_expr_render_and_evaluate_agree_on_rounding_points():
    x = E.Var("x")
    e = E.Round("bf16", E.Var("w") * E.Round("bf16", x * E.Un("rsqrt", E.Var("ss") / 4.0 + 1e-6)))
    xs = np.array([1.0, 2.0, 3.0, 4.0], dtype=np.float32)
    got = E.evaluate(e, {"x": xs, "w": np.float32(1.5), "ss": np.float32((xs * xs).sum())})
    import torch

    t = torch.from_numpy(xs)
    want = (torch.tensor(1.5).bfloat16() * (t * torch.rsqrt((t * t).mean() + 1e-6)).bfloat16()).float().numpy()
    np.testing.assert_array_equal(got, want)
    text = E.render(e, {"x": "xv", "w": "wv", "ss": "acc"})
    assert text.count("emh_round_bf16") == 2 and "rsqrtf" in text
    assert E.variables(e) == {"x", "w", "ss"}


def test_float_literal_roundtrips():
    for v in (1e-6, 0.1, 1 / 3, 2048.0, -1e30):
        lit = E.float_literal(v)
        assert float.fromhex(lit[:-1]) == float(np.float32(v))


def test_resolve_dim():
    assert resolve_dim((4, "seq_len", lambda env: (env["seq_len"] + 15) // 16), {"seq_len": 100}) == 4 * 100 * 7
    assert resolve_dim(7, {}) == 7
    with pytest.raises(KeyError):
        resolve_dim(("unknown",), {})


def test_views_transpose_reshape_slice():
    v = V.View("b", 0, (1, 512, 2048), V.contiguous_strides((1, 512, 2048)), None)
    v = V.apply_layout(v, F.ViewOp(shape=(1, 512, 16, 128)), (1, 512, 16, 128))
    assert v.strides == (0, 2048, 128, 1)
    t = V.apply_layout(v, F.TransposeOp(dim0=1, dim1=2), (1, 16, 512, 128))
    assert t.shape == (1, 16, 512, 128) and t.strides == (0, 128, 2048, 1)
    assert not t.is_contiguous()
    s = V.apply_layout(t, F.SliceOp(dim=3, start=64, end=128), (1, 16, 512, 64))
    assert s.offset == 64 and s.shape[-1] == 64
    with pytest.raises(V.NotViewable):
        V.apply_layout(t, F.ViewOp(shape=(1, 16 * 512, 128)), (1, 16 * 512, 128))  # a transposed tensor cannot be flattened in place
    back = V.apply_layout(V.apply_layout(t, F.TransposeOp(dim0=1, dim1=2), (1, 512, 16, 128)), F.ViewOp(shape=(1, 512, 2048)), (1, 512, 2048))
    assert back.is_contiguous()
    assert v.collapse_leading(1) == (512 * 16, 128)
    assert t.collapse_leading(1) is None


def test_scratch_planner_never_overlaps_live_buffers():
    from deplodock_amd.backend.hip.program import _Launch, compute_live_intervals, plan_offsets

    launches = [
        _Launch("n0", "k", ("in", "a"), (), (), 0, ()),
        _Launch("n1", "k", ("a", "b"), (), (), 0, ()),
        _Launch("n2", "k", ("b", "c"), (), (), 0, ()),
        _Launch("n3", "k", ("c", "a2"), (), (), 0, ()),
    ]
    sizes = {"a": 1000, "b": 4096, "c": 300, "a2": 5000}
    iv = compute_live_intervals(list(sizes), launches)
    assert iv == {"a": (0, 1), "b": (1, 2), "c": (2, 3), "a2": (3, 3)}
    offsets, total = plan_offsets(iv, sizes)
    for x in sizes:
        for y in sizes:
            if x < y and not (iv[x][1] < iv[y][0] or iv[y][1] < iv[x][0]):
                ax, ay = offsets[x], offsets[y]
                assert ax + sizes[x] <= ay or ay + sizes[y] <= ax, (x, y)
    assert total < sum(-(-s // 256) * 256 for s in sizes.values())  # dead intervals share memory
    assert all(o % 256 == 0 for o in offsets.values())


def test_knob_env_grammar(monkeypatch):
    from deplodock_amd import config

    monkeypatch.setenv("EMMY_KNOBS", "REDUCE=b128, tile=a:mfma_32x32x16_bf16/w2x2/f2x2")
    assert config.knob_raw("reduce") == "b128"
    assert config.knob_raw("TILE").startswith("a:mfma")
    monkeypatch.setenv("EMMY_REDUCE", "b64")  # the dedicated variable wins over the aggregate
    assert config.knob_raw("REDUCE") == "b64"
    monkeypatch.setenv("EMMY_KNOBS", "oops")
    with pytest.raises(ValueError):
        config.knobs_aggregate()
