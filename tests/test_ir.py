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
    assert text.count("((float)(((__bf16)(") == 2 and "rsqrtf" in text  # the render target's fp32 -> bf16 -> fp32 round trip
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


# -- render target ----------------------------------------------------------------------------------


def test_hip_render_target_implements_the_protocol_and_spells_gfx950_types():
    from deplodock_amd.backend.hip.render_target import HipRenderTarget
    from deplodock_amd.render_target import RenderTarget, current

    t = HipRenderTarget()
    assert isinstance(t, RenderTarget) and isinstance(current(), HipRenderTarget)
    assert [t.type_name(d) for d in ("f32", "bf16", "f16", "i32")] == ["float", "__bf16", "_Float16", "int"]
    assert t.literal("0.0f", "f32") == "0.0f" and t.literal("0.0f", "bf16") == "((__bf16)(0.0f))"
    assert t.convert("v", "f32", "f32") == "v" and t.convert("v", "f32", "f16") == "((_Float16)(v))"
    assert t.intrinsic("exp", "f32") == "expf" and t.intrinsic("fmax", "f32") == "fmaxf" and t.intrinsic("rsqrt", "f32") == "rsqrtf"
    assert t.intrinsic("exp", "bf16") == "exp"  # no 16-bit forms: the renderer widens to fp32 and rounds back
    assert t.has_native_op("exp", "f32") and t.has_native_op("add", "f32") and not t.has_native_op("add", "bf16")
    assert t.vector_type("f32", 4) == ("f32x4", "float") and t.vector_type("bf16", 8) == ("bf16x8", "__bf16")
    assert t.vector_type("f32", 1) == ("float", "float") and t.vector_type("bf16", 3) is None and t.vector_type("i32", 4) is None
    with pytest.raises(KeyError):
        t.type_name("f64")


def test_emitters_take_their_spellings_from_the_installed_render_target():
    """Another implementation of the protocol changes the emitted text without touching an emitter: every type,
    vector, conversion and intrinsic spelling in a row kernel and a contraction comes from the target."""
    from deplodock_amd import render_target
    from deplodock_amd.backend.hip.render_target import HipRenderTarget
    from deplodock_amd.dtype import BF16, F32
    from deplodock_amd.emit.contraction import emit_contraction
    from deplodock_amd.emit.reduce import emit_row_reduce
    from deplodock_amd.ir.schedule import Stage, TilePlan
    from deplodock_amd.ir.tile import Contraction, RowReduce, Stat

    class Renamed(HipRenderTarget):
        def type_name(self, dtype):
            return {"f32": "my_f32", "bf16": "my_bf16"}.get(dtype, super().type_name(dtype))

        def vector_type(self, dtype, n):
            got = super().vector_type(dtype, n)
            return None if got is None else ("my_" + got[0], self.type_name(dtype))

        def intrinsic(self, op, dt):
            return "my_" + super().intrinsic(op, dt)

    x = E.Var("x")
    row = RowReduce(rows=8, cols=256, x="X", x_dtype=F32, out="out", out_dtype=F32, stats=(Stat("ss", "sum", x * x),),
                    project=x * E.Un("rsqrt", E.Var("ss") / 256.0 + 1e-6), reduce=ReducePlan(coop=64))  # fmt: skip
    gemm = Contraction(m=64, n=64, k=64, a="x", b="w", out="y", in_dtype=BF16, out_dtype=BF16, tile=TilePlan.parse("a:mfma_16x16x32_bf16/w2x2/f2x2/k2"), stage=Stage.parse("d2/sync"))
    plain = emit_row_reduce(row, "k_r").kernel_source, emit_contraction(gemm, "k_c").kernel_source
    old = render_target.use(Renamed())
    try:
        renamed = emit_row_reduce(row, "k_r").kernel_source, emit_contraction(gemm, "k_c").kernel_source
    finally:
        render_target.use(old)
    assert "const float* __restrict__ x" in plain[0] and "rsqrtf(" in plain[0] and "f32x4" in plain[0]
    assert "const my_f32* __restrict__ x" in renamed[0] and "my_rsqrtf(" in renamed[0] and "my_f32x4" in renamed[0]
    assert "const __bf16* __restrict__ A" in plain[1] and "bf16x8 fw[2]" in plain[1]
    assert "const my_bf16* __restrict__ A" in renamed[1] and "my_bf16x8 fw[2]" in renamed[1] and "my_f32x4 acc" in renamed[1]
    assert emit_row_reduce(row, "k_r").kernel_source == plain[0]  # and back
