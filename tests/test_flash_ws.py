"""The software-pipelined attention kernels (``FLASH=.../ws``: four consumer waves and four staging waves;
``.../sp``: eight consumer waves that stage for themselves): their ring protocol replayed on the CPU, and parity
on the GPU through the C-ABI for every shape of the forms (row groups x key-split groups, mirrored pairs, ragged
and unmasked lengths, head_dim 64, the full benchmark size)."""

from __future__ import annotations

import math

import pytest
import torch
from torch import nn

from deplodock_amd import HipBackend, trace_module
from deplodock_amd.dtype import BF16
from deplodock_amd.emit.flash_ws import emit_flash_ws, ws_lds_plan, ws_supported
from deplodock_amd.ir.hip import HipOp
from deplodock_amd.ir.tile import Flash
from oracle import eager


def _body(s=2048, d=128, waves=2, kvs=2, causal=True, pair=False, hq=16, hkv=8):
    qs, ks = (hq * s * d, s * d, d), (hkv * s * d, s * d, d)
    return Flash(batch=1, q_heads=hq, kv_heads=hkv, q_len=s, kv_len=s, head_dim=d, q="q", k="k", v="v", out="o", dtype=BF16, scale=1 / math.sqrt(d), causal=causal,
                 q_strides=qs, k_strides=ks, v_strides=ks, o_strides=qs, waves=waves, block_kv=32, kv_split=kvs, pair=pair, ws=True)  # fmt: skip


# -- the ring protocol, replayed ------------------------------------------------------------------------------


def _replay(ring: int, nsub: int, nacts: list[int], *, k_ahead: int | None = None, v_ahead: int | None = None, lag: int | None = None) -> None:
    """The schedule the kernel's text spells, as events between workgroup barriers.

    Barriers, in order: P, B0, then one at the end of every iteration t = 0 .. nsub - 1, then C.  Positions on a time
    axis: P = -1, B0 = -0.5, the end of iteration t = t.
    Stagers: "iteration" tau (the prologue, before P, is tau = -ring .. -1; iteration t >= 0 runs between the barrier
    before it and the one that ends it) issues V(tau + v_ahead) then K(tau + k_ahead), where they exist
    (``v_ahead = ring - 2``, ``k_ahead = ring``).  Requests retire in issue order; the barrier that ends iteration e
    (P for e = -1) is passed with at most the requests of iterations e - lag + 1 .. e outstanding (``lag = ring - 2``).
    Data of sub-step s lives in slot s % ring of its operand's ring.
    Consumers (one per entry of ``nacts``: its number of active sub-blocks): scores of sub-block 0 between P and B0;
    iteration t < nact - 1 reads V(t - 1) and K(t + 1); the last active sub-block t = nact - 1 reads V(t - 1) in its
    iteration and V(t) after the barrier that ends it, before it passes another.

    Checked: every role passes the same number of barriers; a read never starts before the barrier at which its data
    is guaranteed; a slot is never requested before the barrier that follows the last read of its old content."""
    k_ahead = ring if k_ahead is None else k_ahead
    v_ahead = ring - 2 if v_ahead is None else v_ahead
    lag = ring - 2 if lag is None else lag

    def start_of(t: int) -> float:  # the barrier an iteration (or prologue step) starts after
        return -2.0 if t < 0 else (-0.5 if t == 0 else float(t - 1))

    issued = []  # (operand, sub-step, tau)
    for tau in range(-ring, nsub):
        if 0 <= tau + v_ahead < nsub:
            issued.append(("V", tau + v_ahead, tau))
        if 0 <= tau + k_ahead < nsub:
            issued.append(("K", tau + k_ahead, tau))
    assert sorted(sub for o, sub, _ in issued if o == "K") == list(range(nsub)) and sorted(sub for o, sub, _ in issued if o == "V") == list(range(nsub))
    landed = {(o, sub): float(max(tau + lag, -1)) for o, sub, tau in issued}  # first barrier e with tau <= e - lag
    assert all(v <= nsub - 1 for v in landed.values()), "a request is still outstanding after the last iteration's barrier"
    reads = []  # (operand, sub-step, barrier the read starts after, barrier it ends before)
    counts = []
    for nact in nacts:
        count = 2  # P, B0
        if nact > 0:
            reads.append(("K", 0, -1.0, -0.5))
        for t in range(nact):
            lo, hi = start_of(t), float(t)
            if t > 0:
                reads.append(("V", t - 1, lo, hi))
            if t + 1 < nact:
                reads.append(("K", t + 1, lo, hi))
            count += 1
        if nact > 0:
            reads.append(("V", nact - 1, float(nact - 1), float(nact)))  # after its iteration's barrier, before the next one it passes (C, at position nsub, for the last)
        count += nsub - nact
        count += 1  # C
        counts.append(count)
    assert set(counts) == {nsub + 3}, (counts, nsub)  # what the stagers pass: P, B0, nsub, C
    for o, sub, lo, hi in reads:
        assert landed[(o, sub)] <= lo, f"{o}({sub}) is read after barrier {lo} but guaranteed only at {landed[(o, sub)]} (ring {ring}, nsub {nsub})"
        for o2, s2, tau in issued:
            if o2 == o and s2 != sub and s2 % ring == sub % ring and s2 > sub:
                assert start_of(tau) >= hi, f"{o}({s2}) is requested in iteration {tau} into the slot {o}({sub}) is still read from (until barrier {hi})"


@pytest.mark.parametrize("ring", [2, 3, 4])
def test_ring_protocol_never_overwrites_a_live_slot_and_never_reads_before_landing(ring):
    for nsub in range(1, 14):
        for nact in range(0, nsub + 1):
            _replay(ring, nsub, [nsub, nact, max(nact - 1, 0), 0])


@pytest.mark.parametrize("mutant", [dict(k_ahead=5), dict(v_ahead=3), dict(lag=3), dict(k_ahead=3)])
def test_replay_trips_on_schedules_that_are_wrong(mutant):
    """The check has teeth: K or V requested one iteration too early (into a slot that is still read), a landing wait
    one iteration too lax (a read before its data is guaranteed), K requested one iteration too late (not there when
    its scores are due) — each must fail for a ring of four."""
    with pytest.raises(AssertionError):
        for nsub in range(1, 14):
            _replay(4, nsub, [nsub, nsub // 2], **mutant)


def test_emitted_text_spells_the_replayed_schedule(launcher_lib):
    op = emit_flash_ws(_body(pair=True), "k_ws")
    src = op.kernel_source
    assert "EMH_SUB_BASES(v, t + RING - 2, vbase, V_SS, V_RING) EMH_SUB_BASES(k, t + RING, kbase, K_SS, 0)" in src  # what iteration t requests
    assert "EMH_SUB_BASES(v, tau + RING - 2, vbase, V_SS, V_RING) EMH_SUB_BASES(k, tau + RING, kbase, K_SS, 0)" in src and "for (int tau = -RING; tau < 0; ++tau)" in src
    assert "const bool ok_##tag = sub_##tag >= 0 && sub_##tag < nsub;" in src and "((sub_##tag + RING) % RING) * SLOT" in src  # existence, slot
    assert "const int tau_ = (t_) - d_;" in src and "d_ < RING - 2" in src  # what a landing wait leaves outstanding
    assert src.count("EMH_BARRIER();") >= 8 and "#define RING 4" in src
    assert op.block[0] == (512,) and op.knobs["FLASH"] == "w2/kv32/s2/p/ws" and op.lds_bytes == 2 * 4 * 16384 + 16384
    from deplodock_amd.backend.hip import hiprtc

    assert hiprtc.spilled_vgprs(src, "k_ws") == 0


def test_what_the_form_takes_and_what_it_refuses():
    assert ws_supported(_body()) is None and ws_supported(_body(waves=4, kvs=1)) is None and ws_supported(_body(d=64, waves=1, kvs=4)) is None
    assert "must be 4" in ws_supported(_body(waves=2, kvs=4))
    assert "head_dim" in ws_supported(_body(d=256))
    assert "LDS" in ws_supported(_body(waves=1, kvs=4))  # 32 KiB sub-steps: a ring of three per operand does not fit
    assert ws_lds_plan(2, 2, 128, 160 * 1024)["ring"] == 4 and ws_lds_plan(4, 1, 128, 160 * 1024)["ring"] == 4
    # the self-staging form: eight consumer waves; 32 KiB sub-steps leave room for rings of two
    sp = _body(waves=2, kvs=4)
    sp.ws, sp.sp = False, True
    assert ws_supported(sp) is None and ws_lds_plan(2, 4, 128, 160 * 1024, (4, 3, 2))["ring"] == 2
    bad = _body(waves=2, kvs=2)
    bad.ws, bad.sp = False, True
    assert "must be 8" in ws_supported(bad)


def test_self_staging_form_builds_without_spills_and_carries_its_requests_in_the_slices(launcher_lib):
    from deplodock_amd.backend.hip import hiprtc

    body = _body(waves=2, kvs=4, pair=True)
    body.ws, body.sp = False, True
    op = emit_flash_ws(body, "k_sp")
    src = op.kernel_source
    assert op.knobs["FLASH"] == "w2/kv32/s4/p/sp" and op.block[0] == (512,) and "#define SP 1" in src and "#define RING 2" in src
    assert src.count("EMH_REQ_I(v, 0, vvo0") >= 4 and "EMH_LAND(t + 1)" in src and "EMH_PROLOGUE_REQUESTS()" in src
    assert hiprtc.spilled_vgprs(src, "k_sp") == 0


def test_pin_grammar_reaches_the_emitter(launcher_lib, monkeypatch):
    monkeypatch.setenv("EMMY_FLASH", "w2/kv64/s2/p/ws")  # the key block is the form's own: 32 keys per wave
    case = eager.sdpa_case()
    compiled = HipBackend().compile(trace_module(case.module, case.inputs))
    (op,) = [n.op for n in compiled.nodes.values() if isinstance(n.op, HipOp)]
    assert op.knobs["FLASH"] == "w2/kv32/s2/p/ws" and "wave-specialised" in op.kernel_source
    monkeypatch.setenv("EMMY_FLASH", "w2/kv32/s4/ws")  # not a shape of the form: the pin is dropped, the default lowers
    compiled = HipBackend().compile(trace_module(case.module, case.inputs))
    (op,) = [n.op for n in compiled.nodes.values() if isinstance(n.op, HipOp)]
    assert "/ws" not in op.knobs["FLASH"]


# -- GPU parity -----------------------------------------------------------------------------------------------

CASES = [
    ("small causal", dict(b=1, hq=8, hkv=4, s=320, d=128, seed=9), ["w2/kv32/s2/ws", "w4/kv32/s1/ws"]),
    ("pairs", dict(b=2, hq=4, hkv=2, s=512, d=128, seed=11), ["w2/kv32/s2/p/ws", "w4/kv32/s1/p/ws"]),
    ("ragged causal", dict(b=1, hq=4, hkv=2, s=300, d=128, seed=3), ["w2/kv32/s2/ws", "w4/kv32/s1/ws"]),
    ("shorter than a sub-step", dict(b=1, hq=2, hkv=1, s=40, d=128, seed=4), ["w2/kv32/s2/ws", "w4/kv32/s1/ws"]),
    ("one key", dict(b=1, hq=2, hkv=2, s=1, d=128, seed=5), ["w2/kv32/s2/ws"]),
    ("unmasked ragged", dict(b=1, hq=4, hkv=2, s=333, d=128, seed=5, causal=False), ["w2/kv32/s2/ws", "w4/kv32/s1/ws"]),
    ("head_dim 64", dict(b=1, hq=8, hkv=2, s=512, d=64, seed=15), ["w2/kv32/s2/ws", "w4/kv32/s1/ws", "w1/kv32/s4/ws"]),
    ("small causal", dict(b=1, hq=8, hkv=4, s=320, d=128, seed=9), ["w2/kv32/s4/sp", "w4/kv32/s2/sp", "w8/kv32/s1/sp"]),
    ("pairs", dict(b=2, hq=4, hkv=2, s=512, d=128, seed=11), ["w2/kv32/s4/p/sp", "w4/kv32/s2/p/sp"]),
    ("ragged causal", dict(b=1, hq=4, hkv=2, s=300, d=128, seed=3), ["w2/kv32/s4/sp", "w4/kv32/s2/sp"]),
    ("shorter than a sub-step", dict(b=1, hq=2, hkv=1, s=40, d=128, seed=4), ["w2/kv32/s4/sp", "w8/kv32/s1/sp"]),
    ("unmasked ragged", dict(b=1, hq=4, hkv=2, s=333, d=128, seed=5, causal=False), ["w2/kv32/s4/sp", "w4/kv32/s2/sp"]),
    ("head_dim 64", dict(b=1, hq=8, hkv=2, s=512, d=64, seed=15), ["w4/kv32/s2/sp", "w2/kv32/s4/sp"]),
]


@pytest.mark.gpu
@pytest.mark.parametrize("label,kw,pin", [(label, kw, pin) for label, kw, pins in CASES for pin in pins], ids=lambda v: v if isinstance(v, str) else None)
def test_ws_matches_eager_on_every_shape_of_the_form(device, label, kw, pin, monkeypatch):
    monkeypatch.setenv("EMMY_FLASH", pin)
    case = eager.sdpa_case(**kw)
    be = HipBackend()
    compiled = be.compile(trace_module(case.module, case.inputs))
    assert [n.op.knobs["FLASH"] for n in compiled.nodes.values() if isinstance(n.op, HipOp)] == [pin]
    want = eager.run_eager(case, device)
    prog = be.program(compiled, {n: t.to(device) for n, t in zip(compiled.inputs, case.inputs)})
    try:
        out = prog.output_tensors()[compiled.outputs[0]]
        for rep in range(5):  # the first sub-steps are consumed right after they are staged: every launch is checked
            out.zero_()
            prog.run()
            torch.cuda.synchronize()
            eager.assert_close(out.reshape(want.shape), want, case.rtol, case.atol, f"sdpa {label} {pin} launch {rep}")
    finally:
        prog.close()


@pytest.mark.gpu
@pytest.mark.parametrize("pin", ["w2/kv32/s2/p/ws", "w4/kv32/s1/ws", "w2/kv32/s4/p/sp"])
def test_ws_full_size_rows_and_position_coded_values(device, pin, monkeypatch):
    """The benchmark shape with the scale-aware criteria of the default kernel's test: per-row relative error against
    an fp32 run bounded by 1.5 x 16-bit eager's, rows summing to one, and position-coded values (a skipped or
    misplaced key block shifts a row by far more than rounding)."""
    monkeypatch.setenv("EMMY_FLASH", pin)
    case = eager.sdpa_case()

    def run(c):
        be = HipBackend()
        compiled = be.compile(trace_module(c.module, c.inputs))
        assert [n.op.knobs["FLASH"] for n in compiled.nodes.values() if isinstance(n.op, HipOp)] == [pin]
        prog = be.program(compiled, {n: t.to(device) for n, t in zip(compiled.inputs, c.inputs)})
        try:
            prog.run()
            torch.cuda.synchronize()
            ours = prog.output_tensors()[compiled.outputs[0]].clone()
        finally:
            prog.close()
        want = eager.run_eager(c, device)
        return ours.reshape(want.shape), want

    ours, want = run(case)
    eager.assert_close(ours, want, case.rtol, case.atol, f"sdpa {pin} vs eager")
    q, k, v = (t.to(device).float() for t in case.inputs)
    exact = nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True, enable_gqa=True)
    eager.assert_rows_within_baseline(ours, want, exact, 1.5, f"sdpa {pin} rows vs fp32 eager")
    ones = eager.Case("ones", case.module, (case.inputs[0], case.inputs[1], torch.ones_like(case.inputs[2])), 2e-2, 2e-2)
    o1, _ = run(ones)
    assert float((o1.float() - 1).abs().max()) <= 2**-7
    vpos = eager.position_coded_values(case.inputs[2])
    coded = eager.Case("pos", case.module, (case.inputs[0], case.inputs[1], vpos), 2e-2, 2e-2)
    op_, wp = run(coded)
    exact_p = nn.functional.scaled_dot_product_attention(q, k, vpos.to(device).float(), is_causal=True, enable_gqa=True)
    eager.assert_rows_within_baseline(op_, wp, exact_p, 1.5, f"sdpa {pin} position-coded V vs fp32 eager")


@pytest.mark.gpu
@pytest.mark.parametrize("pin", ["w2/kv32/s2/ws", "w2/kv32/s4/sp"])
def test_ws_large_score_jumps_raise_the_reference_maximum(device, pin, monkeypatch):
    """Keys whose scores grow along the sequence (every sub-block outgrows the reference maximum of the one before by
    more than the slack) exercise the vote, the deferred rescale of the output accumulators and the merge of the
    key-split groups' statistics."""
    monkeypatch.setenv("EMMY_FLASH", pin)
    torch.manual_seed(31)
    s, d = 384, 128
    q = torch.randn(1, 4, s, d)
    k = torch.randn(1, 2, s, d) * torch.linspace(0.2, 6.0, s).reshape(1, 1, s, 1)
    v = torch.randn(1, 2, s, d)
    case = eager.Case("jumps", eager.Sdpa(True), (q.bfloat16(), k.bfloat16(), v.bfloat16()), 2e-2, 2e-2)
    be = HipBackend()
    compiled = be.compile(trace_module(case.module, case.inputs))
    prog = be.program(compiled, {n: t.to(device) for n, t in zip(compiled.inputs, case.inputs)})
    try:
        prog.run()
        torch.cuda.synchronize()
        ours = prog.output_tensors()[compiled.outputs[0]].clone()
    finally:
        prog.close()
    want = eager.run_eager(case, device)
    qf, kf, vf = (t.to(device).float() for t in case.inputs)
    exact = nn.functional.scaled_dot_product_attention(qf, kf, vf, is_causal=True, enable_gqa=True)
    eager.assert_close(ours.reshape(want.shape), exact, 2e-2, 2e-2, "sdpa with growing scores vs fp32 eager")
    eager.assert_rows_within_baseline(ours.reshape(want.shape), want, exact, 1.5, "sdpa with growing scores, rows")


@pytest.mark.gpu
@pytest.mark.parametrize("pin", ["w2/kv32/s2/p/ws", "w2/kv32/s4/p/sp"])
def test_ws_soak_is_bit_stable(device, pin, monkeypatch):
    """2000 launches on fixed inputs reproduce the first bit for bit (the publication fence of the stagers' requests,
    the barrier protocol of the rings), and that result matches eager."""
    monkeypatch.setenv("EMMY_FLASH", pin)
    case = eager.sdpa_case(b=1, hq=16, hkv=8, s=1024, d=128, seed=22)
    be = HipBackend()
    compiled = be.compile(trace_module(case.module, case.inputs))
    prog = be.program(compiled, {n: t.to(device) for n, t in zip(compiled.inputs, case.inputs)})
    try:
        out = prog.output_tensors()[compiled.outputs[0]]
        prog.run()
        torch.cuda.synchronize()
        first = out.clone()
        for i in range(1, 2000):
            out.zero_()
            prog.run()
            torch.cuda.synchronize()
            if not torch.equal(out, first):
                pytest.fail(f"launch {i} differs from the first in {int((out.view(torch.int16) != first.view(torch.int16)).sum())} elements")
    finally:
        prog.close()
    want = eager.run_eager(case, device)
    eager.assert_close(first.reshape(want.shape), want, case.rtol, case.atol, "ws after the soak vs eager")


@pytest.mark.parametrize("flags", ["-DEMH_STAMP=1", "-DEMH_STAMP=2", "-DEMH_ABLATE=1", "-DEMH_ABLATE=2", "-DEMH_ABLATE=3", "-DEMH_ABLATE=4"])
def test_measurement_switches_build(launcher_lib, flags, monkeypatch):
    """The phase stamps (shader clock, summed by wave 0 of workgroup 0) and the ablations ``microbench --flash`` reads are
    compile-time switches of the emitted text: each must build, without spills, for both forms."""
    from deplodock_amd.backend.hip import hiprtc

    monkeypatch.setenv("EMMY_HIPRTC_FLAGS", flags)
    for sp in (False, True):
        body = _body(waves=2, kvs=4 if sp else 2, pair=True)
        body.ws, body.sp = not sp, sp
        op = emit_flash_ws(body, "k_sw")
        assert "__builtin_readcyclecounter" in op.kernel_source and "EMH_ABLATE" in op.kernel_source
        assert hiprtc.spilled_vgprs(op.kernel_source, "k_sw") == 0
