"""Runtime behaviour on the device: graph replays, event timing, the watchdog,
zeroed accumulation targets — all through the C-ABI library."""

from __future__ import annotations

import asyncio

import numpy as np
import pytest
import torch
from torch import nn

from deplodock_amd import HipBackend, trace_module
from deplodock_amd.backend.hip import launcher, program
from deplodock_amd.dtype import F32
from deplodock_amd.graph import Graph, Tensor
from deplodock_amd.ir.hip import HipOp
from oracle import eager

pytestmark = pytest.mark.gpu


def test_device_is_gfx950(launcher_lib, device):
    props = launcher_lib.device_props(0)
    assert props["arch"].startswith("gfx950") and props["wavefront_size"] == 64 and props["compute_units"] == 256


def test_graph_replays_match_eager_every_time(device):
    """A captured whole-program graph is replayed several times with eager work and
    synchronisations in between; every replay must reproduce the eager result."""
    case = eager.qwen3_block_case(seq=64)
    be = HipBackend()
    compiled = be.compile(trace_module(case.module, case.inputs))
    want = eager.run_eager(case, device)
    prog = be.program(compiled, {n: t.to(device) for n, t in zip(compiled.inputs, case.inputs)})
    try:
        out = prog.output_tensors()[compiled.outputs[0]]
        prog.capture_program_graph()
        for i in range(4):
            out.zero_()
            torch.cuda.synchronize()
            prog.replay_program()
            prog.lib.stream_synchronize(prog._ensure_stream())
            eager.assert_close(out.reshape(want.shape), want, case.rtol, case.atol, f"replay {i}")
            _ = (torch.randn(256, 256, device=device) @ torch.randn(256, 256, device=device)).sum().item()  # eager work between replays
    finally:
        prog.close()


def test_zero_outputs_are_cleared_before_each_launch_also_in_graphs(device):
    src = 'extern "C" __global__ void k_acc(const float* x, float* y) { atomicAdd(&y[threadIdx.x % 4], x[threadIdx.x]); }'
    g = Graph()
    g.add_input("x", (64,), F32)
    op = HipOp(kernel_source=src, kernel_name="k_acc", arg_order=("x", "y"), grid=((1,), (1,), (1,)), block=((64,), (1,), (1,)), zero_outputs=("y",))
    g.add_node(op, ["x"], Tensor("y", (4,), F32), "y")
    g.outputs = ["y"]
    x = torch.arange(64, dtype=torch.float32)
    want = x.reshape(16, 4).sum(0)
    prog = program.CompiledProgram.build(g, {"x": x})
    try:
        for _ in range(3):
            prog.run()
        torch.cuda.synchronize()
        torch.testing.assert_close(prog.output_tensors()["y"].cpu(), want)
        prog.capture_program_graph()
        for _ in range(3):
            prog.replay_program()
            prog.lib.stream_synchronize(prog._ensure_stream())
            torch.testing.assert_close(prog.output_tensors()["y"].cpu(), want)
    finally:
        prog.close()


def test_benchmark_reports_event_times_and_e2e(device):
    case = eager.qwen3_block_case(seq=64)
    be = HipBackend()
    compiled = be.compile(trace_module(case.module, case.inputs))
    calls = []
    res = asyncio.run(be.benchmark_async(compiled, warmup=2, num_iters=5, on_iter=lambda b: calls.append(b)))
    assert res.num_launches == 5 and len(res.per_launch) == 5 and res.captured
    assert all(p.time_ms > 0 and len(p.samples) == 5 for p in res.per_launch)
    assert res.e2e_ms is not None and res.e2e_min_ms <= res.e2e_ms
    assert 0 < res.min_ms <= res.time_ms <= res.max_ms
    assert len(calls) >= 7 and all(b >= 1 for b in calls)
    single = be.benchmark(be.compile(trace_module(*(lambda c: (c.module, c.inputs))(eager.rms_norm_case()))), warmup=1, num_iters=3)
    assert single.e2e_ms is None and single.num_launches == 1  # the solo window is the program time


def test_watchdog_raises_instead_of_stalling(device, monkeypatch):
    """Forced from the host: with a negative budget the poll gives up while the
    (perfectly healthy, ~150 us) kernel is still running; the kernel still finishes."""
    case = eager.softmax_case()
    be = HipBackend()
    compiled = be.compile(trace_module(case.module, case.inputs))
    prog = be.program(compiled, {compiled.inputs[0]: case.inputs[0].to(device)})
    monkeypatch.setattr(program, "_KERNEL_TIMEOUT_MS", -1.0)
    try:
        with pytest.raises(program.HungKernelError):
            prog.iter_once([64])
    finally:
        monkeypatch.undo()
        assert prog._hung
        prog.close()  # after the watchdog has fired close() must not wait on the stream (a real hang would never return)
        assert prog._stream is None
    torch.cuda.synchronize()  # the kernels here are healthy: every wave exits normally


def test_isolated_benchmark_worker_is_killed_at_the_wall_limit_and_replaced(device):
    """``bench_wall_timeout_s``: the benchmark runs in a worker process forked from a clean server; a limit
    shorter than a healthy (but very long) run gets the worker killed and reported as a failed benchmark,
    the next benchmark gets a fresh worker, and this process's own device state is untouched."""
    case = eager.softmax_case(shape=(4096, 2048))
    be = HipBackend(bench_wall_timeout_s=170.0)
    compiled = be.compile(trace_module(case.module, case.inputs))
    data = {compiled.inputs[0]: case.inputs[0].to(device)}
    try:
        res = be.benchmark(compiled, warmup=2, num_iters=5, input_data=data)
        assert res.num_launches == 1 and res.time_ms > 0 and res.captured
        assert be._worker.spawned == 1 and be._worker.killed == 0
        again = asyncio.run(be.benchmark_async(compiled, warmup=2, num_iters=5))  # same (kept) worker through the async entry point
        assert again.time_ms > 0 and be._worker.spawned == 1
        be.bench_wall_timeout_s = 0.5
        be.bench_run_timeout_s = 3600.0
        with pytest.raises(RuntimeError, match="wall budget"):
            be.benchmark(compiled, warmup=2, num_iters=50_000_000)  # healthy kernels, far more windows than fit the limit
        assert be._worker.killed == 1
        be.bench_wall_timeout_s, be.bench_run_timeout_s = 170.0, 10.0
        fresh = be.benchmark(compiled, warmup=2, num_iters=5)
        assert fresh.time_ms > 0 and be._worker.spawned == 2
        # an in-worker failure (run budget) comes back as the same RuntimeError the in-process path raises
        be.bench_run_timeout_s = 1e-9
        with pytest.raises(RuntimeError, match="bench_fail"):
            be.benchmark(compiled, warmup=1, num_iters=3)
    finally:
        be.close()
    ours, want = (lambda p: (p.run(), torch.cuda.synchronize(), p.output_tensors()[compiled.outputs[0]].clone(), p.close())[2])(HipBackend().program(compiled, data)), eager.run_eager(case, device)
    eager.assert_close(ours.reshape(want.shape), want, case.rtol, case.atol, "in-process run after worker kills")


def test_debug_run_keeps_a_host_copy_of_every_written_buffer_per_launch(device):
    """``HipBackend(debug=True)``: ``run`` goes launch by launch and ``last_debug_result`` holds, per launch index,
    what every scratch / output buffer held right after it (emmy/compiler/backend/cuda/program.py:1128,
    backend.py:158-161).  On the decoder block: five launches, each launch's own output differs from what it was
    before the launch, the last launch's snapshot of the output is the run's output, and the outputs equal a plain
    run's; a plain run afterwards clears ``last_debug_result``."""
    case = eager.qwen3_block_case(seq=64)
    be = HipBackend(debug=True)
    compiled = be.compile(trace_module(case.module, case.inputs))
    # inputs no other test uses: memory recycled from an earlier run of the same block cannot already hold these results
    data = {n: (t * 0.37 if i == 0 else t).to(device) for i, (n, t) in enumerate(zip(compiled.inputs, case.inputs))}
    res, _ = be.run(compiled, input_data=data)
    dbg = be.last_debug_result
    assert dbg is not None and res.time_ms is None
    launches = [nid for nid in compiled.topological_order() if compiled.node_role(nid) in ("scratch", "output")]
    assert sorted(dbg.per_launch) == list(range(len(launches))) == sorted(dbg.kernel_names) and len(launches) == 5
    out = compiled.outputs[0]
    for i, nid in enumerate(launches):
        assert nid in dbg.per_launch[i] and out in dbg.per_launch[i]
        if i:
            assert not np.array_equal(dbg.per_launch[i][nid], dbg.per_launch[i - 1][nid]), f"launch {i} did not write {nid}"
    assert np.array_equal(dbg.per_launch[len(launches) - 1][out], dbg.outputs[out]) and np.array_equal(res.outputs[out], dbg.outputs[out])
    plain_be = HipBackend(debug=False)
    plain, _ = plain_be.run(compiled, input_data=data)
    assert plain_be.last_debug_result is None and plain.time_ms is not None
    assert np.array_equal(plain.outputs[out], res.outputs[out])
    be.debug = False
    be.run(compiled, input_data=data)
    assert be.last_debug_result is None


def test_benchmark_async_leaves_the_event_loop_running_while_a_worker_benchmarks(device):
    """With the isolated worker, ``benchmark_async`` waits for the worker's answer off the loop's thread: a task
    scheduled beside it keeps ticking while the benchmark runs."""
    case = eager.softmax_case(shape=(4096, 2048))
    be = HipBackend(bench_wall_timeout_s=170.0)
    compiled = be.compile(trace_module(case.module, case.inputs))

    async def both():
        ticks = 0
        done = asyncio.Event()

        async def ticker():
            nonlocal ticks
            while not done.is_set():
                ticks += 1
                await asyncio.sleep(0.005)

        t = asyncio.ensure_future(ticker())
        res = await be.benchmark_async(compiled, warmup=2, num_iters=20)
        done.set()
        await t
        return res, ticks

    try:
        res, ticks = asyncio.run(both())
    finally:
        be.close()
    assert res.time_ms > 0 and res.captured
    assert ticks >= 5, f"the event loop ran {ticks} tick(s) during the benchmark"


def test_run_budget_marks_bench_fail(device):
    case = eager.softmax_case(shape=(64, 2048))
    be = HipBackend(bench_run_timeout_s=1e-9)
    compiled = be.compile(trace_module(case.module, case.inputs))
    with pytest.raises(RuntimeError, match="bench_fail"):
        be.benchmark(compiled, warmup=1, num_iters=3)


def test_misaligned_device_tensor_is_rejected(device):
    case = eager.rms_norm_case(rows=4, cols=64)
    be = HipBackend()
    compiled = be.compile(trace_module(case.module, case.inputs))
    base = torch.randn(4 * 64 + 1, device=device)
    with pytest.raises(ValueError, match="16-byte aligned"):
        be.program(compiled, {compiled.inputs[0]: base[1:].reshape(1, 4, 64)})


def test_launch_errors_surface_as_exceptions(launcher_lib, device):
    from deplodock_amd.backend.hip import hiprtc
    from deplodock_amd.backend.hip.launcher import PackedArgs

    k = hiprtc.load_function('extern "C" __global__ void k_one(float* x) { x[threadIdx.x] = 1.0f; }', "k_one")
    buf = torch.zeros(64, device=device)
    with pytest.raises(launcher.LauncherError, match="1024"):
        launcher_lib.launch(k.fn, (1, 1, 1), (2048, 1, 1), 0, None, PackedArgs([buf.data_ptr()]))
    launcher_lib.launch(k.fn, (1, 1, 1), (64, 1, 1), 0, None, PackedArgs([buf.data_ptr()]))
    torch.cuda.synchronize()
    assert float(buf.sum()) == 64.0
    np.testing.assert_equal(launcher_lib.func_attributes(k.fn)["private_bytes"], 0)


@pytest.mark.parametrize("which", ["rms", "softmax", "linear"])
def test_empty_inputs_run_and_return_empty_outputs(device, which):
    """Zero rows: nothing is launched (the driver rejects empty grids) and the outputs are empty, as in eager."""
    if which == "rms":
        mod, x = nn.RMSNorm(64).eval(), torch.randn(0, 64)
    elif which == "softmax":
        mod, x = nn.Softmax(-1).eval(), torch.randn(3, 0, 16)
    else:
        mod, x = nn.Linear(32, 16, bias=False).bfloat16().eval(), torch.randn(0, 32).bfloat16()
    be = HipBackend()
    compiled = be.compile(trace_module(mod, (x,)))
    res, _ = be.run(compiled, input_data={compiled.inputs[0]: x.to(device)})
    out = res.outputs[compiled.outputs[0]]
    assert out.size == 0 and tuple(out.shape) == tuple(mod(x).shape)


@pytest.mark.gpu
@pytest.mark.parametrize("what", ["attention", "linear_dlm", "linear_pp"])
def test_a_stamped_build_computes_the_same_result_and_leaves_its_clocks_in_the_first_words(device, what, monkeypatch):
    """The measurement build (``-DEMH_STAMP=1``) is the product kernel plus clock reads: apart from the 16 bytes the
    stamps are left in, its output is bit for bit the plain build's, and the four stamps are positive clock counts."""
    from deplodock_amd import workloads as wl

    case = {"attention": lambda: wl.sdpa_case(s=512), "linear_dlm": lambda: wl.linear_case(m=1024, k=1024, n=4096), "linear_pp": lambda: wl.linear_case(m=2048)}[what]()
    if what == "linear_dlm":
        monkeypatch.setenv("EMMY_TILE", "a:mfma_16x16x32_bf16/w2x4/f8x4/k2")
    outs = []
    for flags in (None, "-DEMH_STAMP=1"):
        if flags:
            monkeypatch.setenv("EMMY_HIPRTC_FLAGS", flags)
        be = HipBackend()
        compiled = be.compile(trace_module(case.module, case.inputs))
        (op,) = [n.op for n in compiled.nodes.values() if isinstance(n.op, HipOp)]
        if what != "attention":
            assert op.knobs["STAGE"].endswith("/dlm" if what == "linear_dlm" else "/pp"), op.knobs
        prog = be.program(compiled, {n: t.to(device) for n, t in zip(compiled.inputs, case.inputs)})
        try:
            prog.run()
            torch.cuda.synchronize()
            outs.append((prog.output_tensors()[compiled.outputs[0]].reshape(-1).clone(), op))
        finally:
            prog.close()
    (plain, _), (stamped, op) = outs
    # workgroup 0 leaves the stamps over the first 16 bytes it stored: the start of the output for the contractions, of
    # its query block's first row for attention (the last block of head 0: 512 tokens run unpaired)
    at = 0 if what != "attention" else (512 - 32 * int(op.knobs["FLASH"].split("/")[0][1:])) * 128
    stamps = stamped[at : at + 8].view(torch.float32)
    assert bool((stamps[:3] > 0).all()) and bool((stamps < 1e7).all()), stamps
    keep = torch.ones_like(plain, dtype=torch.bool)
    keep[at : at + 8] = False
    assert torch.equal(plain[keep], stamped[keep])
