"""Runtime contract checks that need no device: graph validation happens before
anything is loaded (mirrors the hand-written-CudaOp tests of the reference,
tests/compiler/backend/test_program.py:74-101)."""

from __future__ import annotations

import pytest

from deplodock_amd.backend.hip import program
from deplodock_amd.dtype import F32
from deplodock_amd.graph import Graph, Tensor
from deplodock_amd.ir.base import Op
from deplodock_amd.ir.hip import HipOp

SRC = 'extern "C" __global__ void k(const float* x, float* y) { y[threadIdx.x] = x[threadIdx.x]; }'


def graph_with(ops):
    g = Graph()
    g.add_input("x", (64,), F32)
    prev = "x"
    for i, op in enumerate(ops):
        nid = f"y{i}"
        if isinstance(op, HipOp) and not op.arg_order:
            op.arg_order = (prev, nid)
        g.add_node(op, [prev], Tensor(nid, (64,), F32), nid)
        prev = nid
    g.outputs = [prev]
    return g


def test_non_hip_node_is_a_type_error():
    with pytest.raises(TypeError, match="non-HipOp"):
        program._compile(graph_with([Op()]))


def test_duplicate_kernel_name_with_other_source_is_rejected():
    a = HipOp(kernel_source=SRC, kernel_name="k", block=((64,), (1,), (1,)))
    b = HipOp(kernel_source=SRC.replace("x[threadIdx.x]", "2.0f * x[threadIdx.x]"), kernel_name="k", block=((64,), (1,), (1,)))
    with pytest.raises(ValueError, match="two distinct sources"):
        program._compile(graph_with([a, b]))


def test_unknown_buffer_is_rejected():
    a = HipOp(kernel_source=SRC, kernel_name="k", arg_order=("x", "nope"))
    with pytest.raises(KeyError, match="unknown buffer"):
        program._compile(graph_with([a]))


def test_batch_calibration_and_iter_budget():
    assert [program.window_issues(dt) for dt in (0.002, 0.5, 3.0, 0.0)] == [500, 2, 1, 1]
    assert [program.window_issues(dt, 0.25) for dt in (0.002, 0.5)] == [125, 1]  # (a program of 400 launches: windows of a quarter millisecond)
    fixed = program.SampleBudget.parse(20)
    assert not fixed.spent(19, 1e9) and fixed.spent(20, 0.0)
    auto = program.SampleBudget.parse("auto")
    assert auto.spent(1, program._AUTO_BUDGET_MS) and not auto.spent(1, 0.5 * program._AUTO_BUDGET_MS) and auto.spent(program._AUTO_MAX_ITERS, 0.0)
    with pytest.raises(ValueError):
        program.SampleBudget.parse("many")


def test_no_device_means_a_loud_error_not_a_fallback():
    import torch

    if torch.cuda.is_available():
        pytest.skip("a device is present")
    from deplodock_amd.backend.hip.launcher import LauncherError

    with pytest.raises(LauncherError, match="no CPU fallback"):
        program._device()


def test_bench_worker_kills_at_the_wall_limit_reports_child_errors_and_respawns():
    """Host-side behaviour of the isolated benchmark worker (no GPU involved): a request that is not
    answered in time gets the child killed and a ``RuntimeError``; an exception inside the child comes
    back as ``RuntimeError`` with its text and the child is replaced before the next job."""
    from deplodock_amd.backend.hip.bench_worker import BenchWorker

    w = BenchWorker()
    try:
        with pytest.raises(RuntimeError, match="wall budget"):
            w.run_job({"graph": None, "input_data": {}, "kwargs": {}}, wall_timeout_s=0.0)
        assert (w.spawned, w.killed) == (1, 1) and w._proc is None
        with pytest.raises(RuntimeError, match="bench worker error: .*topological_order"):
            w.run_job({"graph": "not a graph", "input_data": {}, "kwargs": {}}, wall_timeout_s=120.0)
        assert w.spawned == 2
        with pytest.raises(RuntimeError, match="bench worker error"):
            w.run_job({"graph": "still not a graph", "input_data": {}, "kwargs": {}}, wall_timeout_s=120.0)
        assert w.spawned == 3
    finally:
        w.close()


def test_backend_routes_benchmarks_to_the_worker_only_with_a_wall_limit_and_no_callback(monkeypatch):
    from deplodock_amd import HipBackend
    from deplodock_amd.backend.hip import bench_worker, program

    calls = []
    monkeypatch.setattr(bench_worker, "benchmark_program_isolated", lambda g, **kw: calls.append(("worker", kw["wall_timeout_s"])) or "W")
    monkeypatch.setattr(program, "benchmark_program", lambda g, **kw: calls.append(("inline", None)) or "I")
    g = Graph()
    assert HipBackend().benchmark(g) == "I"
    be = HipBackend(bench_wall_timeout_s=7.0)
    assert be.benchmark(g) == "W"
    assert be.benchmark(g, on_iter=lambda n: None) == "I"  # a callback shares state with this process: in-process
    assert calls == [("inline", None), ("worker", 7.0), ("inline", None)]
