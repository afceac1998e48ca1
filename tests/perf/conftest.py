"""The perf suite's plumbing, after the reference's (tests/perf/conftest.py:78-99, 124-160): tests carry the ``perf``
marker and are skipped unless ``-m perf`` selects them; ``bench_pair`` times one case on both sides and the session
ends with a table sorted by ``ratio = eager_us / ours_us`` (losses first) and a JSON dump under
``tests/perf/.results/`` (``EMMY_PERF_RESULTS`` names another folder).

Unlike the reference's fixture, which spawns its CLI once per case, every case runs in this process: the trace,
compile, accuracy check against eager, and both timings use the functions the ``run --bench`` command is made of.
"""

from __future__ import annotations

import json
import os
from dataclasses import asdict, dataclass
from datetime import datetime, timezone
from pathlib import Path

import pytest

RESULTS = Path(__file__).resolve().parent / ".results"


@dataclass
class PerfRow:
    name: str
    op: str
    shape: str
    dtype: str
    torch_us: float
    emmy_us: float
    ratio: float  # torch_us / emmy_us: above 1 this backend is faster
    launches: int
    iters: int
    kernels: list  # [(kernel name, us)] per launch


def _rows(config) -> list[PerfRow]:
    if not hasattr(config, "_perf_rows"):
        config._perf_rows = []
    return config._perf_rows


def pytest_configure(config):
    config.addinivalue_line("markers", "perf: kernel-level timing against PyTorch eager on an MI355X (select with -m perf)")


def pytest_collection_modifyitems(config, items):
    if "perf" in (config.getoption("-m") or ""):
        return
    skip = pytest.mark.skip(reason="perf marker not selected; run with `pytest tests/perf -m perf` on a GPU box")
    for item in items:
        if "perf" in item.keywords:
            item.add_marker(skip)


@pytest.fixture
def bench_pair(request):
    def run(case, *, warmup: int = 10, iters: int | None = None) -> PerfRow:
        import torch

        from deplodock_amd import HipBackend, trace_module
        from deplodock_amd.commands.code import parse_inline
        from deplodock_amd.commands.run import _eager_us, _flatten_tensors, _to_device, check_accuracy
        from deplodock_amd.ir.hip import HipOp

        if not torch.cuda.is_available():
            pytest.fail("the perf suite needs a HIP device")
        device = torch.device("cuda:0")
        iters = iters or case.iters
        torch.manual_seed(0)
        prog = parse_inline(case.code)
        graph = trace_module(prog.module, prog.args, kwargs=prog.kwargs or None)
        be = HipBackend(device_id=0)
        compiled = be.compile(graph)
        module = prog.module.to(device).eval()
        d_args, d_kwargs = _to_device(prog.args, device), _to_device(prog.kwargs, device)
        data = dict(zip(compiled.inputs, _flatten_tensors(d_args) + _flatten_tensors(d_kwargs)))
        with torch.no_grad():
            want = _flatten_tensors(module(*d_args, **d_kwargs))
        program = be.program(compiled, data)
        try:
            program.run()
            torch.cuda.synchronize()
            for name, w in zip(compiled.outputs, want):
                ok, line = check_accuracy(program.output_tensors()[name], w)
                assert ok, f"{case.name}: {line}"
        finally:
            program.close()
        _, eager_min = _eager_us(module, d_args, d_kwargs, warmup, iters)
        res = be.benchmark(compiled, input_data=data, warmup=warmup, num_iters=iters)
        ours = (res.e2e_min_ms if res.e2e_ms is not None else (res.min_ms or res.time_ms)) * 1e3
        ops = [compiled.nodes[n].op for n in compiled.topological_order() if isinstance(compiled.nodes[n].op, HipOp)]
        times = {lt.idx: (min(lt.samples) if lt.samples else lt.time_ms) * 1e3 for lt in (res.per_launch or [])}
        per_kernel = [(op.kernel_name, round(times[i], 2)) for i, op in enumerate(ops) if i in times]
        row = PerfRow(case.name, case.op, case.shape_str, case.dtype, round(eager_min, 2), round(ours, 2), round(eager_min / ours, 3), len(ops), iters, per_kernel)
        _rows(request.config).append(row)
        return row

    return run


def pytest_terminal_summary(terminalreporter, config):
    rows = sorted(_rows(config), key=lambda r: r.ratio)
    if not rows:
        return
    from deplodock_amd.commands.table import render_table

    tr = terminalreporter
    tr.write_sep("=", "perf: PyTorch eager / this backend (min of timed iterations, us)")
    table = [[r.name, r.shape, f"{r.torch_us:.1f}", f"{r.emmy_us:.1f}", f"{r.ratio:.2f}x", str(r.launches)] for r in rows]
    for line in render_table(["case", "shape", "torch_us", "emmy_us", "ratio", "launches"], table, "llrrrr"):
        tr.write_line(line)
    geo = 1.0
    for r in rows:
        geo *= r.ratio
    tr.write_line(f"geometric mean of the ratio over {len(rows)} cases: {geo ** (1.0 / len(rows)):.2f}x; losses (ratio < 1): {sum(r.ratio < 1 for r in rows)}")
    out_dir = Path(os.environ.get("EMMY_PERF_RESULTS") or RESULTS)
    out_dir.mkdir(parents=True, exist_ok=True)
    path = out_dir / (datetime.now(timezone.utc).strftime("%Y%m%dT%H%M%SZ") + ".json")
    path.write_text(json.dumps({"git_rev": os.environ.get("EMMY_GIT_REV"), "rows": [asdict(r) for r in rows]}, indent=1))
    tr.write_line(f"written to {path}")
