"""Host-side checks of ``bench.py``: the flags it refuses and the arithmetic it does on rocprofv3's counter files.
Nothing here launches a kernel."""

import csv
import importlib.util
import subprocess
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent


@pytest.fixture(scope="module")
def bench():
    spec = importlib.util.spec_from_file_location("bench_under_test", ROOT / "bench.py")
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_more_than_one_gpu_is_refused_with_a_message():
    run = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert run.returncode == 2
    assert "single-GPU" in run.stderr and run.stdout.strip() == ""


def _write_counter_csv(path: Path, counter: str, rows: list[tuple[str, float]]) -> None:
    path.parent.mkdir(parents=True, exist_ok=True)
    with open(path, "w", newline="") as fh:
        w = csv.writer(fh, quoting=csv.QUOTE_NONNUMERIC)
        w.writerow(["Dispatch_Id", "Kernel_Name", "Counter_Name", "Counter_Value"])
        for i, (name, value) in enumerate(rows):
            w.writerow([i + 1, name, counter, value])
            w.writerow([i + 1, name, "SOME_OTHER_COUNTER", 1e9])


def test_traffic_calibration_ignores_the_runtimes_small_copies(bench, tmp_path):
    """A copy of known size fixes the worth of one count; a stray 4 KiB copy by the same runtime kernel must not move it
    (a mean over the copies would: 5 real copies + 1 small one reads 1.2x too many bytes per count)."""
    probe_kib = bench.COPY_PROBE_BYTES / 1024
    kernel = "k_softmax_reduce_abc123"
    fetch = [("__amd_rocclr_copyBuffer", probe_kib / 2)] * 5 + [("__amd_rocclr_copyBuffer", 2.0)] + [(kernel, probe_kib / 2 + 10)] * 13 + [("other_kernel", 7.0)]
    write = [("__amd_rocclr_copyBuffer", probe_kib)] * 5 + [("__amd_rocclr_copyBuffer", 4.0)] + [(kernel, probe_kib + 12)] * 13
    _write_counter_csv(tmp_path / "f" / "host" / "1_counter_collection.csv", "FETCH_SIZE", fetch)
    _write_counter_csv(tmp_path / "w" / "host" / "1_counter_collection.csv", "WRITE_SIZE", write)
    total = 0.0
    for sub, counter, worth in (("f", "FETCH_SIZE", 2048.0), ("w", "WRITE_SIZE", 1024.0)):
        sums = bench._counter_values(tmp_path / sub, counter)
        assert set(sums) >= {"__amd_rocclr_copyBuffer", kernel} and len(sums[kernel]) == 13
        per_count, counts = bench._calibrate(sums, kernel, counter)
        assert per_count == pytest.approx(worth)
        total += per_count * counts
    # one read and one write of the probe's bytes, plus the 10 and 12 extra counts at their worth
    assert total == pytest.approx(2 * bench.COPY_PROBE_BYTES + 10 * 2048 + 12 * 1024)


def test_traffic_calibration_fails_loudly_without_its_dispatches(bench, tmp_path):
    _write_counter_csv(tmp_path / "1_counter_collection.csv", "FETCH_SIZE", [("k_softmax_reduce_abc123", 5.0)])
    sums = bench._counter_values(tmp_path, "FETCH_SIZE")
    with pytest.raises(RuntimeError, match="no copy dispatches"):
        bench._calibrate(sums, "k_softmax_reduce_abc123", "FETCH_SIZE")
    with pytest.raises(RuntimeError, match="k_missing"):
        bench._calibrate({"__amd_rocclr_copyBuffer": [1.0]}, "k_missing", "FETCH_SIZE")


def test_recorded_traffic_is_keyed_by_kernel_name(bench):
    """The recorded figure belongs to one code object: another kernel name reads null, never a stale number."""
    assert bench.MEASURED_TRAFFIC_BYTES.get("k_softmax_reduce_000000") is None
    for name, value in bench.MEASURED_TRAFFIC_BYTES.items():
        assert name.startswith("k_softmax_reduce_") and 0.99 < value / (2 * bench.COPY_PROBE_BYTES) < 1.10


def test_recorded_traffic_names_the_kernel_the_headline_launches(bench):
    """The emitted kernel's name is a hash of its source: when the emitter changes, the name changes and the recorded
    traffic must be measured again (``bench.py --live-traffic``) instead of quietly turning into null."""
    import torch

    from deplodock_amd import HipBackend, trace_module
    from deplodock_amd.ir.hip import HipOp

    compiled = HipBackend().compile(trace_module(torch.nn.Softmax(dim=-1).eval(), (torch.empty(1, 28, 2048, 2048),)))
    names = [n.op.kernel_name for n in compiled.nodes.values() if isinstance(n.op, HipOp)]
    assert len(names) == 1 and names[0] in bench.MEASURED_TRAFFIC_BYTES, names
