"""Shared fixtures.  ``gpu`` marks tests that need an MI355X; everything else runs on the CPU."""

from __future__ import annotations

import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a HIP device (run on an MI355X box)")
    # The benchmark worker's fork server must be a process that never touched the GPU: start it before any test does.
    from deplodock_amd.backend.hip.bench_worker import start_server

    start_server()


@pytest.fixture(scope="session")
def launcher_lib():
    """The in-tree ``libemmy_hip.so``; built once if the tree has none."""
    from deplodock_amd import config as cfg
    from deplodock_amd.backend.hip import launcher

    if not cfg.lib_path().exists():
        subprocess.run(["make", "-C", str(ROOT / "deplodock_amd" / "csrc")], check=True, capture_output=True)
    return launcher.load()


@pytest.fixture(scope="session")
def golden():
    return np.load(ROOT / "tests" / "golden" / "vectors.npz")


@pytest.fixture(autouse=True)
def _isolated_cache(tmp_path_factory, monkeypatch):
    """Keep knob pins of one test from leaking into the next."""
    for k in ("EMMY_REDUCE", "EMMY_TILE", "EMMY_STAGE", "EMMY_FLASH", "EMMY_KNOBS", "EMMY_NT", "EMMY_HIPRTC_FLAGS"):
        monkeypatch.delenv(k, raising=False)
    yield


@pytest.fixture(scope="session")
def device():
    import torch

    if not torch.cuda.is_available():
        pytest.fail("a gpu-marked test was collected on a host without a HIP device")
    return torch.device("cuda:0")
