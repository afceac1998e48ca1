"""Backend abstraction: ``Graph`` → compiled artifact → run / benchmark.

Same call surface as the reference's ``Backend`` ABC and result records
(emmy/compiler/backend/base.py:44-205):

    compiled = backend.compile(graph)
    result, pre = backend.run(compiled, input_data={...}, pre_run=fn)
    outputs = result.outputs        # dict[name, ndarray]
"""

from __future__ import annotations

from abc import ABC, abstractmethod
from collections.abc import Callable
from dataclasses import dataclass
from typing import Any


@dataclass
class RunResult:
    """Outputs of one program run as host arrays, plus optional wall time (base.py:44-49)."""

    outputs: dict[str, Any]
    time_ms: float | None = None


@dataclass
class LaunchTime:
    """Per-launch device-event timing inside a benchmark (base.py:52-66):
    ``time_ms`` is the median of ``samples`` (ms per single launch)."""

    idx: int
    kernel_name: str
    time_ms: float
    samples: tuple[float, ...] | None = None


@dataclass
class BenchmarkResult:
    """Result of benchmarking a program (base.py:69-91).

    ``time_ms``/``min_ms`` sum the per-launch windows (each replays one kernel
    back to back); ``e2e_ms`` times one graph holding every launch in program
    order.  ``captured`` says the windows were graph replays (pure device
    time) rather than plain launches."""

    time_ms: float
    min_ms: float | None = None
    max_ms: float | None = None
    num_launches: int = 0
    per_launch: list[LaunchTime] | None = None
    captured: bool = False
    e2e_ms: float | None = None
    e2e_min_ms: float | None = None


class Backend(ABC):
    """Abstract backend (base.py:94-205)."""

    name: str = "stub"
    bench_compile_timeout_s: float = 30.0
    bench_run_timeout_s: float = 10.0
    bench_wall_timeout_s: float | None = None

    @abstractmethod
    def compile(self, graph) -> Any:
        """Lower a ``Graph`` to a backend-specific runnable artifact."""

    @abstractmethod
    def run(self, compiled, *, input_data: dict | None = None, pre_run: Callable[[], Any] | None = None) -> tuple[RunResult, Any]:
        """Execute; return ``(RunResult, pre_run_result)``."""
