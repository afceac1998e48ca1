"""Isolated, killable benchmark worker.

A benchmark that must not be able to stall its caller runs in a child process: the
parent hands over the lowered graph and the operands, waits for the answer for at
most ``wall_timeout_s`` and otherwise kills the child — its stream, and whatever is
queued behind a kernel that does not end, die with the process, and the next
benchmark starts a fresh child on a clean device.  Role of the reference's
``_AsyncBenchWorker`` / ``_bench_worker`` pair
(emmy/compiler/backend/cuda/program.py:1382-1533,
emmy/compiler/backend/cuda/_bench_worker.py), with two differences that follow from
the platform:

* children come from a ``multiprocessing`` **fork server**, not from an exec of the
  parent: the server is a clean process that never touches the GPU (start it before
  the parent's first GPU call — ``start_server()``; constructing a ``HipBackend``
  with ``bench_wall_timeout_s`` does), and every worker is a fork of it, so no
  process that holds a GPU context is ever replaced or duplicated;
* operands travel as host arrays (bf16 as ``uint16`` bit patterns) and are uploaded
  by the child; device tensors of the parent are copied to the host first.

After any failure the child reports and exits (a failed launch can leave its context
unusable, and after the hung-kernel watchdog a synchronisation would never return);
a healthy child is kept and reused.
"""

from __future__ import annotations

import logging
import multiprocessing as mp
import time
import traceback

logger = logging.getLogger(__name__)

_PRELOAD = ["deplodock_amd.backend.hip.bench_worker", "deplodock_amd.backend.hip.program", "numpy", "torch"]


def _context():
    return mp.get_context("forkserver")


def start_server() -> None:
    """Start the fork server now (idempotent).  Call it before the process first touches the GPU;
    afterwards every worker is forked from that clean server."""
    ctx = _context()
    ctx.set_forkserver_preload(_PRELOAD)
    from multiprocessing import forkserver

    forkserver.ensure_running()


def _to_wire(data: dict | None) -> dict:
    """Operands as host arrays: tensors leave the device, bf16 becomes ``uint16`` bit patterns."""
    import numpy as np

    out = {}
    for name, v in (data or {}).items():
        if hasattr(v, "detach"):  # a torch tensor
            import torch

            t = v.detach().cpu().contiguous()
            out[name] = t.view(torch.int16).numpy().view(np.uint16) if t.dtype == torch.bfloat16 else t.numpy()
        else:
            out[name] = np.asarray(v)
    return out


def _plain_graph(graph):
    """The lowered graph without what only the parent needs (re-trace recipe, size variants, traced values)."""
    from dataclasses import replace

    g = graph.copy()
    for node in g.nodes.values():
        if getattr(node.op, "source", None) is not None:
            node.op = replace(node.op, source=None)  # the lowering chain behind a kernel is attribution only
        node.hints = {k: v for k, v in node.hints.items() if k in ("stacked", "output_alias")}
    return g


def _serve(conn, device_id) -> None:
    """Child main loop: one request at a time until the pipe closes or a job fails."""
    while True:
        try:
            req = conn.recv()
        except (EOFError, OSError):
            return
        if req is None:
            return
        try:
            from deplodock_amd import config
            from deplodock_amd.backend.hip.program import benchmark_program

            if device_id is not None:
                import torch

                torch.cuda.set_device(device_id)
            with config.hiprtc_flags_override(req.get("hiprtc_flags")):
                result = benchmark_program(req["graph"], input_data=req["input_data"], **req["kwargs"])
            conn.send({"ok": True, "result": result})
        except BaseException as exc:  # noqa: BLE001 - everything is reported to the parent
            try:
                conn.send({"ok": False, "error": f"{type(exc).__name__}: {exc}", "traceback": traceback.format_exc()})
            finally:
                return  # the context may be unusable (or hold a kernel that never ends): leave it to process teardown


class BenchWorker:
    """Parent-side handle of one worker process (spawned on first use, respawned after a kill)."""

    def __init__(self, *, device_id: int | None = None) -> None:
        self.device_id = device_id
        self._proc = None
        self._conn = None
        self.spawned = 0
        self.killed = 0

    def _spawn(self) -> None:
        start_server()
        ctx = _context()
        parent, child = ctx.Pipe()
        proc = ctx.Process(target=_serve, args=(child, self.device_id), daemon=True)
        proc.start()
        child.close()
        self._proc, self._conn = proc, parent
        self.spawned += 1
        logger.info("[bench-worker] spawned pid=%s device=%s", proc.pid, self.device_id)

    def _alive(self) -> bool:
        return self._proc is not None and self._proc.is_alive()

    def _kill(self) -> None:
        proc, conn = self._proc, self._conn
        self._proc = self._conn = None
        if conn is not None:
            conn.close()
        if proc is not None and proc.is_alive():
            proc.kill()
            self.killed += 1
        if proc is not None:
            proc.join(5.0)

    def close(self) -> None:
        if self._alive():
            try:
                self._conn.send(None)
                self._proc.join(2.0)
            except (OSError, ValueError):
                pass
        self._kill()

    def run_job(self, request: dict, *, wall_timeout_s: float) -> dict:
        """Send one request and return the response; a worker that has not answered after
        ``wall_timeout_s`` is killed and ``RuntimeError`` raised (the caller's bench_fail)."""
        deadline = time.perf_counter() + wall_timeout_s
        for attempt in (0, 1):
            if not self._alive():
                self._kill()
                self._spawn()
            try:
                self._conn.send(request)
            except (BrokenPipeError, OSError) as exc:
                self._kill()
                if attempt == 1:
                    raise RuntimeError(f"bench worker died during request send: {exc}") from exc
                continue
            remaining = deadline - time.perf_counter()
            try:
                ready = remaining > 0 and self._conn.poll(remaining)
                if not ready:
                    self._kill()
                    raise RuntimeError(f"bench worker exceeded {wall_timeout_s:.1f}s wall budget — killed, stream cleaned")
                resp = self._conn.recv()
            except EOFError as exc:
                self._kill()
                raise RuntimeError("bench worker ended before it answered") from exc
            if not resp.get("ok"):
                self._kill()  # it exits by itself after a failure; make sure before the next job
                raise RuntimeError(f"bench worker error: {resp.get('error', '?')}")
            return resp
        raise RuntimeError("bench worker unreachable")


def benchmark_program_isolated(graph, *, worker: BenchWorker, wall_timeout_s: float, input_data: dict | None = None, hiprtc_flags: str | None = None, **kwargs):
    """``benchmark_program`` in ``worker``'s process under a wall-clock limit (program.py:1536-1580)."""
    request = {"graph": _plain_graph(graph), "input_data": _to_wire(input_data), "hiprtc_flags": hiprtc_flags, "kwargs": kwargs}
    return worker.run_job(request, wall_timeout_s=wall_timeout_s)["result"]


__all__ = ["BenchWorker", "benchmark_program_isolated", "start_server"]
