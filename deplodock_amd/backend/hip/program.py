"""Program runtime: buffers, scratch slab, launches, graphs and event timing.

Takes a lowered ``Graph[HipOp + InputOp + ConstantOp]`` and runs it on the
current HIP device through ``libemmy_hip.so``.  Same responsibilities as the
reference's ``program.py`` (emmy/compiler/backend/cuda/program.py: ``_compile``
:177-226, ``_allocate`` :340-364, ``_launch`` :394-424, ``CompiledProgram``
:614-1090, ``benchmark_program`` :1152-1325) with two deliberate differences:
device memory is PyTorch-ROCm tensors (the launcher only borrows their
pointers), and inputs that already live on the device are used in place.
"""

from __future__ import annotations

import contextlib
import fcntl
import logging
import statistics
import time
from dataclasses import dataclass, field

import numpy as np

from deplodock_amd import config
from deplodock_amd.backend import BenchmarkResult, LaunchTime, RunResult
from deplodock_amd.backend.hip import hiprtc, launcher
from deplodock_amd.backend.hip.launcher import PackedArgs
from deplodock_amd.dtype import BF16, DType, bf16_bits_from_f32, to_torch
from deplodock_amd.graph import Graph, Node
from deplodock_amd.ir.base import ConstantOp, InputOp
from deplodock_amd.ir.hip import HipOp, resolve_dim

logger = logging.getLogger(__name__)

_STATIC_LDS_CAP = 64 * 1024  # per-workgroup LDS available without opting in
_KERNEL_TIMEOUT_MS = 1000.0  # per-window watchdog
_WARMUP_TARGET_MS = 10.0  # keep warming until this much device time has run
_BATCH_TARGET_MS = 1.0  # launches per event window are sized to cover this
_PASS_TARGET_MS = 100.0  # ... but a pass over all of a program's windows to no more than this (a program of hundreds of launches)
_AUTO_BUDGET_MS = 100.0
_AUTO_MAX_ITERS = 20000
_SLAB_ALIGN = 256
_E2E_MAX_COPIES = 64  # program copies one whole-program timing graph holds at most


class HungKernelError(RuntimeError):
    """An event window did not complete within the watchdog budget."""


class GraphCaptureError(RuntimeError):
    """Capturing launches into a HIP graph failed; timing falls back to plain launches."""


@contextlib.contextmanager
def gpu_lock():
    """Cross-process device lock (``EMMY_GPU_LOCK``; emmy/compiler/backend/gpu_lock.py)."""
    path = config.gpu_lock_path()
    try:
        fh = open(path, "a+")
    except OSError:
        yield
        return
    try:
        fcntl.flock(fh, fcntl.LOCK_EX)
        yield
    finally:
        fcntl.flock(fh, fcntl.LOCK_UN)
        fh.close()


# ---------------------------------------------------------------------------
# Compile: kernels + buffer plan + launch list
# ---------------------------------------------------------------------------


@dataclass
class _Buffer:
    name: str
    shape: tuple
    dtype: DType
    role: str  # input | constant | output | scratch

    def resolve_shape(self, sym_values: dict[str, int]) -> tuple[int, ...]:
        """The shape at this launch's symbolic sizes: a ``str`` dim is a bare symbol, an ``Affine`` ``a * symbol + b``."""
        return tuple(int(sym_values[d]) if isinstance(d, str) else int(d.at(sym_values)) if hasattr(d, "at") else int(d) for d in self.shape)


@dataclass
class _Launch:
    node_id: str
    kernel_name: str
    arg_names: tuple[str, ...]
    grid: tuple
    block: tuple
    lds_bytes: int
    zero_outputs: tuple[str, ...]
    runtime_args: tuple[str, ...] = ()
    algo_bytes: int = 0
    algo_flops: int = 0


@dataclass
class _Compiled:
    bufs: list[_Buffer]
    buf_by_name: dict[str, _Buffer]
    constants: dict[str, float]
    kernels: dict[str, hiprtc.LoadedKernel]
    launches: list[_Launch]
    symbolic_bindings: dict[str, tuple[str, int]] = field(default_factory=dict)
    symbolic_hints: dict[str, int] = field(default_factory=dict)  # the sizes the graph was traced at (used when an input is not supplied)


_ZERO_KERNEL_NAME = "emh_zero_words"
_ZERO_KERNEL_SRC = r"""
extern "C" __global__ __launch_bounds__(256) void emh_zero_words(unsigned int* __restrict__ p, int n) {
  for (int i = blockIdx.x * 256 + threadIdx.x; i < n; i += gridDim.x * 256) p[i] = 0u;
}
"""


def _kernel_nodes(graph: Graph) -> list[Node]:
    """The graph's launches in program order; anything that is neither a kernel nor an input / constant is a
    lowering bug and is reported by node."""
    order = [graph.nodes[nid] for nid in graph.topological_order()]
    stray = next((n for n in order if not isinstance(n.op, (InputOp, ConstantOp, HipOp))), None)
    if stray is not None:
        raise TypeError(f"HipBackend: node {stray.id!r} has non-HipOp {type(stray.op).__name__!r}; lowering must produce Graph[HipOp].")
    return [n for n in order if isinstance(n.op, HipOp)]


def _buffers(graph: Graph) -> list[_Buffer]:
    return [_Buffer(nid, tuple(graph.nodes[nid].output.shape), graph.nodes[nid].output.dtype, graph.node_role(nid)) for nid in graph.topological_order()]


def _symbolic_bindings(graph: Graph) -> dict[str, tuple[str, int]]:
    out: dict[str, tuple[str, int]] = {}
    for nid in graph.inputs:
        for i, d in enumerate(graph.nodes[nid].output.shape):
            if isinstance(d, str) and d not in out:
                out[d] = (nid, i)
    return out


def _compile(graph: Graph) -> _Compiled:
    bufs = _buffers(graph)
    launches: list[_Launch] = []
    sources: dict[str, str] = {}
    # Pass 1 — validate the whole graph before anything touches the device.
    for node in _kernel_nodes(graph):
        op: HipOp = node.op
        kname = op.kernel_name
        if sources.setdefault(kname, op.kernel_source) != op.kernel_source:
            raise ValueError(f"kernel name {kname!r} used by two distinct sources")
        known = {b.name for b in bufs}
        for arg in (*op.arg_order, *op.zero_outputs):
            if arg not in known:
                raise KeyError(f"kernel {kname!r} references unknown buffer {arg!r}")
        launches.append(
            _Launch(
                node_id=node.id,
                kernel_name=kname,
                arg_names=tuple(op.arg_order),
                grid=op.grid,
                block=op.block,
                lds_bytes=op.lds_bytes,
                zero_outputs=tuple(op.zero_outputs),
                runtime_args=tuple(op.runtime_args),
                algo_bytes=op.algo_bytes,
                algo_flops=op.algo_flops,
            )
        )
    if any(ln.zero_outputs for ln in launches):
        sources[_ZERO_KERNEL_NAME] = _ZERO_KERNEL_SRC
    # Pass 2 — compile (cached) and load.
    kernels = {name: hiprtc.load_function(src, name) for name, src in sources.items()}
    constants = {nid: float(op.value) for nid, op in graph.constant_ops() if op.value is not None}
    hints = dict(getattr(getattr(graph, "dynamic", None), "hints", {}) or {})
    return _Compiled(bufs, {b.name: b for b in bufs}, constants, kernels, launches, _symbolic_bindings(graph), hints)


# ---------------------------------------------------------------------------
# Scratch planning (role of the reference's backend/cuda/_planner.py)
# ---------------------------------------------------------------------------


def compute_live_intervals(names: list[str], launches: list[_Launch]) -> dict[str, tuple[int, int]]:
    """``name -> (first launch index that touches it, last one)``."""
    out: dict[str, tuple[int, int]] = {}
    wanted = set(names)
    for i, ln in enumerate(launches):
        for n in (*ln.arg_names, *ln.zero_outputs):
            if n in wanted:
                lo, hi = out.get(n, (i, i))
                out[n] = (min(lo, i), max(hi, i))
    for n in names:
        out.setdefault(n, (0, max(len(launches) - 1, 0)))
    return out


def plan_offsets(intervals: dict[str, tuple[int, int]], sizes: dict[str, int], align: int = _SLAB_ALIGN) -> tuple[dict[str, int], int]:
    """Greedy first-fit: buffers whose live intervals overlap never share bytes.
    Largest first; each lands at the lowest aligned offset free for its interval."""
    placed: list[tuple[int, int, int, int]] = []  # (offset, end, lo, hi)
    offsets: dict[str, int] = {}
    total = 0
    for name in sorted(sizes, key=lambda n: (-sizes[n], n)):
        size = -(-sizes[name] // align) * align
        lo, hi = intervals[name]
        conflicts = sorted((o, e) for o, e, plo, phi in placed if not (phi < lo or hi < plo))
        off = 0
        for o, e in conflicts:
            if off + size <= o:
                break
            off = max(off, e)
        offsets[name] = off
        placed.append((off, off + size, lo, hi))
        total = max(total, off + size)
    return offsets, total


# ---------------------------------------------------------------------------
# Buffer materialization
# ---------------------------------------------------------------------------


def _torch():
    import torch

    return torch


def _device():
    torch = _torch()
    if not torch.cuda.is_available():
        raise launcher.LauncherError("no HIP device is visible: the HIP backend cannot run (there is no CPU fallback)")
    return torch.device("cuda", torch.cuda.current_device())


def _to_device(src, buf: _Buffer, shape: tuple[int, ...]):
    """Host array / tensor → device tensor of ``buf``'s dtype.  A device tensor
    that already matches is used in place (no copy)."""
    torch = _torch()
    want = to_torch(buf.dtype)
    if isinstance(src, torch.Tensor):
        t = src
        if t.dtype != want:
            raise TypeError(f"buffer {buf.name!r}: expected {want}, got {t.dtype}")
        t = t.reshape(shape)
        if not t.is_cuda:
            t = t.contiguous().to(_device())
        elif not t.is_contiguous():
            t = t.contiguous()
        return t
    arr = np.asarray(src)
    if buf.dtype is BF16:
        if arr.dtype != np.uint16:
            arr = bf16_bits_from_f32(np.asarray(arr, dtype=np.float32))
        arr = np.ascontiguousarray(arr).reshape(shape)
        return torch.from_numpy(arr.view(np.int16)).to(_device()).view(torch.bfloat16)
    arr = np.ascontiguousarray(arr, dtype=buf.dtype.np).reshape(shape)
    return torch.from_numpy(arr).to(_device())


def _materialize(buf: _Buffer, shape: tuple[int, ...], src, constants: dict[str, float]):
    torch = _torch()
    if src is not None:
        return _to_device(src, buf, shape)
    want = to_torch(buf.dtype)
    if buf.role == "constant":
        if buf.name not in constants:
            raise KeyError(f"constant {buf.name!r} has no static value and was not supplied in input_data")
        return torch.full(shape, constants[buf.name], dtype=want, device=_device())
    if buf.role == "input":
        # Deterministic pseudo-random fill for un-supplied inputs, values in
        # [-0.5, 0.5] (same recipe as emmy/compiler/backend/cuda/program.py:265-276).
        n = int(np.prod(shape)) if shape else 1
        idx = np.arange(n, dtype=np.int64)
        vals = (0.01 * ((idx.astype(np.float32) * 7 + 13) % 101 - 50)).astype(np.float32)
        return torch.from_numpy(vals.reshape(shape)).to(_device()).to(want)
    return torch.zeros(shape, dtype=want, device=_device())


def _resolve_symbolic(compiled: _Compiled, input_data: dict) -> dict[str, int]:
    env: dict[str, int] = {}
    for name, (buf, dim) in compiled.symbolic_bindings.items():
        arr = input_data.get(buf)
        if arr is None:
            if name in compiled.symbolic_hints:
                env[name] = int(compiled.symbolic_hints[name])  # synthetic inputs: the traced size
                continue
            raise ValueError(f"symbolic dim {name!r} reads from input {buf!r}.shape[{dim}] but no array was supplied")
        env[name] = int(arr.shape[dim])
    for name, (buf, dim) in compiled.symbolic_bindings.items():
        # every input that carries the symbol must agree on it
        for b in compiled.bufs:
            if b.role == "input" and b.name in input_data and b.name != buf:
                for i, d in enumerate(b.shape):
                    if d == name and int(input_data[b.name].shape[i]) != env[name]:
                        raise ValueError(f"inputs disagree on {name!r}: {buf!r} gives {env[name]}, {b.name!r} gives {int(input_data[b.name].shape[i])}")
    return env


def _host(t, dtype: DType) -> np.ndarray:
    """Device tensor → host ndarray (bf16 as uint16 bit patterns)."""
    torch = _torch()
    if dtype is BF16:
        return t.view(torch.int16).cpu().numpy().view(np.uint16)
    return t.cpu().numpy()


# ---------------------------------------------------------------------------
# CompiledProgram
# ---------------------------------------------------------------------------


@dataclass(frozen=True)
class _LibraryScratch:
    """A scratch buffer that lives in the launcher library's own device array (``emh_launch_scratch``)
    instead of a tensor: the bytes ``[offset, offset + nbytes)`` of that array."""

    offset: int
    nbytes: int


class CompiledProgram:
    """A compiled graph bound to device buffers, ready to launch repeatedly.

    Scratch buffers are typed views into one liveness-planned slab that lives
    as long as the program, so pointers baked into argument packs and captured
    graphs stay valid across replays (program.py:281-337)."""

    def __init__(self, compiled: _Compiled, arrays: dict, sym_values: dict[str, int], slab, slab_bytes: int, naive_bytes: int):
        self.lib = launcher.load()
        self.compiled = compiled
        self.arrays = arrays
        self.sym_values = sym_values
        self._slab = slab
        self.slab_bytes = slab_bytes
        self.naive_scratch_bytes = naive_bytes
        self._packs: list[tuple] = []  # (args, grid, block, fills of zeroed outputs, borrowed scratch range or None) per launch
        self._stream: int | None = None  # private stream for capture / timing
        self._launch_graphs: dict[int, int] = {}
        self._launch_graph_sizes: list[int] | None = None
        self._program_graph: int | None = None
        self._program_graph_repeat = 1
        self._events: list[int] = []
        self._hung = False  # set by the watchdog: the private stream may never drain
        self._build_packs()

    # -- construction ---------------------------------------------------------
    @classmethod
    def build(cls, graph: Graph, input_data: dict | None = None, compile_timeout_s: float | None = None, library_scratch: bool = False) -> CompiledProgram:
        """``library_scratch``: intermediates (the workspace of a split contraction) are not allocated at all;
        each launch borrows the launcher library's device scratch array through ``emh_launch_scratch``, for
        callers that must not allocate.  Limits: the planned scratch must fit that array, and a launch may name
        one scratch buffer only."""
        t0 = time.perf_counter()
        compiled = _compile(graph)
        input_data = dict(input_data or {})
        sym_values = _resolve_symbolic(compiled, input_data)
        torch = _torch()
        arrays: dict = {}
        for buf in compiled.bufs:
            if buf.role == "scratch":
                continue
            shape = buf.resolve_shape(sym_values) or (1,)
            arrays[buf.name] = _materialize(buf, shape, input_data.get(buf.name), compiled.constants)
        sizes = {}
        for buf in compiled.bufs:
            if buf.role == "scratch":
                shape = buf.resolve_shape(sym_values) or (1,)
                sizes[buf.name] = max(1, int(np.prod(shape))) * buf.dtype.nbytes
        intervals = compute_live_intervals(list(sizes), compiled.launches)
        offsets, total = plan_offsets(intervals, sizes)
        if library_scratch:
            # what the library checks per launch is offset + size rounded up to whole 32-bit words
            need = max((off + -(-sizes[name] // 4) * 4 for name, off in offsets.items()), default=0)
            if max(total, need) > launcher.EMH_SCRATCH_MAX_BYTES:
                raise ValueError(f"the program's intermediates need {max(total, need)} bytes; the library's scratch array holds {launcher.EMH_SCRATCH_MAX_BYTES}")
            slab = None
            for name, off in offsets.items():
                arrays[name] = _LibraryScratch(off, -(-sizes[name] // 4) * 4)
        else:
            slab = torch.zeros(max(total, _SLAB_ALIGN), dtype=torch.uint8, device=_device())
        for buf in compiled.bufs:
            if buf.role == "scratch" and not library_scratch:
                shape = buf.resolve_shape(sym_values) or (1,)
                off = offsets[buf.name]
                arrays[buf.name] = slab[off : off + sizes[buf.name]].view(to_torch(buf.dtype)).view(shape)
        prog = cls(compiled, arrays, sym_values, slab, total, sum(sizes.values()))
        # Uploads ran on torch's stream; timing and capture use a private one.
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
        if compile_timeout_s is not None and elapsed > compile_timeout_s:
            raise RuntimeError(f"benchmark compile stage exceeded {compile_timeout_s:.1f}s ({elapsed:.1f}s) — variant marked bench_fail")
        return prog

    def _build_packs(self) -> None:
        self._packs = []
        for ln in self.compiled.launches:
            ptrs = []
            scratch = None  # (parameter index, offset, bytes, clear first) when the launch borrows the library's scratch array
            for i, name in enumerate(ln.arg_names):
                t = self.arrays[name]
                if isinstance(t, _LibraryScratch):
                    if scratch is not None:
                        # also for one buffer named in two parameter slots: the library repoints a single slot
                        raise ValueError(f"kernel {ln.kernel_name!r} takes scratch memory in two parameter slots; a launch can borrow one range of the library's scratch array for one parameter")
                    scratch = (i, t.offset, t.nbytes, name in ln.zero_outputs)
                    ptrs.append(0)
                    continue
                ptr = t.data_ptr()
                if ptr % 16:
                    raise ValueError(f"buffer {name!r} is not 16-byte aligned (vector loads require it)")
                ptrs.append(ptr)
            ints = [self.sym_values[n] for n in ln.runtime_args]
            pack = PackedArgs(ptrs, ints)
            grid = tuple(resolve_dim(s, self.sym_values) for s in ln.grid)
            block = tuple(resolve_dim(s, self.sym_values) for s in ln.block)
            zero_packs = []
            for z in ln.zero_outputs:
                t = self.arrays[z]
                if isinstance(t, _LibraryScratch):
                    continue  # cleared by emh_launch_scratch itself
                nbytes = t.numel() * t.element_size()
                if nbytes % 4:
                    raise ValueError(f"zero_outputs buffer {z!r} is not a whole number of 32-bit words")
                zero_packs.append((PackedArgs([t.data_ptr()], [nbytes // 4]), nbytes // 4))
            if ln.lds_bytes > _STATIC_LDS_CAP:
                self.lib.func_set_dynamic_lds(self.compiled.kernels[ln.kernel_name].fn, ln.lds_bytes)
            self._packs.append((pack, grid, block, zero_packs, scratch))

    # -- launching ----------------------------------------------------------------
    def _torch_stream(self) -> int:
        return int(_torch().cuda.current_stream().cuda_stream)

    def launch_one(self, i: int, stream: int | None) -> None:
        ln = self.compiled.launches[i]
        pack, grid, block, zero_packs, scratch = self._packs[i]
        for zp, words in zero_packs:
            zgrid = (max(1, min(1024, -(-words // 256))), 1, 1)
            self.lib.launch(self.compiled.kernels[_ZERO_KERNEL_NAME].fn, zgrid, (256, 1, 1), 0, stream, zp)
        if grid[0] * grid[1] * grid[2] == 0:
            return  # an empty index space (zero rows): nothing to compute, and the driver rejects empty grids
        if scratch is not None:
            self.lib.launch_scratch(self.compiled.kernels[ln.kernel_name].fn, grid, block, ln.lds_bytes, stream, pack, *scratch)
        else:
            self.lib.launch(self.compiled.kernels[ln.kernel_name].fn, grid, block, ln.lds_bytes, stream, pack)

    def run(self, stream: int | None = None) -> None:
        """Issue every launch once, in program order, on ``stream`` (default: torch's current stream)."""
        s = self._torch_stream() if stream is None else stream
        for i in range(len(self.compiled.launches)):
            self.launch_one(i, s)

    def outputs(self) -> dict[str, np.ndarray]:
        _torch().cuda.synchronize()
        return {b.name: _host(self.arrays[b.name], b.dtype) for b in self.compiled.bufs if b.role == "output"}

    def snapshot(self) -> dict[str, np.ndarray]:
        """Host copies of every buffer the program writes (scratch and outputs), as they are now."""
        _torch().cuda.synchronize()
        return {b.name: _host(self.arrays[b.name], b.dtype) for b in self.compiled.bufs if b.role in ("scratch", "output") and b.name in self.arrays}

    def output_tensors(self) -> dict:
        return {b.name: self.arrays[b.name] for b in self.compiled.bufs if b.role == "output"}

    # -- timing -----------------------------------------------------------------------
    def _ensure_stream(self) -> int:
        if self._stream is None:
            self._stream = self.lib.stream_create()
        return self._stream

    def _event(self) -> int:
        e = self.lib.event_create()
        self._events.append(e)
        return e

    def _wait_for_event(self, event: int, what: str) -> None:
        """Poll instead of blocking so a hung kernel raises instead of stalling (program.py:574-611)."""
        deadline = time.perf_counter() + _KERNEL_TIMEOUT_MS / 1000.0
        while not self.lib.event_query(event):
            if time.perf_counter() > deadline:
                self._hung = True
                raise HungKernelError(f"{what} did not finish within {_KERNEL_TIMEOUT_MS:.0f} ms")
            time.sleep(0)

    def _elapsed(self, start: int, stop: int, what: str) -> float:
        ms = self.lib.event_elapsed_ms(start, stop)
        if not ms > 0.0:
            raise RuntimeError(f"{what} reported {ms:.3f}ms elapsed — degenerate launch, variant marked bench_fail")
        return ms

    def iter_once(self, batch_sizes: list[int], pre_iter=None) -> list[float]:
        """One benchmark iteration: for each launch, one event window around
        ``batch_sizes[i]`` back-to-back issues (a graph replay when captured).
        Returns per-launch ms normalised to one issue."""
        stream = self._ensure_stream()
        if pre_iter is not None:
            pre_iter(max(batch_sizes) if batch_sizes else 1)
        out: list[float] = []
        if not hasattr(self, "_win"):
            self._win = (self._event(), self._event())
        start, stop = self._win
        for i, ln in enumerate(self.compiled.launches):
            self.lib.event_record(start, stream)
            g = self._launch_graphs.get(i) if self._launch_graph_sizes == batch_sizes else None
            if g is not None:
                self.lib.graph_launch(g, stream)
            else:
                for _ in range(batch_sizes[i]):
                    self.launch_one(i, stream)
            self.lib.event_record(stop, stream)
            self._wait_for_event(stop, f"kernel {ln.kernel_name!r}")
            out.append(self._elapsed(start, stop, f"kernel {ln.kernel_name!r}") / batch_sizes[i])
        return out

    def capture_launch_graphs(self, batch_sizes: list[int]) -> None:
        """Capture each launch's batch into its own graph; no-op when already captured at these sizes."""
        if self._launch_graph_sizes == batch_sizes:
            return
        self._drop_launch_graphs()
        stream = self._ensure_stream()
        self.lib.stream_synchronize(stream)
        try:
            for i in range(len(self.compiled.launches)):
                self.lib.graph_begin_capture(stream)
                try:
                    for _ in range(batch_sizes[i]):
                        self.launch_one(i, stream)
                except BaseException:
                    # the capture must still be ended, and the graph it hands back released
                    with contextlib.suppress(launcher.LauncherError):
                        self.lib.graph_destroy(self.lib.graph_end_capture(stream))
                    raise
                self._launch_graphs[i] = self.lib.graph_end_capture(stream)
        except launcher.LauncherError as exc:
            self._drop_launch_graphs()
            raise GraphCaptureError(f"graph capture failed: {exc}") from exc
        self._launch_graph_sizes = list(batch_sizes)

    def _drop_launch_graphs(self) -> None:
        for g in self._launch_graphs.values():
            self.lib.graph_destroy(g)
        self._launch_graphs = {}
        self._launch_graph_sizes = None

    def capture_program_graph(self, repeat: int = 1) -> None:
        """One graph holding every launch in program order, ``repeat`` times back to back.  Timing windows use
        ``repeat`` > 1 so that what they measure is device time: one graph launch per replay of a program of a
        few short kernels would add the host's per-graph launch latency (several microseconds) to every replay,
        which a caller that chains programs inside one graph — a model is many blocks — never pays."""
        repeat = max(1, int(repeat))
        if self._program_graph is not None and self._program_graph_repeat == repeat:
            return
        if self._program_graph is not None:
            self.lib.graph_destroy(self._program_graph)
            self._program_graph = None
        stream = self._ensure_stream()
        self.lib.stream_synchronize(stream)
        try:
            self.lib.graph_begin_capture(stream)
            try:
                for _ in range(repeat):
                    self.run(stream)
            except BaseException:
                with contextlib.suppress(launcher.LauncherError):
                    self.lib.graph_destroy(self.lib.graph_end_capture(stream))
                raise
            g = self.lib.graph_end_capture(stream)
        except launcher.LauncherError as exc:
            raise GraphCaptureError(f"whole-program graph capture failed: {exc}") from exc
        self._program_graph, self._program_graph_repeat = g, repeat

    def replay_program(self, stream: int | None = None) -> None:
        if self._program_graph is None or self._program_graph_repeat != 1:
            self.capture_program_graph()
        self.lib.graph_launch(self._program_graph, self._ensure_stream() if stream is None else stream)

    def time_program_window(self, replays: int) -> float:
        """ms per whole-program run over one event window of ``replays`` launches of the program graph (each
        holding the program ``repeat`` times)."""
        stream = self._ensure_stream()
        if not hasattr(self, "_win"):
            self._win = (self._event(), self._event())
        start, stop = self._win
        self.lib.event_record(start, stream)
        for _ in range(replays):
            self.lib.graph_launch(self._program_graph, stream)
        self.lib.event_record(stop, stream)
        self._wait_for_event(stop, "whole-program graph")
        return self._elapsed(start, stop, "whole-program graph") / (replays * self._program_graph_repeat)

    def close(self) -> None:
        """Release graphs, events and the private stream.  The kernels' modules are shared through
        ``hiprtc.load_function``'s per-device cache and stay loaded.  After the watchdog has fired the
        stream may hold a kernel that never ends: waiting for it, or destroying it (which waits too),
        would turn the ``HungKernelError`` into a stall, so the stream and what is queued on it are
        abandoned to process teardown."""
        if self._hung:
            self._launch_graphs, self._launch_graph_sizes, self._program_graph = {}, None, None
            self._events, self._stream = [], None
            if hasattr(self, "_win"):
                del self._win
            return
        self._drop_launch_graphs()
        if self._program_graph is not None:
            self.lib.graph_destroy(self._program_graph)
            self._program_graph = None
        for e in self._events:
            self.lib.event_destroy(e)
        self._events = []
        if hasattr(self, "_win"):
            del self._win
        if self._stream is not None:
            self.lib.stream_synchronize(self._stream)
            self.lib.stream_destroy(self._stream)
            self._stream = None


# ---------------------------------------------------------------------------
# Entry points
# ---------------------------------------------------------------------------


def run_program(graph: Graph, input_data: dict | None = None, pre_run=None) -> tuple[RunResult, object]:
    """Compile, allocate, launch once and fetch outputs — all inside the GPU lock (program.py:1098-1119)."""
    with gpu_lock():
        prog = CompiledProgram.build(graph, input_data)
        try:
            pre_result = pre_run() if pre_run is not None else None
            torch = _torch()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            prog.run()
            torch.cuda.synchronize()
            elapsed = (time.perf_counter() - t0) * 1000.0
            outputs = prog.outputs()
        finally:
            prog.close()
    return RunResult(outputs=outputs, time_ms=elapsed), pre_result


@dataclass
class DebugResult:
    """What a debug run keeps: the program's outputs and, per launch index, a host copy of every buffer that is
    not an input or a constant, taken right after that launch finished (the reference's ``DebugResult``,
    emmy/compiler/backend/cuda/program.py:1122-1125)."""

    outputs: dict[str, np.ndarray]
    per_launch: dict[int, dict[str, np.ndarray]] = field(default_factory=dict)
    kernel_names: dict[int, str] = field(default_factory=dict)


def run_program_debug(graph: Graph, input_data: dict | None = None, pre_run=None) -> tuple[DebugResult, object]:
    """Run the program once, launch by launch, synchronising after each launch and copying every scratch and
    output buffer to the host (program.py:1128-1149).  Scratch buffers share one slab planned by live interval:
    a buffer read *after its last use* shows whatever took its place, a launch's own output is what that launch
    wrote."""
    shots: dict[int, dict[str, np.ndarray]] = {}
    names: dict[int, str] = {}
    with gpu_lock():
        prog = CompiledProgram.build(graph, input_data)
        try:
            pre_result = pre_run() if pre_run is not None else None
            torch = _torch()
            stream = prog._torch_stream()
            for i, ln in enumerate(prog.compiled.launches):
                prog.launch_one(i, stream)
                torch.cuda.synchronize()
                shots[i] = prog.snapshot()
                names[i] = ln.kernel_name
            outputs = prog.outputs()
        finally:
            prog.close()
    return DebugResult(outputs=outputs, per_launch=shots, kernel_names=names), pre_result


@dataclass(frozen=True)
class SampleBudget:
    """When sampling stops: after ``max_samples`` measured passes, or — ``device_ms`` set, the ``"auto"`` mode — once
    that much device time has been measured, whichever comes first."""

    max_samples: int
    device_ms: float | None = None

    @classmethod
    def parse(cls, num_iters) -> "SampleBudget":
        if num_iters == "auto":
            return cls(_AUTO_MAX_ITERS, _AUTO_BUDGET_MS)
        if isinstance(num_iters, str):
            raise ValueError(f"num_iters must be an int or 'auto', got {num_iters!r}")
        return cls(int(num_iters))

    def spent(self, samples: int, measured_ms: float) -> bool:
        return samples >= self.max_samples or (self.device_ms is not None and measured_ms >= self.device_ms)


def window_issues(per_issue_ms: float, target_ms: float = _BATCH_TARGET_MS) -> int:
    """Back-to-back issues of one launch that make an event window of about ``target_ms``."""
    if not 0.0 < per_issue_ms < target_ms:
        return 1
    return max(1, round(target_ms / per_issue_ms))


class _BenchSession:
    """The three phases of a benchmark over one built program: *probe* (single issues, to learn how long each
    launch takes), *settle* (size the event windows from the probe, capture them into graphs, keep the device
    busy until it has warmed up) and *sample*.  Every pass over the program goes through ``_pass``, which keeps
    the device-time account the run budget is checked against."""

    def __init__(self, prog: "CompiledProgram", *, on_iter, run_timeout_s: float | None, capture: bool) -> None:
        self.prog = prog
        self.on_iter = on_iter
        self.limit_ms = None if run_timeout_s is None else run_timeout_s * 1000.0
        self.capture = capture
        self.n = len(prog.compiled.launches)
        self.issues = [1] * self.n
        self.device_ms = 0.0
        self.last: list[float] = []

    def _charge(self, ms: float) -> None:
        self.device_ms += ms
        if self.limit_ms is not None and self.device_ms > self.limit_ms:
            raise RuntimeError(f"benchmark run stage exceeded {self.limit_ms / 1000.0:.1f}s of GPU time — variant marked bench_fail")

    def _pass(self) -> float:
        """One pass over the program's windows; returns the device time it took."""
        self.last = self.prog.iter_once(self.issues, pre_iter=self.on_iter)
        took = sum(dt * k for dt, k in zip(self.last, self.issues))
        self._charge(took)
        return took

    def _capture_windows(self) -> None:
        if not self.capture:
            return
        try:
            self.prog.capture_launch_graphs(self.issues)
        except GraphCaptureError as exc:
            logger.warning("[hip] %s — continuing with uncaptured (dispatch-inclusive) timing", exc)
            self.capture = False

    def probe(self, passes: int) -> None:
        for _ in range(passes):
            self._pass()

    def settle(self) -> None:
        if self.last:
            target = min(_BATCH_TARGET_MS, _PASS_TARGET_MS / max(1, self.n))
            self.issues = [window_issues(dt, target) for dt in self.last]
        self._capture_windows()
        if not self.last:
            return  # no warm-up asked for: sample from the first pass on
        took = self._pass() if self.device_ms < _WARMUP_TARGET_MS else 0.0
        while took > 0.0 and self.device_ms < _WARMUP_TARGET_MS:
            took = self._pass()

    def sample(self, budget: SampleBudget) -> tuple[list[list[float]], list[float]]:
        per_launch: list[list[float]] = [[] for _ in range(self.n)]
        whole: list[float] = []
        whole_windows = self._whole_program_windows if self.n > 1 and self.capture else None
        measured_ms, count = 0.0, 0
        while not budget.spent(count, measured_ms):
            measured_ms += self._pass()
            count += 1
            for column, dt in zip(per_launch, self.last):
                column.append(dt)
            if whole_windows is not None:
                dt = whole_windows()
                if dt is None:
                    whole_windows = None
                else:
                    whole.append(dt)
        return per_launch, whole

    _whole_replays = 0

    def _whole_program_windows(self) -> float | None:
        """ms per run of the whole program from one window of graph launches; the graph (up to
        ``_E2E_MAX_COPIES`` copies of the program, so the window holds device time only) is built on first use."""
        prog = self.prog
        if self._whole_replays == 0:
            self._whole_replays = window_issues(sum(self.last))
            try:
                prog.capture_program_graph(repeat=min(self._whole_replays, _E2E_MAX_COPIES))
            except GraphCaptureError as exc:
                logger.warning("[hip] %s — skipping whole-program e2e timing", exc)
                return None
        copies = prog._program_graph_repeat
        launches = max(1, -(-self._whole_replays // copies))
        dt = prog.time_program_window(launches)
        self._charge(dt * launches * copies)
        return dt


def _samples_to_result(samples: list[list[float]], launches: list[_Launch], *, captured: bool, e2e_samples: list[float]) -> BenchmarkResult:
    per_launch = []
    for i, ln in enumerate(launches):
        s = samples[i]
        per_launch.append(LaunchTime(idx=i, kernel_name=ln.kernel_name, time_ms=statistics.median(s) if s else 0.0, samples=tuple(s)))
    total = sum(p.time_ms for p in per_launch)
    mins = sum(min(samples[i]) for i in range(len(launches)) if samples[i])
    maxs = sum(max(samples[i]) for i in range(len(launches)) if samples[i])
    return BenchmarkResult(
        time_ms=total,
        min_ms=mins,
        max_ms=maxs,
        num_launches=len(launches),
        per_launch=per_launch,
        captured=captured,
        e2e_ms=statistics.median(e2e_samples) if e2e_samples else None,
        e2e_min_ms=min(e2e_samples) if e2e_samples else None,
    )


def benchmark_program(
    graph: Graph,
    input_data: dict | None = None,
    warmup: int = 5,
    num_iters=20,
    on_iter=None,
    compile_timeout_s: float | None = None,
    run_timeout_s: float | None = None,
    capture_graphs: bool = True,
) -> BenchmarkResult:
    """Time the program's launches with device events (the contract of the reference's
    ``benchmark_program``, program.py:1152-1325: ``BenchmarkResult`` with per-launch medians and samples,
    ``captured``, whole-program ``e2e_ms`` for a multi-launch program).

    Three phases (``_BenchSession``): ``warmup`` probe passes of single issues; then each launch's event window
    is sized to about ``_BATCH_TARGET_MS`` of back-to-back issues, captured into a graph when ``capture_graphs``
    holds, and passes go on until ``_WARMUP_TARGET_MS`` of device time has run; then ``num_iters`` measured passes
    (``"auto"``: until ``_AUTO_BUDGET_MS`` of measured device time).  A multi-launch program also gets
    whole-program graph windows per measured pass.  Budgets: the per-window watchdog (``HungKernelError``),
    ``run_timeout_s`` of accumulated device time, and zero-elapsed windows raise ``RuntimeError`` (bench_fail)."""
    budget = SampleBudget.parse(num_iters)
    with gpu_lock():
        prog = CompiledProgram.build(graph, input_data, compile_timeout_s=compile_timeout_s)
        try:
            session = _BenchSession(prog, on_iter=on_iter, run_timeout_s=run_timeout_s, capture=capture_graphs)
            session.probe(max(0, int(warmup)))
            session.settle()
            per_launch, whole = session.sample(budget)
            return _samples_to_result(per_launch, prog.compiled.launches, captured=session.capture, e2e_samples=whole)
        finally:
            prog.close()
