"""HIP backend: ``Graph`` → lowered ``Graph[HipOp]`` → hipRTC → MI355X.

Same call surface as the reference's ``CudaBackend``
(emmy/compiler/backend/cuda/backend.py:59-237): the compiled artifact is the
lowered graph itself; ``run`` returns host arrays; ``benchmark_async`` is the
single benchmarking entry point.  Differences that follow from the platform:
constants traced from a module are bound automatically from the traced
parameter values unless ``input_data`` overrides them, and tensors may be
passed as device ``torch.Tensor`` objects, in which case they are used in place.
"""

from __future__ import annotations

from collections import OrderedDict

from deplodock_amd import config
from deplodock_amd.backend import Backend, BenchmarkResult, RunResult
from deplodock_amd.context import Context
from deplodock_amd.graph import Graph
from deplodock_amd.pipeline import HIP_PASSES, Pipeline


class HipBackend(Backend):
    name = "hip"

    def __init__(
        self,
        *,
        debug: bool | None = None,
        dump=None,
        bench_wall_timeout_s: float | None = None,
        bench_compile_timeout_s: float = 30.0,
        bench_run_timeout_s: float = 10.0,
        tune_db=None,
        device_id: int | None = None,
        context: Context | None = None,
    ) -> None:
        self.debug = config.debug_enabled() if debug is None else debug
        #: what the last ``run`` under ``debug`` kept: per-launch host copies of every scratch / output buffer
        #: (``DebugResult``); ``None`` after a plain run (emmy/compiler/backend/cuda/backend.py:158-161)
        self.last_debug_result = None
        self.dump = dump
        self.bench_wall_timeout_s = bench_wall_timeout_s
        self._worker = None
        if bench_wall_timeout_s is not None:
            # Benchmarks will run in a killable child forked from a clean server process: start that server
            # now, while this process (if the backend is built first, as the tuner does) has not touched the GPU.
            from deplodock_amd.backend.hip.bench_worker import start_server

            start_server()
        self.bench_compile_timeout_s = bench_compile_timeout_s
        self.bench_run_timeout_s = bench_run_timeout_s
        self.device_id = device_id
        self.context = context or Context()
        # ``tune_db``: None = heuristics only; "auto" = the per-user database; a path; or an open TuneDB.
        if tune_db is not None:
            from dataclasses import replace

            from deplodock_amd.tune import TuneDB

            tune_db = tune_db if isinstance(tune_db, TuneDB) else TuneDB(tune_db, arch=self.context.arch)
            self.context = replace(self.context, tune_db=tune_db)
        self.tune_db = tune_db

    # -- compile ------------------------------------------------------------
    def compile(self, graph: Graph) -> Graph:
        """Lower ``Graph`` → ``Graph[TileOp]`` → ``Graph[HipOp]`` (needs no GPU).

        A graph traced with ``dynamic_shapes`` is lowered at its example sizes; the
        result remembers how to re-trace (``compiled.dynamic``) and ``run`` /
        ``program`` / ``benchmark`` pick — building on first use — the variant that
        matches the shapes of the inputs they are given."""
        spec = getattr(graph, "dynamic", None)
        if spec is not None and len(spec.hints) == 1 and self.symbolic_kernels:
            symbolic = self._compile_symbolic(graph, spec)
            if symbolic is not None:
                return symbolic
        compiled = Pipeline.build(HIP_PASSES, self.context).run(graph, dump_dir=self.dump)
        if spec is not None:
            compiled.dynamic = spec
            compiled.variants = OrderedDict({tuple(sorted(spec.hints.items())): compiled})
        return compiled

    #: lower a graph with one symbolic axis to kernels that take its extent as a runtime ``int`` (one code object per
    #: kernel for every size); False: always specialise per size
    symbolic_kernels = True

    def _compile_symbolic(self, graph: Graph, spec) -> Graph | None:
        """One lowering for every size of the symbolic axis: the module is fused at the traced size and at two
        others, what changes must be affine in the size and must be something a kernel can take at run time
        (``passes.symbolic``); the kernels are then scheduled at the traced size and emitted with a trailing
        ``int`` parameter, run-time guards and launch-time grid factors.  ``None`` when the module does not
        symbolise (the caller then lowers per size)."""
        import logging

        from deplodock_amd.emit.errors import LoweringError
        from deplodock_amd.ir.sym import Affine
        from deplodock_amd.passes.fuse import FusionError, fuse
        from deplodock_amd.passes.symbolic import SymbolicError, symbolize

        (name, s0), = spec.hints.items()
        sizes = [s0, s0 + 7, s0 + 96]
        try:
            tiles = [fuse(graph)] + [fuse(spec.retrace({name: s})) for s in sizes[1:]]
            base = symbolize(tiles, name, sizes)
            compiled = base
            for _pass_name, fn in HIP_PASSES[1:]:
                compiled = fn(compiled, self.context)
        except (SymbolicError, FusionError, LoweringError) as exc:
            logging.getLogger(__name__).info("[hip] %s does not lower to runtime-int kernels (%s): specialising per size", name, exc)
            return None
        for node in compiled.nodes.values():
            sym_shape = node.hints.get("sym_shape")
            if sym_shape is not None:
                # a dim that is the bare symbol is spelled by its name (how the runtime binds it to an input's shape)
                node.output.shape = tuple(d.name if isinstance(d, Affine) and (d.a, d.b) == (1, 0) else d for d in sym_shape)
        compiled.dynamic = spec
        compiled.symbolic = name
        return compiled

    #: distinct size combinations kept per dynamically shaped graph
    VARIANT_CACHE = 8

    def variant(self, compiled: Graph, input_data: dict | None) -> Graph:
        """The lowering of ``compiled``'s module at the sizes ``input_data`` has."""
        spec = getattr(compiled, "dynamic", None)
        if spec is None or not input_data or getattr(compiled, "symbolic", None) is not None:
            return compiled  # static, or one lowering that takes the size at run time
        shapes = []
        for nid, axes in zip(compiled.inputs, spec.input_axes):
            if nid not in input_data:
                if axes:
                    return compiled  # benchmark-style call with synthetic inputs: the traced sizes
                shapes.append(compiled.nodes[nid].output.shape)
                continue
            shapes.append(tuple(input_data[nid].shape))
        env = spec.env_of(shapes)
        key = tuple(sorted(env.items()))
        cache = compiled.variants
        if key in cache:
            cache.move_to_end(key)
            return cache[key]
        g = Pipeline.build(HIP_PASSES, self.context).run(spec.retrace(env), dump_dir=self.dump)
        if g.inputs != compiled.inputs or g.outputs != compiled.outputs:
            raise ValueError("re-tracing at another size changed the graph's inputs or outputs")
        g.dynamic, g.variants = spec, cache
        cache[key] = g
        while len(cache) > self.VARIANT_CACHE:
            cache.popitem(last=False)
        return g

    # -- binding ------------------------------------------------------------
    @staticmethod
    def _bind_prefix_tables(compiled: Graph, data: dict, traced: dict) -> None:
        """Constants of a runtime-int lowering whose rows follow the symbolic axis (position tables computed when the
        module was traced; ``passes.symbolic._prefix_table``): bind the leading rows the inputs' size needs.  A size
        beyond the largest table held re-traces the module once at (at least) twice that size and keeps the larger
        tables for every later call."""
        tables = [(nid, n.hints["prefix_table"], n.hints["sym_shape"]) for nid, n in compiled.nodes.items() if "prefix_table" in n.hints and nid not in data and nid in traced]
        if not tables:
            return
        spec, name = compiled.dynamic, compiled.symbolic
        size = None
        for nid, axes in zip(compiled.inputs, spec.input_axes):
            for dim, sym in (axes or {}).items():
                if sym == name and nid in data:
                    size = int(data[nid].shape[dim])
        if size is None:
            size = int(spec.hints[name])  # synthetic inputs: the traced size
        if any(traced[nid].shape[d] < shape[d].at({name: size}) for nid, d, shape in tables):
            from deplodock_amd.passes.fuse import fuse

            if not hasattr(spec, "retrace"):
                raise ValueError(f"{name} = {size} needs more rows of {[t[0] for t in tables]} than the graph holds and the module is not here to re-trace: pass the tables in input_data")
            held = max(int(spec.hints[name]), getattr(compiled, "prefix_table_size", 0))
            grown = max(size, 2 * held)
            values = fuse(spec.retrace({name: grown})).constant_values
            for nid, _d, _shape in tables:
                traced[nid] = values[nid]
            compiled.prefix_table_size = grown
        for nid, d, shape in tables:
            data[nid] = traced[nid].narrow(d, 0, shape[d].at({name: size})).contiguous()

    @staticmethod
    def bind(compiled: Graph, input_data: dict | None) -> dict:
        """``input_data`` completed with the traced parameter values of every
        constant it does not override (stacked constants are assembled here)."""
        from deplodock_amd.passes.fuse import StackedConstant

        data = dict(input_data or {})
        traced = getattr(compiled, "constant_values", {})
        if getattr(compiled, "symbolic", None) is not None:
            HipBackend._bind_prefix_tables(compiled, data, traced)
        for nid, _op in compiled.constant_ops():
            if nid in data:
                continue
            stacked = compiled.nodes[nid].hints.get("stacked")
            if isinstance(stacked, StackedConstant):
                import torch

                parts = [data[p] if p in data else traced[p] for p in stacked.parts]
                whole = torch.cat([p if isinstance(p, torch.Tensor) else torch.as_tensor(p) for p in parts], dim=0).contiguous()
                if stacked.k_scale is not None:
                    ks = data[stacked.k_scale] if stacked.k_scale in data else traced[stacked.k_scale]
                    ks = ks if isinstance(ks, torch.Tensor) else torch.as_tensor(ks)
                    whole = (whole.float() * ks.to(whole.device).float().reshape(1, -1)).to(whole.dtype)
                if stacked.transpose:
                    whole = whole.transpose(-1, -2).contiguous()
                if stacked.pad_rows_to > whole.shape[0]:
                    whole = torch.cat([whole, whole.new_zeros((stacked.pad_rows_to - whole.shape[0], *whole.shape[1:]))], dim=0)
                data[nid] = whole
            elif nid in traced:
                data[nid] = traced[nid]
        return data

    # -- run ------------------------------------------------------------------
    def run(self, compiled: Graph, *, input_data: dict | None = None, pre_run=None) -> tuple[RunResult, object]:
        from deplodock_amd.backend.hip.program import run_program, run_program_debug

        self._select_device()
        compiled = self.variant(compiled, input_data)
        if self.debug:
            # launch by launch with a device synchronisation and a host copy of every written buffer after each
            result, pre = run_program_debug(compiled, input_data=self.bind(compiled, input_data), pre_run=pre_run)
            self.last_debug_result = result
            result = RunResult(outputs=result.outputs, time_ms=None)
        else:
            self.last_debug_result = None
            result, pre = run_program(compiled, input_data=self.bind(compiled, input_data), pre_run=pre_run)
        outputs = {}
        for name, vals in result.outputs.items():
            outputs[name] = vals
            for alias, shape in compiled.nodes[name].hints.get("output_alias", []):
                outputs[alias] = vals.reshape(shape)
        return RunResult(outputs=outputs, time_ms=result.time_ms), pre

    def program(self, compiled: Graph, input_data: dict | None = None, *, library_scratch: bool = False):
        """A persistent :class:`CompiledProgram` bound to device buffers (for serving loops).  With
        ``library_scratch`` the program's intermediates live in the launcher library's own device scratch
        array (``emh_launch_scratch``): nothing is allocated for them, at the price of a size limit and of
        sharing that array with every other such program on the GPU."""
        from deplodock_amd.backend.hip.program import CompiledProgram

        self._select_device()
        compiled = self.variant(compiled, input_data)
        return CompiledProgram.build(compiled, self.bind(compiled, input_data), library_scratch=library_scratch)

    # -- benchmark --------------------------------------------------------------
    async def benchmark_async(
        self,
        compiled: Graph,
        *,
        warmup: int = 5,
        num_iters=20,
        on_iter=None,
        nvcc_flags: str | None = None,
        capture_graphs: bool = True,
        input_data: dict | None = None,
    ) -> BenchmarkResult:
        """Event-timed benchmark (backend.py:179-237).  ``nvcc_flags`` keeps the
        reference's keyword; here it re-points ``EMMY_HIPRTC_FLAGS`` for this one
        compile.  With ``bench_wall_timeout_s`` set and no ``on_iter`` callback the
        benchmark runs in an isolated worker process that is killed at the limit
        (``RuntimeError``, the caller's bench_fail); otherwise in this process.

        The worker path waits for the worker's answer on a helper thread, so the event
        loop keeps running other tasks while the benchmark is under way (the reference
        awaits its subprocess, backend/cuda/program.py:1382-1533).  The in-process path
        issues device work from the calling thread — torch's current device and stream
        are per thread — and blocks for its (bounded) duration."""
        kwargs = dict(warmup=warmup, num_iters=num_iters, on_iter=on_iter, hiprtc_flags=nvcc_flags, capture_graphs=capture_graphs, input_data=input_data)
        if self.bench_wall_timeout_s is not None and on_iter is None:
            import asyncio
            import functools

            return await asyncio.get_running_loop().run_in_executor(None, functools.partial(self.benchmark, compiled, **kwargs))
        return self.benchmark(compiled, **kwargs)

    def benchmark(self, compiled: Graph, *, warmup: int = 5, num_iters=20, on_iter=None, hiprtc_flags: str | None = None, capture_graphs: bool = True, input_data: dict | None = None) -> BenchmarkResult:
        from deplodock_amd.backend.hip.program import benchmark_program

        self._select_device()
        compiled = self.variant(compiled, input_data)
        if self.bench_wall_timeout_s is not None and on_iter is None:
            from deplodock_amd.backend.hip.bench_worker import BenchWorker, benchmark_program_isolated

            if self._worker is None:
                self._worker = BenchWorker(device_id=self.device_id)
            return benchmark_program_isolated(
                compiled,
                worker=self._worker,
                wall_timeout_s=self.bench_wall_timeout_s,
                input_data=self.bind(compiled, input_data),
                hiprtc_flags=hiprtc_flags,
                warmup=warmup,
                num_iters=num_iters,
                compile_timeout_s=self.bench_compile_timeout_s,
                run_timeout_s=self.bench_run_timeout_s,
                capture_graphs=capture_graphs,
            )
        with config.hiprtc_flags_override(hiprtc_flags):
            return benchmark_program(
                compiled,
                input_data=self.bind(compiled, input_data),
                warmup=warmup,
                num_iters=num_iters,
                on_iter=on_iter,
                compile_timeout_s=self.bench_compile_timeout_s,
                run_timeout_s=self.bench_run_timeout_s,
                capture_graphs=capture_graphs,
            )

    def close(self) -> None:
        """End the benchmark worker process, if one was started."""
        if self._worker is not None:
            self._worker.close()
            self._worker = None

    def _select_device(self) -> None:
        if self.device_id is not None:
            import torch

            torch.cuda.set_device(self.device_id)
