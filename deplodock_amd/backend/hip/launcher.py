"""ctypes binding of ``libemmy_hip.so`` — the only door to the device.

Every entry point of ``include/emmy_hip.h`` is bound here with its exact
signature.  There is no fallback: when the library is missing or a call
fails, a :class:`LauncherError` is raised with the library's own message.
Stands where cupy's driver bindings stand in the reference
(emmy/compiler/backend/cuda/nvcc.py:177, backend/cuda/program.py:394-424).
"""

from __future__ import annotations

import ctypes as C
import threading
from pathlib import Path

from deplodock_amd import config

EMH_RTC_ERROR_BASE = 100000
EMH_ABI_VERSION = 1
EMH_SCRATCH_MAX_BYTES = 16 * 1024 * 1024  # include/emmy_hip.h

# name -> (restype, argtypes); mirrors include/emmy_hip.h declaration by declaration.
_U3 = C.c_uint * 3
SIGNATURES: dict[str, tuple] = {
    "emh_abi_version": (C.c_int, []),
    "emh_device_count": (C.c_int, [C.POINTER(C.c_int)]),
    "emh_device_props": (
        C.c_int,
        [C.c_int, C.c_char_p, C.c_size_t, C.POINTER(C.c_int), C.POINTER(C.c_int), C.POINTER(C.c_int), C.POINTER(C.c_int), C.POINTER(C.c_size_t)],
    ),
    "emh_compile": (
        C.c_int,
        [C.c_char_p, C.c_char_p, C.c_char_p, C.POINTER(C.c_char_p), C.c_int, C.POINTER(C.c_void_p), C.POINTER(C.c_size_t), C.POINTER(C.c_void_p)],
    ),
    "emh_free": (None, [C.c_void_p]),
    "emh_module_load": (C.c_int, [C.c_void_p, C.c_size_t, C.POINTER(C.c_void_p)]),
    "emh_module_unload": (C.c_int, [C.c_void_p]),
    "emh_get_function": (C.c_int, [C.c_void_p, C.c_char_p, C.POINTER(C.c_void_p)]),
    "emh_func_set_dynamic_lds": (C.c_int, [C.c_void_p, C.c_int]),
    "emh_func_attributes": (C.c_int, [C.c_void_p, C.POINTER(C.c_int), C.POINTER(C.c_int), C.POINTER(C.c_int), C.POINTER(C.c_int)]),
    "emh_launch": (C.c_int, [C.c_void_p, _U3, _U3, C.c_uint, C.c_void_p, C.POINTER(C.c_void_p), C.c_int]),
    "emh_launch_scratch": (C.c_int, [C.c_void_p, _U3, _U3, C.c_uint, C.c_void_p, C.POINTER(C.c_void_p), C.c_int, C.c_int, C.c_size_t, C.c_size_t, C.c_int]),
    "emh_memset_async": (C.c_int, [C.c_void_p, C.c_int, C.c_size_t, C.c_void_p]),
    "emh_stream_create": (C.c_int, [C.POINTER(C.c_void_p)]),
    "emh_stream_destroy": (C.c_int, [C.c_void_p]),
    "emh_stream_synchronize": (C.c_int, [C.c_void_p]),
    "emh_event_create": (C.c_int, [C.POINTER(C.c_void_p)]),
    "emh_event_record": (C.c_int, [C.c_void_p, C.c_void_p]),
    "emh_event_synchronize": (C.c_int, [C.c_void_p]),
    "emh_event_query": (C.c_int, [C.c_void_p, C.POINTER(C.c_int)]),
    "emh_event_elapsed_ms": (C.c_int, [C.c_void_p, C.c_void_p, C.POINTER(C.c_float)]),
    "emh_event_destroy": (C.c_int, [C.c_void_p]),
    "emh_graph_begin_capture": (C.c_int, [C.c_void_p]),
    "emh_graph_end_capture": (C.c_int, [C.c_void_p, C.POINTER(C.c_void_p)]),
    "emh_graph_launch": (C.c_int, [C.c_void_p, C.c_void_p]),
    "emh_graph_destroy": (C.c_int, [C.c_void_p]),
    "emh_last_error": (C.c_char_p, []),
}


class LauncherError(RuntimeError):
    """A ``libemmy_hip.so`` call failed, or the library could not be loaded."""

    def __init__(self, message: str, code: int = -1):
        super().__init__(message)
        self.code = code


class CompileError(LauncherError):
    """hipRTC rejected the source; ``log`` holds the compiler output."""

    def __init__(self, message: str, code: int, log: str):
        super().__init__(message, code)
        self.log = log


class PackedArgs:
    """Kernel-parameter storage kept alive for the lifetime of a launch record.

    ``ptrs`` are device addresses, ``ints`` 32-bit runtime values, in signature
    order (pointers first).  ``array`` is the ``void**`` handed to emh_launch."""

    __slots__ = ("slots", "array", "n")

    def __init__(self, ptrs, ints=()):
        self.slots = [C.c_void_p(int(p)) for p in ptrs] + [C.c_int(int(v)) for v in ints]
        self.n = len(self.slots)
        self.array = (C.c_void_p * max(self.n, 1))(*[C.cast(C.pointer(s), C.c_void_p) for s in self.slots])

    def set_ptr(self, i: int, p: int) -> None:
        self.slots[i].value = int(p)

    def set_int(self, i: int, v: int) -> None:
        self.slots[i].value = int(v)


class Launcher:
    """Typed Python face of one loaded ``libemmy_hip.so``."""

    def __init__(self, path: Path):
        self.path = Path(path)
        if not self.path.exists():
            raise LauncherError(
                f"{self.path} not found: build it first (python -c 'import __graft_entry__ as g; g.build()' "
                f"or make -C deplodock_amd/csrc). There is no fallback path."
            )
        try:
            self._dll = C.CDLL(str(self.path))
        except OSError as exc:
            raise LauncherError(f"cannot load {self.path}: {exc}") from exc
        for name, (res, args) in SIGNATURES.items():
            try:
                fn = getattr(self._dll, name)
            except AttributeError as exc:
                raise LauncherError(f"{self.path} does not export {name}") from exc
            fn.restype = res
            fn.argtypes = args
        got = self._dll.emh_abi_version()
        if got != EMH_ABI_VERSION:
            raise LauncherError(f"{self.path}: ABI version {got}, expected {EMH_ABI_VERSION}")

    # -- error plumbing -----------------------------------------------------
    def last_error(self) -> str:
        msg = self._dll.emh_last_error()
        return msg.decode(errors="replace") if msg else ""

    def _check(self, rc: int, what: str) -> None:
        if rc != 0:
            raise LauncherError(f"{what} failed ({rc}): {self.last_error()}", rc)

    # -- discovery ------------------------------------------------------------
    def device_count(self) -> int:
        n = C.c_int(0)
        self._check(self._dll.emh_device_count(C.byref(n)), "emh_device_count")
        return n.value

    def device_props(self, device: int = 0) -> dict:
        arch = C.create_string_buffer(256)
        cu, lds, wave, clk = C.c_int(), C.c_int(), C.c_int(), C.c_int()
        mem = C.c_size_t()
        self._check(
            self._dll.emh_device_props(device, arch, 256, C.byref(cu), C.byref(lds), C.byref(wave), C.byref(clk), C.byref(mem)),
            "emh_device_props",
        )
        return {
            "arch": arch.value.decode(),
            "compute_units": cu.value,
            "lds_bytes_per_block": lds.value,
            "wavefront_size": wave.value,
            "clock_khz": clk.value,
            "global_mem_bytes": mem.value,
        }

    # -- compile --------------------------------------------------------------
    def compile(self, source: str, name: str, arch: str, options: list[str]) -> tuple[bytes, str]:
        """hipRTC-compile ``source``; returns ``(code_object, log)``."""
        opts = (C.c_char_p * max(len(options), 1))(*[o.encode() for o in options])
        code = C.c_void_p()
        size = C.c_size_t()
        log = C.c_void_p()
        rc = self._dll.emh_compile(source.encode(), name.encode(), arch.encode(), opts, len(options), C.byref(code), C.byref(size), C.byref(log))
        log_text = ""
        if log.value:
            log_text = C.string_at(log.value).decode(errors="replace")
            self._dll.emh_free(log)
        if rc != 0:
            raise CompileError(f"hipRTC compile of {name!r} failed ({rc}): {self.last_error()}", rc, log_text)
        try:
            blob = C.string_at(code.value, size.value)
        finally:
            self._dll.emh_free(code)
        return blob, log_text

    # -- modules / functions --------------------------------------------------
    def module_load(self, blob: bytes) -> int:
        mod = C.c_void_p()
        buf = C.create_string_buffer(blob, len(blob))
        self._check(self._dll.emh_module_load(C.cast(buf, C.c_void_p), len(blob), C.byref(mod)), "emh_module_load")
        return mod.value

    def module_unload(self, module: int) -> None:
        self._check(self._dll.emh_module_unload(module), "emh_module_unload")

    def get_function(self, module: int, name: str) -> int:
        fn = C.c_void_p()
        self._check(self._dll.emh_get_function(module, name.encode(), C.byref(fn)), f"emh_get_function({name})")
        return fn.value

    def func_set_dynamic_lds(self, fn: int, nbytes: int) -> None:
        self._check(self._dll.emh_func_set_dynamic_lds(fn, nbytes), "emh_func_set_dynamic_lds")

    def func_attributes(self, fn: int) -> dict:
        regs, lds, priv, thr = C.c_int(), C.c_int(), C.c_int(), C.c_int()
        self._check(self._dll.emh_func_attributes(fn, C.byref(regs), C.byref(lds), C.byref(priv), C.byref(thr)), "emh_func_attributes")
        return {"num_regs": regs.value, "static_lds_bytes": lds.value, "private_bytes": priv.value, "max_threads": thr.value}

    # -- launch -----------------------------------------------------------------
    def launch(self, fn: int, grid, block, lds_bytes: int, stream: int | None, args: PackedArgs) -> None:
        rc = self._dll.emh_launch(fn, _U3(*grid), _U3(*block), lds_bytes, stream, args.array, args.n)
        if rc != 0:
            raise LauncherError(f"emh_launch failed ({rc}): {self.last_error()}", rc)

    def launch_scratch(self, fn: int, grid, block, lds_bytes: int, stream: int | None, args: PackedArgs, scratch_arg: int, scratch_offset: int, scratch_bytes: int, zero_first: bool) -> None:
        """``launch`` with parameter ``scratch_arg`` pointed at the library's own device scratch array (no allocation anywhere)."""
        rc = self._dll.emh_launch_scratch(fn, _U3(*grid), _U3(*block), lds_bytes, stream, args.array, args.n, scratch_arg, scratch_offset, scratch_bytes, int(zero_first))
        if rc != 0:
            raise LauncherError(f"emh_launch_scratch failed ({rc}): {self.last_error()}", rc)

    def memset_async(self, dptr: int, value: int, nbytes: int, stream: int | None) -> None:
        self._check(self._dll.emh_memset_async(dptr, value, nbytes, stream), "emh_memset_async")

    # -- streams ------------------------------------------------------------------
    def stream_create(self) -> int:
        s = C.c_void_p()
        self._check(self._dll.emh_stream_create(C.byref(s)), "emh_stream_create")
        return s.value

    def stream_destroy(self, stream: int) -> None:
        self._check(self._dll.emh_stream_destroy(stream), "emh_stream_destroy")

    def stream_synchronize(self, stream: int | None) -> None:
        self._check(self._dll.emh_stream_synchronize(stream), "emh_stream_synchronize")

    # -- events ---------------------------------------------------------------------
    def event_create(self) -> int:
        e = C.c_void_p()
        self._check(self._dll.emh_event_create(C.byref(e)), "emh_event_create")
        return e.value

    def event_record(self, event: int, stream: int | None) -> None:
        self._check(self._dll.emh_event_record(event, stream), "emh_event_record")

    def event_synchronize(self, event: int) -> None:
        self._check(self._dll.emh_event_synchronize(event), "emh_event_synchronize")

    def event_query(self, event: int) -> bool:
        done = C.c_int()
        self._check(self._dll.emh_event_query(event, C.byref(done)), "emh_event_query")
        return bool(done.value)

    def event_elapsed_ms(self, start: int, stop: int) -> float:
        ms = C.c_float()
        self._check(self._dll.emh_event_elapsed_ms(start, stop, C.byref(ms)), "emh_event_elapsed_ms")
        return float(ms.value)

    def event_destroy(self, event: int) -> None:
        self._check(self._dll.emh_event_destroy(event), "emh_event_destroy")

    # -- graphs -----------------------------------------------------------------------
    def graph_begin_capture(self, stream: int) -> None:
        self._check(self._dll.emh_graph_begin_capture(stream), "emh_graph_begin_capture")

    def graph_end_capture(self, stream: int) -> int:
        g = C.c_void_p()
        self._check(self._dll.emh_graph_end_capture(stream, C.byref(g)), "emh_graph_end_capture")
        return g.value

    def graph_launch(self, graph_exec: int, stream: int | None) -> None:
        self._check(self._dll.emh_graph_launch(graph_exec, stream), "emh_graph_launch")

    def graph_destroy(self, graph_exec: int) -> None:
        self._check(self._dll.emh_graph_destroy(graph_exec), "emh_graph_destroy")


_lock = threading.Lock()
_loaded: dict[Path, Launcher] = {}


def load(path: Path | None = None) -> Launcher:
    """The process-wide :class:`Launcher` for ``path`` (default: the in-tree build)."""
    p = Path(path) if path is not None else config.lib_path()
    with _lock:
        if p not in _loaded:
            _loaded[p] = Launcher(p)
        return _loaded[p]
