"""Content-addressed code-object cache over hipRTC.

Role of the reference's ``nvcc.py`` (emmy/compiler/backend/cuda/nvcc.py:105-177):
``compile_to_hsaco`` is GPU-free and idempotent (compile to a temp file, then
an atomic ``os.replace``), keyed by sha1(source, name, arch, toolchain, flags);
``load_function`` makes sure the code object exists, then loads it on the
current device and returns the function handle.
"""

from __future__ import annotations

import functools
import hashlib
import os
import re
import shutil
import tempfile
from pathlib import Path

from deplodock_amd import config
from deplodock_amd.backend.hip import launcher

# Always-on options.  -ffp-contract=fast is clang's HIP default (fma contraction);
# fast-math is NOT enabled: fp32 kernels must match eager to rtol 1e-5.  The
# packed-fp32 feature is switched off because some packed forms have produced
# wrong results on this hardware generation.
_BASE_FLAGS = ["-O3", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def effective_flags() -> list[str]:
    """Base flags + ``EMMY_HIPRTC_FLAGS`` (read live; folded into the cache key)."""
    return [*_BASE_FLAGS, *config.hiprtc_flags().split()]


def cache_dir() -> Path:
    return config.hsaco_cache_dir()


def clear_cache() -> None:
    shutil.rmtree(cache_dir(), ignore_errors=True)


@functools.cache
def _toolkit_tag() -> str:
    """Digest of the ROCm toolchain identity so an upgrade never reuses old code objects."""
    ver = "?"
    for cand in ("/opt/rocm/.info/version", "/opt/rocm/.info/version-dev"):
        try:
            ver = Path(cand).read_text().strip()
            break
        except OSError:
            continue
    return hashlib.sha1(ver.encode()).hexdigest()[:12]


def cache_key(source: str, name: str, arch: str) -> str:
    h = hashlib.sha1()
    for part in (source, name, arch, _toolkit_tag(), "\x1f".join(effective_flags())):
        h.update(part.encode())
        h.update(b"\0")
    return h.hexdigest()


# A kernel that defines this macro waits for part of its outstanding direct-to-LDS loads by count
# (the contraction's slab ring): it must compile without vector-register spills, because spill
# stores share the counter and complete out of order with loads.
NO_SPILL_CONTRACT = "#define EMH_SLAB_SYNC(n)"


def vgpr_spill_counts(code_object: bytes) -> list[int]:
    """``.vgpr_spill_count`` of every kernel in a code object, read from the msgpack metadata note
    (key string followed by a msgpack unsigned integer)."""
    key = b".vgpr_spill_count"
    out, pos = [], code_object.find(key)
    while pos >= 0:
        v = code_object[pos + len(key) : pos + len(key) + 5]
        if v[:1] and v[0] <= 0x7F:
            out.append(v[0])
        elif v[:1] == b"\xcc":
            out.append(v[1])
        elif v[:1] == b"\xcd":
            out.append(int.from_bytes(v[1:3], "big"))
        elif v[:1] == b"\xce":
            out.append(int.from_bytes(v[1:5], "big"))
        pos = code_object.find(key, pos + 1)
    return out


def compile_to_hsaco(source: str, name: str, *, arch: str = "gfx950") -> Path:
    """Compile ``source`` into the cache and return the code-object path.

    Raises :class:`launcher.CompileError` on a compiler error."""
    cache = cache_dir()
    cache.mkdir(parents=True, exist_ok=True)
    out = cache / f"{cache_key(source, name, arch)}.hsaco"
    if out.exists() and out.stat().st_size > 0:
        return out
    blob, _log = launcher.load().compile(source, name, arch, effective_flags())
    if NO_SPILL_CONTRACT in source:
        spilled = max(vgpr_spill_counts(blob), default=0)
        if spilled:
            raise launcher.CompileError(
                f"{name}: the compiler spilled {spilled} vector registers, and this kernel waits for part of its outstanding "
                "direct-to-LDS loads by count (spill stores complete out of order with loads and would satisfy the wait early): "
                "pick a smaller tile or register staging",
                0,
                _log or "",
            )
    fd, tmp = tempfile.mkstemp(dir=cache, suffix=".tmp")
    try:
        with os.fdopen(fd, "wb") as fh:
            fh.write(blob)
        os.replace(tmp, out)  # atomic publish
    except BaseException:
        Path(tmp).unlink(missing_ok=True)
        raise
    return out


def spilled_vgprs(source: str, name: str, *, arch: str = "gfx950") -> int:
    """Vector registers the compiler spills building ``source``.  The code object is cached as by
    ``compile_to_hsaco`` (so the loader compiles nothing twice), except a spilling kernel under the
    no-spill contract, which is never cached."""
    try:
        return max(vgpr_spill_counts(compile_to_hsaco(source, name, arch=arch).read_bytes()), default=0)
    except launcher.CompileError as exc:
        found = re.search(r"spilled (\d+) vector registers", str(exc))
        if found is None:
            raise
        return int(found.group(1))


class LoadedKernel:
    """A launchable function plus the module that owns it."""

    __slots__ = ("name", "module", "fn", "path")

    def __init__(self, name: str, module: int, fn: int, path: Path):
        self.name, self.module, self.fn, self.path = name, module, fn, path


# (device, code-object file name, kernel name) -> the loaded kernel.  A code object is loaded onto a
# device once per process and stays loaded: programs come and go (benchmark sweeps build hundreds, a
# serving loop one per sequence length) and share the modules, whose number is bounded by the number of
# distinct kernels, not by the number of programs.
_loaded: dict[tuple[int, str, str], LoadedKernel] = {}


def _current_device() -> int:
    import torch

    return torch.cuda.current_device() if torch.cuda.is_available() else -1


def load_function(source: str, name: str, *, arch: str = "gfx950", cached: bool = True) -> LoadedKernel:
    """Compile (cached on disk) and load ``name`` on the current device.  With ``cached`` (the default)
    the module is shared by every caller in the process and must not be unloaded by them; with
    ``cached=False`` the caller owns the module and unloads it (one-off probe kernels)."""
    path = compile_to_hsaco(source, name, arch=arch)
    lib = launcher.load()
    key = (_current_device(), path.name, name)
    if cached and key in _loaded:
        return _loaded[key]
    module = lib.module_load(path.read_bytes())
    try:
        fn = lib.get_function(module, name)
    except launcher.LauncherError:
        lib.module_unload(module)
        raise
    kernel = LoadedKernel(name, module, fn, path)
    if cached:
        _loaded[key] = kernel
    return kernel


def unload_all() -> int:
    """Unload every cached module (process teardown, or tests that count modules); returns how many."""
    lib = launcher.load()
    n = 0
    for kernel in list(_loaded.values()):
        lib.module_unload(kernel.module)
        n += 1
    _loaded.clear()
    return n


def loaded_module_count() -> int:
    return len(_loaded)
