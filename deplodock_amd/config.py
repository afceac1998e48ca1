"""``EMMY_*`` environment handling — one place for every spelling.

Mirrors the reference's env conventions (emmy/config.py:34-50, 130-145) so
knob pins and cache locations keep their names: getters read ``os.environ``
live on every call (tests monkeypatch it), nothing is cached at import.
The nvcc-specific names gain HIP twins: ``EMMY_HIPRTC_FLAGS`` (extra compiler
options, folded into the cache key) and ``EMMY_HSACO_CACHE`` (code-object
cache directory).
"""

from __future__ import annotations

import os
from contextlib import contextmanager
from pathlib import Path

PREFIX = "EMMY_"
HIPRTC_FLAGS = "EMMY_HIPRTC_FLAGS"
HSACO_CACHE = "EMMY_HSACO_CACHE"
DEBUG = "EMMY_DEBUG"
DUMP_DIR = "EMMY_DUMP_DIR"
KNOBS = "EMMY_KNOBS"
GPU_LOCK = "EMMY_GPU_LOCK"
TUNE_DB = "EMMY_TUNE_DB"
LIB = "EMMY_HIP_LIB"

_CACHE_ROOT = Path.home() / ".cache" / "emmy"
_TRUTHY = {"1", "true", "yes", "on"}


def knob_var(name: str) -> str:
    """``EMMY_<NAME>`` for a knob called ``name`` (emmy/config.py knob_var)."""
    return f"{PREFIX}{name.upper()}"


def knobs_aggregate() -> dict[str, str]:
    """Decode ``EMMY_KNOBS="K=V,K2=V2"`` into a dict (keys upper-cased)."""
    raw = os.environ.get(KNOBS, "")
    out: dict[str, str] = {}
    for part in raw.split(","):
        part = part.strip()
        if not part:
            continue
        if "=" not in part:
            raise ValueError(f"{KNOBS}: expected K=V, got {part!r}")
        k, v = part.split("=", 1)
        out[k.strip().upper()] = v.strip()
    return out


def knob_raw(name: str) -> str | None:
    """The pinned value of knob ``name``: ``EMMY_<NAME>`` wins over the
    ``EMMY_KNOBS`` aggregate; ``None`` when neither pins it."""
    direct = os.environ.get(knob_var(name))
    if direct is not None:
        return direct
    return knobs_aggregate().get(name.upper())


def _bool(name: str, default: bool = False) -> bool:
    raw = os.environ.get(name)
    if raw is None:
        return default
    return raw.strip().lower() in _TRUTHY


def debug_enabled() -> bool:
    return _bool(DEBUG)


def dump_dir() -> Path | None:
    raw = os.environ.get(DUMP_DIR)
    return Path(raw) if raw else None


def hiprtc_flags() -> str:
    """Extra hipRTC options (space separated) from ``EMMY_HIPRTC_FLAGS``."""
    return os.environ.get(HIPRTC_FLAGS, "")


@contextmanager
def hiprtc_flags_override(flags: str | None):
    """Temporarily re-point ``EMMY_HIPRTC_FLAGS`` (``None`` = leave as is)."""
    if flags is None:
        yield
        return
    old = os.environ.get(HIPRTC_FLAGS)
    os.environ[HIPRTC_FLAGS] = flags
    try:
        yield
    finally:
        if old is None:
            os.environ.pop(HIPRTC_FLAGS, None)
        else:
            os.environ[HIPRTC_FLAGS] = old


def hsaco_cache_dir() -> Path:
    """Content-addressed code-object cache directory.

    ``EMMY_HSACO_CACHE`` wins; otherwise the in-tree ``deplodock_amd/_kcache``
    when it is writable (so code objects compiled ahead of time travel with the
    source tree), else ``~/.cache/emmy/hsaco``."""
    override = os.environ.get(HSACO_CACHE)
    if override:
        return Path(override)
    in_tree = Path(__file__).resolve().parent / "_kcache"
    try:
        in_tree.mkdir(parents=True, exist_ok=True)
        if os.access(in_tree, os.W_OK):
            return in_tree
    except OSError:
        pass
    return _CACHE_ROOT / "hsaco"


def gpu_lock_path() -> Path:
    override = os.environ.get(GPU_LOCK)
    return Path(override) if override else Path("/tmp/emmy_gpu.lock")


def tune_db_path() -> Path:
    override = os.environ.get(TUNE_DB)
    return Path(override) if override else _CACHE_ROOT / "autotune_gfx950.db"


def lib_path() -> Path:
    """Location of ``libemmy_hip.so`` (``EMMY_HIP_LIB`` overrides the in-tree build)."""
    override = os.environ.get(LIB)
    if override:
        return Path(override)
    return Path(__file__).resolve().parent / "lib" / "libemmy_hip.so"
