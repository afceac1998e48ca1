"""Knob tuner and its database for gfx950.

The reference's tuner (MCTS over knob pins with a learned prior, results in a
SQLite database consulted by the cold schedule pick:
emmy/compiler/pipeline/search/, emmy/commands/tune.py) is replaced by the
smallest thing that fills the same two roles on this backend:

* :class:`TuneDB` — SQLite table ``tuned(arch, key, knobs, us, baseline_us)`` keyed
  by a kernel's *shape key* (``shape_key``).  ``passes.schedule`` asks it for
  pins when the environment does not pin a knob itself; a stored pin goes
  through the same validation / degrade path as ``EMMY_<KNOB>``.
* :func:`tune_graph` — exhaustive sweep of a candidate list per knob family.
  The pins of different families do not interact, so one compile + benchmark
  of the whole graph samples one candidate of every family at once; every
  candidate's outputs are checked against the untuned compile before its time
  counts.
"""

from __future__ import annotations

import contextlib
import json
import os
import sqlite3
import time
from dataclasses import dataclass, field
from pathlib import Path

from deplodock_amd import config
from deplodock_amd.ir.tile import Contraction, Flash, RowReduce

TILE_SWEEP: tuple[str, ...] = (
    "a:mfma_16x16x32_bf16/w2x4/f8x4/k2",
    "a:mfma_16x16x32_bf16/w2x4/f4x4/k2",
    "a:mfma_16x16x32_bf16/w2x4/f4x3/k2",
    "a:mfma_16x16x32_bf16/w4x2/f2x6/k2",
    "a:mfma_16x16x32_bf16/w4x2/f2x4/k2",
    "a:mfma_32x32x16_bf16/w2x2/f2x2/k4",
    "a:mfma_16x16x32_bf16/w4x2/f2x3/k2",
    "a:mfma_16x16x32_bf16/w2x4/f2x4/k2",
    "a:mfma_16x16x32_bf16/w2x4/f2x2/k4",
    "a:mfma_16x16x32_bf16/w4x2/f1x3/k2",
    "a:mfma_16x16x32_bf16/w2x4/f2x1/k4",
    "a:mfma_16x16x32_bf16/w2x2/f2x2/k4",
    "a:mfma_16x16x32_bf16/w2x4/f1x2/k4",
    "a:mfma_16x16x32_bf16/w2x2/f1x3/k4",
    "a:mfma_16x16x32_bf16/w2x4/f1x1/k8",
    "a:mfma_16x16x32_bf16/w1x4/f2x1/k8",
    "a:mfma_16x16x32_bf16/w2x2/f1x1/k8",
    "a:mfma_16x16x32_bf16/w1x4/f1x2/k8",
    "a:mfma_16x16x32_bf16/w1x2/f1x1/k8",
    # the few-row tiles on 128-deep slabs (room for a third ring slot where 256-deep ones leave none)
    "a:mfma_16x16x32_bf16/w2x4/f1x1/k4",
    "a:mfma_16x16x32_bf16/w1x4/f1x2/k4",
    "a:mfma_16x16x32_bf16/w1x2/f1x1/k4",
    "a:mfma_16x16x32_bf16/w1x1/f1x1/k8",
)  # every tile that won an in-graph ranking of the decoder block's contractions at 64 ... 2048 tokens, and their neighbours
# The fp32 tier (fp32 MFMA atoms; slab depth in atom steps of 4): the tiles that ranked first somewhere in a sweep of the
# decoder layer's projections at 32 / 128 / 512 tokens in fp32.
TILE_SWEEP_F32: tuple[str, ...] = tuple(
    f"a:mfma_16x16x4_f32/{units}/k{bk}"
    for units in ("w4x2/f1x3", "w2x2/f2x3", "w2x4/f2x2", "w2x4/f2x1", "w4x2/f1x2", "w2x2/f2x2", "w2x4/f1x1", "w2x2/f1x2", "w2x2/f1x1", "w1x4/f1x1", "w1x2/f1x1")
    for bk in (16, 32, 8)
) + tuple(
    f"a:mfma_32x32x2_f32/{units}/k{bk}"
    for units in ("w2x2/f1x1", "w2x4/f1x1", "w4x2/f1x1", "w2x2/f2x1", "w2x2/f1x2", "w2x4/f2x1", "w2x2/f2x2")
    for bk in (16, 32)
)  # (the 32x32x2 atoms never ranked first at these sizes: kept so that a sweep says so)
STAGE_SWEEP_F32: tuple[str, ...] = ("d3/dl", "d2/dl")
STAGE_SWEEP: tuple[str, ...] = ("d2/dl", "d3/dl", "d2/sync/p2")
# the k-split few-row form has no tile: waves that split the reduction axis x output columns a workgroup (16 unless named)
FEW_ROW_SWEEP: tuple[str, ...] = ("d8/ks", "d4/ks", "d2/ks", "d8/ks/c12", "d4/ks/c12", "d8/ks/c8", "d4/ks/c8", "d2/ks/c8", "d8/ks/c4", "d4/ks/c4")
REDUCE_SWEEP: tuple[str, ...] = ("b8", "b16", "b32", "b64", "b128", "b256", "b512", "b1024")
NT_SWEEP: tuple[str, ...] = ("0", "1")
FLASH_SWEEP: tuple[str, ...] = (
    "w4/kv64/s2", "w2/kv64/s2", "w1/kv64/s2", "w2/kv32/s4", "w1/kv32/s4", "w4/kv32/s2", "w4/kv64/s1",
    "w2/kv32/s4/p", "w2/kv64/s2/p", "w1/kv32/s4/p", "w4/kv64/s2/p", "w8/kv64/s1", "w8/kv64/s1/p",
)  # fmt: skip
#: attention on fp32 MFMA atoms: row groups that share each staged block, or waves that split a row group's key blocks
#: (``/o``: a wave's K and V blocks take turns in one LDS region; ``/sp``: the software-pipelined order)
FLASH_SWEEP_F32: tuple[str, ...] = ("f32/w1", "f32/w2", "f32/w4", "f32/s2", "f32/s4", "f32/s8", "f32/s2/o", "f32/s4/o", "f32/s8/o", "f32/s4/sp")


def shape_key(body) -> str | None:
    """What a tuned pin is valid for: the kernel family and every size / dtype /
    structural flag its schedule depends on."""
    if isinstance(body, Contraction):
        return f"contraction/m{body.m}/n{body.n}/k{body.k}/{body.in_dtype.name}>{body.out_dtype.name}/g{int(body.gate_pair)}/p{int(body.post is not None)}/a{int(body.a_prologue is not None)}" + (f"/e{body.row_epilogue.cols}" if body.row_epilogue is not None else "") + (
            f"/x{body.batch}" if getattr(body, "batch", 1) > 1 else "")
    if isinstance(body, RowReduce):
        return f"row_reduce/r{body.rows}/c{body.cols}/{body.x_dtype.name}>{body.out_dtype.name}/s{len(body.stats)}/rot{int(body.rotate is not None)}"
    if isinstance(body, Flash):
        return f"flash/b{body.batch}/hq{body.q_heads}/hkv{body.kv_heads}/sq{body.q_len}/skv{body.kv_len}/d{body.head_dim}/c{int(body.causal)}/{body.dtype.name}"
    return None


FAMILY_KNOBS = {"contraction": ("TILE", "STAGE"), "row_reduce": ("REDUCE", "NT"), "flash": ("FLASH",)}


class TuneDB:
    """SQLite store of the best measured knob pins per (arch, shape key)."""

    def __init__(self, path: str | os.PathLike | None = None, arch: str = "gfx950"):
        self.path = Path(path) if path not in (None, "auto") else config.tune_db_path()
        self.arch = arch
        self.path.parent.mkdir(parents=True, exist_ok=True)
        self._db = sqlite3.connect(str(self.path))
        self._db.execute(
            "CREATE TABLE IF NOT EXISTS tuned (arch TEXT NOT NULL, key TEXT NOT NULL, knobs TEXT NOT NULL, us REAL NOT NULL, "
            "baseline_us REAL, created REAL NOT NULL, PRIMARY KEY (arch, key))"
        )
        self._db.commit()

    def lookup(self, key: str | None) -> dict[str, str]:
        if key is None:
            return {}
        row = self._db.execute("SELECT knobs FROM tuned WHERE arch = ? AND key = ?", (self.arch, key)).fetchone()
        return json.loads(row[0]) if row else {}

    def store(self, key: str, knobs: dict[str, str], us: float, baseline_us: float | None = None) -> None:
        """Keep ``knobs`` for ``key`` unless a faster entry is already there."""
        row = self._db.execute("SELECT us FROM tuned WHERE arch = ? AND key = ?", (self.arch, key)).fetchone()
        if row is not None and row[0] <= us:
            return
        self._db.execute(
            "INSERT OR REPLACE INTO tuned (arch, key, knobs, us, baseline_us, created) VALUES (?, ?, ?, ?, ?, ?)",
            (self.arch, key, json.dumps(knobs, sort_keys=True), float(us), baseline_us, time.time()),
        )
        self._db.commit()

    def rows(self) -> list[tuple[str, dict[str, str], float, float | None]]:
        cur = self._db.execute("SELECT key, knobs, us, baseline_us FROM tuned WHERE arch = ? ORDER BY key", (self.arch,))
        return [(k, json.loads(j), us, base) for k, j, us, base in cur.fetchall()]

    def close(self) -> None:
        self._db.close()


@contextlib.contextmanager
def pinned(knobs: dict[str, str]):
    """Pin ``knobs`` through ``EMMY_KNOBS`` for the duration of the block (direct
    ``EMMY_<KNOB>`` variables of the same names are lifted meanwhile)."""
    saved = {config.KNOBS: os.environ.get(config.KNOBS)}
    for k in knobs:
        saved[config.knob_var(k)] = os.environ.pop(config.knob_var(k), None)
    os.environ[config.KNOBS] = ",".join(f"{k}={v}" for k, v in knobs.items())
    try:
        yield
    finally:
        for var, val in saved.items():
            if val is None:
                os.environ.pop(var, None)
            else:
                os.environ[var] = val


@dataclass
class KernelTuning:
    key: str
    kernel: str
    baseline_knobs: dict[str, str]
    baseline_us: float
    best_knobs: dict[str, str]
    best_us: float
    tried: int = 0
    rejected: list[str] = field(default_factory=list)

    @property
    def speedup(self) -> float:
        return self.baseline_us / self.best_us if self.best_us > 0 else 1.0


def _kernels(compiled) -> list:
    """``(launch index, HipOp, shape key)`` of every tunable launch, in program order."""
    from deplodock_amd.ir.hip import HipOp

    out = []
    idx = 0
    for nid in compiled.topological_order():
        op = compiled.nodes[nid].op
        if isinstance(op, HipOp):
            src = getattr(op, "source", None)
            out.append((idx, op, shape_key(src.body) if src is not None else None))
            idx += 1
    return out


def candidate_rounds(families: set[str]) -> list[dict[str, str]]:
    """One pin set per round; round r holds the r-th candidate of every family present."""
    per_family: dict[str, list[dict[str, str]]] = {}
    if "contraction" in families:
        per_family["contraction"] = [{"TILE": t, "STAGE": s} for s in STAGE_SWEEP for t in TILE_SWEEP] + [{"TILE": TILE_SWEEP[-1], "STAGE": s} for s in FEW_ROW_SWEEP]
    if "row_reduce" in families:
        per_family["row_reduce"] = [{"REDUCE": r, "NT": n} for n in NT_SWEEP for r in REDUCE_SWEEP]
    if "flash" in families:
        per_family["flash"] = [{"FLASH": f} for f in FLASH_SWEEP]
    rounds = max((len(v) for v in per_family.values()), default=0)
    out = []
    for r in range(rounds):
        pins: dict[str, str] = {}
        for cands in per_family.values():
            if r < len(cands):
                pins.update(cands[r])
        out.append(pins)
    if "contraction_f32" in families:
        # rounds of their own: TILE / STAGE name one atom type, and a 16-bit contraction of the same graph keeps its defaults meanwhile
        out += [{"TILE": t, "STAGE": s} for s in STAGE_SWEEP_F32 for t in TILE_SWEEP_F32]
    if "flash_f32" in families:
        out += [{"FLASH": f} for f in FLASH_SWEEP_F32]  # (rounds of their own for the same reason)
    return out


def _family(key: str) -> str:
    """Candidate family of a shape key: fp32 contractions sweep fp32 atoms."""
    fam = key.split("/")[0]
    if fam == "flash" and key.endswith("/f32"):
        return "flash_f32"
    return "contraction_f32" if fam == "contraction" and "/f32>" in key else fam


def tune_graph(graph, backend, db: TuneDB | None = None, *, input_data: dict | None = None, warmup: int = 3, num_iters: int = 10,
               min_gain: float = 1.02, max_rounds: int | None = None, progress=None) -> list[KernelTuning]:  # fmt: skip
    """Sweep the candidate pins over ``graph`` on the GPU; store winners in ``db``.

    A candidate counts for a kernel only if the schedule kept the pin (an
    unrealisable pin degrades, and the degraded kernel is the baseline again) and
    the program's outputs match the untuned program's."""
    import torch

    def outputs_of(compiled) -> dict:
        prog = backend.program(compiled, input_data)
        try:
            prog.run()
            torch.cuda.synchronize()
            return {k: v.float().clone() for k, v in prog.output_tensors().items() if k in compiled.outputs}
        finally:
            prog.close()

    with pinned({}):
        base = backend.compile(graph)
    want = outputs_of(base)
    base_bench = backend.benchmark(base, warmup=warmup, num_iters=num_iters, input_data=input_data)
    base_us = {lt.idx: (min(lt.samples) if lt.samples else lt.time_ms) * 1e3 for lt in base_bench.per_launch}
    results: dict[str, KernelTuning] = {}
    for idx, op, key in _kernels(base):
        if key is None or key in results:
            continue
        fam = key.split("/")[0]
        knobs = {k: str(op.knobs[k]) for k in FAMILY_KNOBS[fam] if k in op.knobs}
        results[key] = KernelTuning(key, op.kernel_name, knobs, base_us[idx], dict(knobs), base_us[idx])
    rounds = candidate_rounds({_family(k) for k in results})
    if max_rounds is not None:
        rounds = rounds[:max_rounds]
    for r, pins in enumerate(rounds):
        with pinned(pins):
            try:
                compiled = backend.compile(graph)
            except Exception as exc:  # noqa: BLE001 - a candidate that cannot be lowered is just not a candidate
                if progress:
                    progress(r, len(rounds), pins, f"skipped: {exc}")
                continue
        try:
            got = outputs_of(compiled)
            ok = all(torch.allclose(got[k], want[k], rtol=2e-2, atol=2e-2) for k in want)
            bench = backend.benchmark(compiled, warmup=warmup, num_iters=num_iters, input_data=input_data)
        except Exception as exc:  # noqa: BLE001 - e.g. a launch the device refuses
            if progress:
                progress(r, len(rounds), pins, f"failed: {exc}")
            continue
        us = {lt.idx: (min(lt.samples) if lt.samples else lt.time_ms) * 1e3 for lt in bench.per_launch}
        timed: list[str] = []  # what the progress line reports: every kernel that kept its pin, with its time
        for idx, op, key in _kernels(compiled):
            res = results.get(key)
            if res is None:
                continue
            fam = key.split("/")[0]
            want_pins = {k: pins[k] for k in FAMILY_KNOBS[fam] if k in pins}
            kept = all(str(op.knobs.get(k)) == v for k, v in want_pins.items())
            if not want_pins or not kept:
                continue
            res.tried += 1
            timed.append(f"{op.kernel_name} {us[idx]:.2f} us")
            if not ok:
                res.rejected.append(",".join(f"{k}={v}" for k, v in want_pins.items()))
                continue
            if us[idx] < res.best_us:
                res.best_us, res.best_knobs = us[idx], dict(want_pins)
        if progress:
            progress(r, len(rounds), pins, ("ok" if ok else "outputs differ: rejected") + (f" [{'; '.join(timed)}]" if timed else " [pin not kept]"))
    out = list(results.values())
    if db is not None:
        for res in out:
            if res.best_knobs != res.baseline_knobs and res.baseline_us / res.best_us >= min_gain:
                db.store(res.key, res.best_knobs, res.best_us, res.baseline_us)
    return out
