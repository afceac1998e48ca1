"""Schedule plans and their string codecs, re-derived for gfx950.

The *grammar* of the three knob families is the reference's
(emmy/compiler/ir/schedule.py): ``REDUCE`` = ``g<n>[a|k]/b<n>/r<n>`` (:435-443),
``TILE`` = ``a:<atom>/w<WM>x<WN>/f<FM>x<FN>/k<bk>`` (:552-561) and ``STAGE`` =
``d<depth>/<transport>[/ring][/p<reg_depth>]`` (:697-785), so existing
``EMMY_REDUCE`` / ``EMMY_TILE`` / ``EMMY_STAGE`` pins keep their shape.  The
*value space* is new: atoms are 64-lane MFMA shapes, the cooperative reduce
width counts wave64 lanes, and the transports are ``sync`` (global → VGPR →
LDS) and ``dl`` (direct-to-LDS global loads, the CDNA4 analogue of the
reference's ``cp`` token, which is accepted as an alias).
"""

from __future__ import annotations

import re
from dataclasses import dataclass


class ScheduleError(ValueError):
    """A knob value does not parse or is not legal for gfx950."""


# --------------------------------------------------------------------------
# Atoms (emmy/compiler/ir/atom.py:66-120 registers 32-lane mma.sync atoms)
# --------------------------------------------------------------------------


@dataclass(frozen=True)
class Atom:
    """One MFMA instruction shape: a wave64 computes an ``m x n`` fp32 tile
    from ``m x k`` and ``n x k`` operands; each lane feeds ``k_per_lane``
    consecutive k-values of one row/column and owns ``m*n/64`` accumulators.
    The fp32 atoms (``v_mfma_f32_32x32x2_f32`` / ``16x16x4``: full fp32 products,
    no reduced-precision pass) stand where the reference's scalar fp32 tier does
    (emmy/compiler/pipeline/passes/lowering/kernel/_atom.py:717-786)."""

    name: str
    m: int
    n: int
    k: int
    dtype: str  # operand dtype
    builtin: str
    lanes: int = 64

    @property
    def k_per_lane(self) -> int:
        return self.m * self.k // self.lanes

    @property
    def acc_per_lane(self) -> int:
        return self.m * self.n // self.lanes

    @property
    def elem_bytes(self) -> int:
        return 4 if self.dtype == "f32" else 2

    @property
    def frag_k(self) -> int:
        """k-values one fragment read covers: every lane fetches a 16-byte chunk of its row, and the
        ``64 / m`` lane groups of a row fetch neighbouring chunks.  A 16-bit atom consumes that in one
        MFMA (``frag_k == k``), an fp32 atom in four."""
        return (16 // self.elem_bytes) * (self.lanes // self.m)


ATOMS: dict[str, Atom] = {
    a.name: a
    for a in (
        Atom("mfma_32x32x16_bf16", 32, 32, 16, "bf16", "__builtin_amdgcn_mfma_f32_32x32x16_bf16"),
        Atom("mfma_16x16x32_bf16", 16, 16, 32, "bf16", "__builtin_amdgcn_mfma_f32_16x16x32_bf16"),
        Atom("mfma_32x32x16_f16", 32, 32, 16, "f16", "__builtin_amdgcn_mfma_f32_32x32x16_f16"),
        Atom("mfma_16x16x32_f16", 16, 16, 32, "f16", "__builtin_amdgcn_mfma_f32_16x16x32_f16"),
        Atom("mfma_32x32x2_f32", 32, 32, 2, "f32", "__builtin_amdgcn_mfma_f32_32x32x2f32"),
        Atom("mfma_16x16x4_f32", 16, 16, 4, "f32", "__builtin_amdgcn_mfma_f32_16x16x4f32"),
    )
}


def _ints(tok: str, what: str) -> tuple[int, ...]:
    try:
        vals = tuple(int(p) for p in tok.split("x"))
    except ValueError as exc:
        raise ScheduleError(f"{what}: expected integers, got {tok!r}") from exc
    if any(v <= 0 for v in vals):
        raise ScheduleError(f"{what}: values must be positive, got {tok!r}")
    return vals


def _pow2(v: int) -> bool:
    return v > 0 and (v & (v - 1)) == 0


# --------------------------------------------------------------------------
# REDUCE
# --------------------------------------------------------------------------


@dataclass(frozen=True)
class ReducePlan:
    """How one reduce axis is partitioned, coarse → fine (schedule.py:447-538).

    ``cta``   workgroups that split the axis (cross-workgroup; ``finalize`` is
              ``atomic`` = fp32 atomic adds into a zeroed output, or ``kernel``
              = partials workspace + a combine kernel).
    ``coop``  lanes that cooperate on one row inside a workgroup.  ≤ 64 is a
              (sub-)wave combined with DPP/swizzle butterflies only; a multiple
              of 64 adds one LDS hand-off of ``coop/64`` partials.
    ``reg``   independent accumulators per lane (ILP)."""

    cta: int = 1
    coop: int = 1
    reg: int = 1
    finalize: str = "kernel"

    def __post_init__(self) -> None:
        if not (_pow2(self.coop) and self.coop <= 1024):
            raise ScheduleError(f"REDUCE b<n>: n must be a power of two <= 1024, got {self.coop}")
        if self.cta < 1 or self.reg < 1:
            raise ScheduleError("REDUCE g<n>/r<n>: n must be >= 1")
        if self.finalize not in ("atomic", "kernel"):
            raise ScheduleError(f"REDUCE finalize must be atomic|kernel, got {self.finalize!r}")

    @classmethod
    def parse(cls, spec: str | None) -> ReducePlan:
        if not spec:
            return cls()
        kw: dict = {}
        for tok in spec.split("/"):
            tok = tok.strip()
            m = re.fullmatch(r"g(\d+)([ak]?)", tok)
            if m:
                kw["cta"] = int(m.group(1))
                kw["finalize"] = {"a": "atomic", "k": "kernel", "": "kernel"}[m.group(2)]
                continue
            m = re.fullmatch(r"b(\d+)", tok)
            if m:
                kw["coop"] = int(m.group(1))
                continue
            m = re.fullmatch(r"r(\d+)", tok)
            if m:
                kw["reg"] = int(m.group(1))
                continue
            raise ScheduleError(f"REDUCE: cannot parse {tok!r} (expect g<n>[a|k] / b<n> / r<n>)")
        return cls(**kw)

    def spell(self) -> str:
        parts = []
        if self.cta > 1:
            parts.append(f"g{self.cta}{'a' if self.finalize == 'atomic' else 'k'}")
        if self.coop > 1:
            parts.append(f"b{self.coop}")
        if self.reg > 1:
            parts.append(f"r{self.reg}")
        return "/".join(parts)


# --------------------------------------------------------------------------
# TILE
# --------------------------------------------------------------------------


@dataclass(frozen=True)
class TilePlan:
    """A contraction's output tile on the MFMA tier (schedule.py:574-660).

    ``units`` = waves (WM, WN) per workgroup, ``regs`` = atoms (FM, FN) per
    wave, ``bk`` = K-chunk per staged slab in atom-k units.  A workgroup
    computes ``tile_m x tile_n`` with ``WM*WN*64`` threads."""

    atom: Atom
    units: tuple[int, int] = (2, 2)
    regs: tuple[int, int] = (2, 2)
    bk: int = 1

    @property
    def waves(self) -> int:
        return self.units[0] * self.units[1]

    @property
    def block_threads(self) -> int:
        return self.waves * self.atom.lanes

    @property
    def tile_m(self) -> int:
        return self.units[0] * self.regs[0] * self.atom.m

    @property
    def tile_n(self) -> int:
        return self.units[1] * self.regs[1] * self.atom.n

    @property
    def bk_elems(self) -> int:
        return self.bk * self.atom.k

    @property
    def acc_regs_per_lane(self) -> int:
        return self.regs[0] * self.regs[1] * self.atom.acc_per_lane

    @classmethod
    def parse(cls, spec: str) -> TilePlan:
        atom = None
        kw: dict = {}
        for tok in spec.split("/"):
            tok = tok.strip()
            if tok.startswith("a:"):
                name = tok[2:]
                if name not in ATOMS:
                    raise ScheduleError(f"TILE: unknown atom {name!r}; known: {', '.join(sorted(ATOMS))}")
                atom = ATOMS[name]
            elif tok.startswith("w"):
                v = _ints(tok[1:], "TILE w<WM>x<WN>")
                if len(v) != 2:
                    raise ScheduleError(f"TILE: w needs two dims, got {tok!r}")
                kw["units"] = v
            elif tok.startswith("f"):
                v = _ints(tok[1:], "TILE f<FM>x<FN>")
                if len(v) != 2:
                    raise ScheduleError(f"TILE: f needs two dims, got {tok!r}")
                kw["regs"] = v
            elif tok.startswith("k"):
                (kw["bk"],) = _ints(tok[1:], "TILE k<bk>")
            else:
                raise ScheduleError(f"TILE: cannot parse {tok!r} (expect a:<atom> / w<WM>x<WN> / f<FM>x<FN> / k<bk>)")
        if atom is None:
            raise ScheduleError("TILE: the a:<atom> token is required on gfx950 (MFMA tier only)")
        plan = cls(atom=atom, **kw)
        if plan.block_threads > 1024:
            raise ScheduleError(f"TILE: {plan.waves} waves exceed 1024 threads per workgroup")
        return plan

    def spell(self) -> str:
        s = f"a:{self.atom.name}/w{self.units[0]}x{self.units[1]}/f{self.regs[0]}x{self.regs[1]}"
        if self.bk > 1:
            s += f"/k{self.bk}"
        return s


# --------------------------------------------------------------------------
# STAGE
# --------------------------------------------------------------------------

_TRANSPORTS = {"sync": "sync", "dl": "dl", "dli": "dli", "dlm": "dlm", "pp": "pp", "cp": "dl", "mix": "mix", "ks": "ks"}


@dataclass(frozen=True)
class Stage:
    """Operand staging through LDS over the K loop (schedule.py:710-785).

    ``depth``      LDS slabs in the ring (2 = double buffer).
    ``transport``  ``sync``: global → registers → ``ds_write`` (software
                   pipelined through ``reg_depth`` register sets);
                   ``dl``: global loads that write LDS directly, no VGPR hop;
                   ``dli``: the same loads, issued one at a time between the MFMAs of
                   the slab before instead of as a burst behind its barrier;
                   ``dlm``: as ``dl`` (any ring depth), the requests of the steady state
                   spread among the MFMAs of the slab's last step;
                   ``pp``: the same loads issued by four extra waves (one per SIMD) that
                   do nothing else, while the tile's eight waves alternate in two groups
                   half a slab apart (one computes while the other reads fragments);
                   ``mix``: the a operand as ``sync``, the b operand as ``dl``;
                   ``ks``: no LDS staging of the weights — a few rows, the reduction axis split
                   over ``depth`` waves that load their fragments straight from global
                   memory, all at once; ``c<n>`` output columns per workgroup.
    ``ring``       kept for grammar compatibility (a depth > 1 is a ring)."""

    depth: int = 2
    transport: str = "sync"
    ring: bool = False
    reg_depth: int = 1
    cols: int = 0  # ``ks`` only: output columns per workgroup (``c4`` / ``c8`` / ``c12``; 0 = 16)

    @classmethod
    def parse(cls, spec: str | None) -> Stage | None:
        """``None`` / ``""`` = no staging pin.  ``tma`` has no CDNA4 counterpart:
        it raises so the caller can degrade the pin to its OFF value."""
        if not spec:
            return None
        kw: dict = {}
        for tok in spec.split("/"):
            tok = tok.strip()
            if re.fullmatch(r"d\d+", tok):
                kw["depth"] = int(tok[1:])
            elif tok in _TRANSPORTS:
                kw["transport"] = _TRANSPORTS[tok]
            elif tok == "tma":
                raise ScheduleError("STAGE: tma transport does not exist on gfx950")
            elif tok == "ring":
                kw["ring"] = True
            elif re.fullmatch(r"p\d+", tok):
                kw["reg_depth"] = int(tok[1:])
            elif re.fullmatch(r"c\d+", tok):
                kw["cols"] = int(tok[1:]) % 16
            else:
                raise ScheduleError(f"STAGE: cannot parse {tok!r} (expect d<depth> / sync|dl|mix / ring / p<reg_depth>)")
        st = cls(**kw)
        if not 1 <= st.depth <= 8:
            raise ScheduleError(f"STAGE: depth must be 1..8, got {st.depth}")
        return st

    def spell(self) -> str:
        s = f"d{self.depth}/{self.transport}"
        if self.ring:
            s += "/ring"
        if self.reg_depth > 1:
            s += f"/p{self.reg_depth}"
        if self.cols:
            s += f"/c{self.cols}"
        return s
