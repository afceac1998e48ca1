"""Schedule selection for gfx950: stamp ``ReducePlan`` / ``TilePlan`` / ``Stage`` on each tile.

Plays the role of the reference's ``_schedule`` (emmy/compiler/pipeline/passes/lowering/tile/_schedule.py:
``_pick_coop`` :104-117, contraction rows :382-419, ``schedule`` :819-899) with the
constants re-derived for 256 CUs, wave64 and 160 KB of LDS:

* ``EMMY_REDUCE`` / ``EMMY_TILE`` / ``EMMY_STAGE`` (or ``EMMY_KNOBS``) pins are
  authoritative.  A pin that does not parse or cannot be realised degrades to the
  heuristic pick and the *resolved* spelling is stamped on the op's ``knobs``
  (_schedule.py:755-761, 813-815).
* Row reductions: the reference refuses cooperation above 256 free rows
  (``_FREE_CAP``) and falls back to one thread per row; here every row kernel
  is cooperative and coalesced, and the lane count per row follows the row
  length so the row stays register-resident.
* Contractions: the tile is chosen so the launch fills the CUs (>= one workgroup
  per CU where the problem allows) before it is chosen for operand reuse; the
  candidates and their measured ranking live in ``TILE_CANDIDATES``.
"""

from __future__ import annotations

import logging

from deplodock_amd import config
from deplodock_amd.context import Context
from deplodock_amd.graph import Graph
from deplodock_amd.ir.schedule import ATOMS, ReducePlan, ScheduleError, Stage, TilePlan
from deplodock_amd.ir.tile import Contraction, Flash, IndexRows, LoopNest, Map, RowReduce, StridedCopy, TileOp

logger = logging.getLogger(__name__)

# (tile_m, tile_n, waves_m, waves_n, atom, bk) — ordered by measured throughput on
# MI355X (first fit that fills the machine wins).  The large tiles are ranked on a
# compute-bound 2048x3072x1024 problem; the small ones on 512-row and decode-size
# problems timed with operands rotating through more memory than the L2s hold,
# where a step of the k loop costs one L2-miss round trip whatever its size: deep
# slabs (256 elements) and 4-8 waves per workgroup won every such shape.
TILE_CANDIDATES: tuple[tuple[int, int, int, int, str, int], ...] = (
    (256, 256, 2, 4, "mfma_16x16x32_bf16", 2),  # 4096^3 with a two-slab dl ring: 111.8 us = 1 230 TFLOP/s (32x32x16 atoms, same tile: 119.5 us)
    (128, 256, 2, 4, "mfma_16x16x32_bf16", 2),
    (128, 192, 2, 4, "mfma_16x16x32_bf16", 2),  # 2048x3072x1024: 16.9 us as 2x4 waves of 64x48, 17.2 as 4x2 of 32x96 (less LDS read traffic)
    # eight waves on 16x16x32 atoms, 64-deep slabs: 1024 tokens q/k/v 16.3 us, gate/up 21.2 (four waves on 32x32x16 atoms: 18.2, 23.2)
    (128, 128, 4, 2, "mfma_16x16x32_bf16", 2),
    (128, 96, 4, 2, "mfma_16x16x32_bf16", 4),
    (64, 128, 2, 4, "mfma_16x16x32_bf16", 4),
    (64, 64, 2, 4, "mfma_16x16x32_bf16", 4),  # eight waves of 32x16: 1024x1024x2048 7.7 us (four of 32x32: 8.9)
    # Few-row problems (the decoder block at 64-256 tokens), ranked inside the block's graph: the tile that
    # makes about one multi-wave workgroup per CU wins over more, smaller ones (256 rows: o / down
    # projections 7.98 / 13.85 us on 1024 one-wave 16x16 tiles, 4.76 / 6.02 us on 256 four-wave 32x32 tiles;
    # q/k/v projection 9.29 us on 64x128, 6.91 us on 32x128; 128 rows: 16x32 tiles 4.16 / 5.11 against 4.49 / 7.45 us).
    (32, 128, 2, 4, "mfma_16x16x32_bf16", 4),
    (32, 64, 1, 4, "mfma_16x16x32_bf16", 8),
    (32, 32, 2, 2, "mfma_16x16x32_bf16", 8),
    (16, 128, 1, 4, "mfma_16x16x32_bf16", 4),  # 128-deep slabs leave the LDS for a third ring slot: the q/k/v projection at 64 / 128 tokens 5.95 / 6.11 us (256-deep, two slots: 6.35 / 6.49)
    (16, 32, 1, 2, "mfma_16x16x32_bf16", 8),
    (16, 16, 1, 1, "mfma_16x16x32_bf16", 8),
)

# A launch "fills the machine" from this fraction of the CUs on: 192 workgroups of
# a 64x128 tile beat 384 of a 64x64 tile on the gate/up shape (12.1 vs 16.1 us).
_FILL_FRACTION = 0.75


def _pin(name: str, tuned: dict | None = None) -> str | None:
    """The value knob ``name`` is pinned to: the environment first, then the tune database's entry for this kernel."""
    raw = config.knob_raw(name)
    if raw is None and tuned:
        raw = tuned.get(name)
    return raw


def _tuned(body, ctx: Context) -> dict:
    db = getattr(ctx, "tune_db", None)
    if db is None:
        return {}
    from deplodock_amd.tune import shape_key

    return db.lookup(shape_key(body))


def pick_coop(cols: int, elem_bytes: int, rows: int, ctx: Context, *, rotate: bool = False, stats: int = 2) -> int:
    """Lanes that share one row.  A lane keeps at most 32 row elements resident; beyond that the width
    follows the number of 16-byte loads per lane that streams fastest (one with a single statistic, two
    with more), on up to 512 lanes for machine-filling rows (1024 for rows of 2048 chunks and more)."""
    vec = max(1, 16 // elem_bytes)
    chunks = max(1, cols // vec) if cols % vec == 0 else cols
    if rotate:
        while vec > 1 and cols % vec == 0 and (cols // vec) % 2:
            vec //= 2  # as the emitter: each half of the row is whole vectors
        chunks = max(1, cols // vec) if cols % vec == 0 else cols
        lanes = 1
        while lanes * 2 <= 64 and (chunks // 2) % (lanes * 2) == 0 and chunks // (lanes * 2) >= 2:
            lanes *= 2
        return lanes
    lanes = 1
    while lanes < 1024 and cols > lanes * 32:
        lanes *= 2
    # Bandwidth-bound rows: what matters is how many 16-byte loads a lane keeps in flight and how many hand-off
    # barriers the workgroup takes.  Swept over machine-filling fp32 rows of 1024 / 2048 / 4096 / 8192 columns
    # (64 Mi elements in, as many out; us, best two widths):
    #   one statistic (RMSNorm):  b256 81.6 / b128 82.9;  b512 82.1 / b128 84.9;  b256 86.3 / b512 86.3;  b1024 85.6 / b128 86.9
    #   two statistics (softmax): b128 81.6 / b64 84.4;   b256 81.3 / b128 85.1;  b512 81.3 / b256 85.1;  b1024 86.7 / b128 88.6
    # i.e. one load per lane with one statistic, two with more, on at most 512 lanes — 1024 once a lane of a
    # 512-lane workgroup would hold four loads or more.  Rows that do not fill the machine stay at 256 lanes at
    # most (wider workgroups only add hand-off latency there).
    per_lane = 1 if stats == 1 else 2
    filling = rows * 512 >= ctx.compute_units * 2048
    limit = (1024 if chunks >= 4 * 512 else 512) if filling else 256
    while lanes < limit and chunks >= lanes * 2 * per_lane:
        lanes *= 2
    # Few rows: spread each row over more lanes so more CUs take part.
    while lanes < 256 and rows * lanes < ctx.compute_units * 64 and chunks >= lanes * 2:
        lanes *= 2
    return min(lanes, 1024)


def _pow2_floor(v: int) -> int:
    p = 1
    while p * 2 <= v:
        p *= 2
    return p


#: fp32 row elements a lane keeps resident at most (the register-resident emitter's limit)
_MAX_RESIDENT = 64


def schedule_row_reduce(body: RowReduce, ctx: Context) -> dict:
    tuned = _tuned(body, ctx)
    pinned = _pin("REDUCE", tuned)
    streamable = body.rotate is None and not body.row_operands
    if streamable and ((pinned or "").endswith("/stream") or -(-body.cols // ctx.max_threads_per_block) > _MAX_RESIDENT):
        # Too long to hold in registers (or pinned): one workgroup streams the row, one pass per statistic level.
        body.stream = True
        body.reduce = ReducePlan(coop=ctx.max_threads_per_block)
        return {"REDUCE": f"b{ctx.max_threads_per_block}/stream", "NT": 0}
    plan = None
    if pinned is not None:
        try:
            plan = ReducePlan.parse(pinned)
            if plan.cta != 1:
                # one value per row from a single statistic: the columns split across workgroups (partial row kernel into
                # an fp32 workspace, combine row kernel with the projection); anything that writes the row back does not
                addr = body.x_addr
                if not (body.scalar_out and len(body.stats) == 1 and not body.col_operands and not body.row_operands and body.rotate is None):
                    raise ScheduleError("cross-workgroup split does not apply to a projected row")
                if addr is not None and addr.div != 1:
                    raise ScheduleError("cross-workgroup split needs uniformly strided rows")
                if getattr(body, "sym", None) is not None and body.sym.fields:
                    raise ScheduleError("cross-workgroup split does not combine with a symbolic row count")
                vec = max(1, 16 // body.x_dtype.nbytes)
                if body.cols % plan.cta or (body.cols // plan.cta) % vec:
                    raise ScheduleError(f"{body.cols} columns do not split into {plan.cta} slices of whole 16-byte chunks")
                if plan.finalize == "atomic":
                    logger.warning("EMMY_REDUCE=%r: a row's projection is applied once, after the fold: g%dk instead", pinned, plan.cta)
                    plan = ReducePlan(cta=plan.cta, coop=plan.coop, reg=plan.reg, finalize="kernel")
                if plan.coop == 1:
                    plan = ReducePlan(cta=plan.cta, coop=pick_coop(body.cols // plan.cta, body.x_dtype.nbytes, body.rows * plan.cta, ctx, stats=1), reg=plan.reg, finalize="kernel")
            if -(-(body.cols // plan.cta) // plan.coop) > 64:
                raise ScheduleError(f"{body.cols // plan.cta} columns over {plan.coop} lanes do not fit the register-resident row")
            if body.rotate is not None:
                vec = 16 // max(body.x_dtype.nbytes, body.out_dtype.nbytes)
                if (body.cols // vec // 2) % plan.coop:
                    raise ScheduleError("rotate-half needs both halves of a row in one lane")
        except ScheduleError as exc:
            logger.warning("EMMY_REDUCE=%r ignored: %s", pinned, exc)
            plan = None
    if plan is None:
        eb = max(body.x_dtype.nbytes, body.out_dtype.nbytes)
        plan = ReducePlan(coop=pick_coop(body.cols, eb, body.rows, ctx, rotate=body.rotate is not None, stats=len(body.stats)))
    body.reduce = plan
    nt = _pin("NT", tuned)
    if nt is not None:
        body.nontemporal = nt.strip().lower() in ("1", "true", "yes", "on")
    else:
        # Streaming rows far larger than the caches: bypass-style accesses measured ~10 % faster.
        body.nontemporal = body.algo_bytes() > 256 * 1024 * 1024
    return {"REDUCE": plan.spell(), "NT": int(body.nontemporal)}


def pick_tile(m: int, n: int, k: int, gate_pair: bool, ctx: Context, row_prologue: bool = False, group_cols: tuple[int, int] | None = None, copies: int = 1) -> TilePlan:
    """The largest candidate that makes one workgroup per CU (0.9-1.0 of the CUs, no ragged
    edge), else the first (in measured-throughput order) whose launch covers 75 % of the CUs,
    else the one that launches the most workgroups.

    One round of workgroups, each as large as that allows, is what the decoder block's
    projections prefer at every token count (in-graph times, us): 2048 tokens q/k/v 34.6 on
    256 tiles of 128x128 with four waves, 28.2 on 256 tiles of 128x256; 1024 tokens gate/up
    22.6 on 192 tiles of 128x128, 18.2 on 256 tiles of 128x96; 512 tokens gate/up 12.8 on 192
    tiles of 64x128, 10.4 on 256 of 64x96; 256 tokens gate/up 9.93 on 64x64, 8.85 on 32x96.

    ``copies``: independent products of this shape in the one launch (a batched contraction): each adds its own
    workgroups."""
    best = None
    candidates = TILE_CANDIDATES
    one_round_only = {(128, 256)}  # offered only as an exact fit: as a 75 % cover it was not measured
    if m > 64:
        # Beyond 64 rows: eight waves of one fragment each on the 32x64 tile (more
        # loads in flight per CU than four waves of two): 6.20 vs 6.39 us on
        # 512x1024x2048, 7.94 vs 9.16 us on 512x1024x3072, inside the decoder block; the
        # gate / up pair at 80 / 96 / 112 rows 6.53 / 6.60 / 6.58 against 7.75 / 7.61 / 7.69.
        # (below 128 rows the four-wave form stays behind it, for the shapes the eight-wave one does not divide)
        eight = (32, 64, 2, 4, "mfma_16x16x32_bf16", 8)
        candidates = tuple(x for c in candidates for x in ((eight,) if c[:4] == (32, 64, 1, 4) and m >= 128 else (eight, c) if c[:4] == (32, 64, 1, 4) else (c,)))
    if gate_pair:
        # two weight rows per output column: 96-column tiles make 32 column blocks of 2 x 3072 outputs
        extra = ((128, 96, 4, 2, "mfma_16x16x32_bf16", 2), (64, 96, 4, 2, "mfma_16x16x32_bf16", 2), (32, 96, 2, 2, "mfma_16x16x32_bf16", 4))
        one_round_only |= {c[:2] for c in extra}
        if not row_prologue:
            # a gate/up pair stages two weight rows per output column, so the balanced
            # slab is twice as tall as wide: 128x64 moves 20 % fewer bytes through the L1
            # than 64x128 for the same workgroup count (10.96 vs 12.04 us on 512x1024x(2x3072)).
            # Not with a row-normalised operand: its statistic pass re-reads the tile's rows,
            # and twice the rows cost more than the slabs save (17.2 vs 15.9 us).
            extra = (*extra, (128, 64, 4, 2, "mfma_16x16x32_bf16", 4))
        i = next(k for k, c in enumerate(candidates) if c[:2] == (128, 96))
        candidates = (*candidates[:i], *extra, *candidates[i:])
    plans = []
    for cand in candidates:
        tm, tn, wm, wn, atom_name, bk = cand
        atom = ATOMS[atom_name]
        if tm % (wm * atom.m) or tn % (wn * atom.n):
            continue
        if group_cols is not None and (tn % group_cols[0] or group_cols[1] % tn or (tm * tn // 8) % (wm * wn * 64)):
            continue  # a row epilogue works on whole column groups of a staged output tile
        fm, fn = tm // (wm * atom.m), tn // (wn * atom.n)
        if fm * fn * atom.acc_per_lane * (2 if gate_pair else 1) > 160:
            continue  # two waves per SIMD leave 256 registers a lane: accumulators, fragments and addresses
        nb = 2 if gate_pair else 1
        if k % atom.k and k % 8 == 0 and not row_prologue:
            bk = 2 if k > 2 * atom.k else 1  # a short last slab (zero-filled on the register-staged path)
        else:
            while bk > 1 and (k % (bk * atom.k) or 2 * (tm + tn * nb) * bk * atom.k * 2 > ctx.lds_bytes_per_cu):
                bk //= 2
            if k % (bk * atom.k):
                continue
            if bk == 8 and 3 * (tm + tn * nb) * bk * atom.k * 2 > ctx.lds_bytes_per_cu and k % (4 * atom.k) == 0:
                # the few-row tiles' 256-deep slabs give way to 128-deep ones where only those leave the LDS for a third ring
                # slot (the gate / up pair on the eight-wave 32x64 tile at 96 / 128 rows: 6.18 / 6.21 us against 6.60 / 6.62)
                bk = 4
        threads = wm * wn * 64
        cpr = bk * atom.k // 8
        if (tm * cpr) % threads or (tn * cpr * (2 if gate_pair else 1)) % threads:
            continue
        plans.append((cand, TilePlan(atom=atom, units=(wm, wn), regs=(fm, fn), bk=bk)))
    cus = ctx.compute_units
    for (tm, tn, wm, wn, *_), plan in plans:
        groups = -(-m // tm) * -(-n // tn) * copies
        # (the gate / up pair's 64x96 tile also as a three-quarter cover: 384 rows, 192 workgroups 10.23 us against 11.80
        # on 144 of 64x128 and more on 288 of 64x64)
        floor = 0.75 if gate_pair and (tm, tn) == (64, 96) else 0.9
        if wm * wn > 1 and m % tm == 0 and n % tn == 0 and floor * cus <= groups <= cus:
            return plan  # (the one-wave tile is the last resort: two waves on half as many 16x32 tiles beat it)
    half_round = None  # the first (largest) tile that covers at least half the CUs
    for (tm, tn, *_), plan in plans:
        if (tm, tn) in one_round_only:
            continue
        groups = -(-m // tm) * -(-n // tn) * copies
        # penalise tiles that mostly hang over the edge of a small problem
        waste = (-(-m // tm) * tm * -(-n // tn) * tn) / float(max(m * n, 1))
        if half_round is None and 0.5 * cus <= groups <= cus and waste < 1.5:
            half_round = plan
        if half_round is not None and cus < groups < 1.5 * cus and waste < 1.5:
            # a second round of workgroups for a few stragglers: the tile twice the size does the same work in one round
            # (96 rows, gate / up pair of 3072 columns: 288 workgroups of 32x32 11.07 us, 144 of 32x64 6.60)
            return half_round
        # two waves on a 16x32 tile beat one wave on each of twice as many 16x16 tiles down to a quarter of the CUs
        # (64 rows x 1024 columns: 4.11 / 5.01 us on 128 workgroups against 4.84 / 6.43 us on 256; 32 rows x 1024
        # columns, K = 3072: 4.70 us on 64 workgroups against 7.04 us on 128)
        fill = 0.25 if (tm, tn) == (16, 32) else _FILL_FRACTION
        if groups >= fill * cus and waste < 1.5:
            return plan
        one_wave = (tm, tn) == (16, 16)  # a lone wave walks the whole reduction axis: worth half a multi-wave workgroup
        score = (min(groups, cus) * (0.5 if one_wave else 1.0) / max(waste, 1e-9), tm * tn)
        if best is None or score > best[0]:
            best = (score, plan)
    if best is None:
        raise ScheduleError(f"no MFMA tile fits M={m} N={n} K={k}")
    return best[1]


def _check_tile(plan: TilePlan, body: Contraction, ctx: Context, depth: int, dl: bool = False) -> None:
    """The emitter's shape constraints, checked at schedule time so that an
    unrealisable pin degrades for the one kernel it does not fit instead of
    failing the whole lowering."""
    bk = plan.bk_elems
    es = plan.atom.elem_bytes
    epck = 16 // es
    cpr = bk // epck
    nb = 2 if body.gate_pair else 1
    threads = plan.block_threads
    if bk % epck or bk * es > 512 or cpr & (cpr - 1) or bk % plan.atom.frag_k:
        raise ScheduleError(f"slab depth {bk} must be a power-of-two number of 16-byte chunks, whole fragment reads, at most 512 bytes a row")
    a_chunks, b_chunks = plan.tile_m * cpr, plan.tile_n * cpr * nb
    if a_chunks % threads or b_chunks % threads:
        raise ScheduleError(f"tile {plan.tile_m}x{plan.tile_n}x{bk} does not divide over {threads} threads")
    if dl and (a_chunks % 64 or b_chunks % 64):
        raise ScheduleError("direct-to-LDS staging needs whole-wave chunk counts")
    if (plan.tile_m + plan.tile_n * nb) * bk * es * depth > ctx.lds_bytes_per_cu:
        raise ScheduleError("slabs exceed the LDS")
    if plan.regs[0] * plan.regs[1] * plan.atom.acc_per_lane * nb > 256:
        raise ScheduleError("accumulators exceed the 256 accumulation registers of a lane")
    if threads > ctx.max_threads_per_block:
        raise ScheduleError(f"{threads} threads per workgroup is not launchable")
    if dl and plan.regs[0] * plan.regs[1] * plan.atom.acc_per_lane * nb > (256 if threads <= 256 else 128 if threads <= 512 else 64):
        # the ring waits for part of its outstanding loads by count; spill stores share that counter and
        # complete out of order with loads, so a direct-to-LDS kernel must not spill
        raise ScheduleError("accumulators take more than half the registers of a lane: direct-to-LDS staging must not spill")
    if dl and (depth - 1) * ((a_chunks + b_chunks) // threads) > 63:
        raise ScheduleError("too many direct-to-LDS loads in flight for the six-bit vector-memory counter")
    re = body.row_epilogue
    if re is not None and (plan.tile_n % re.cols or re.col_end % plan.tile_n or (plan.tile_m * plan.tile_n // 8) % threads):
        raise ScheduleError(f"the row epilogue needs output tiles of whole {re.cols}-column groups")
    if re is not None and plan.tile_m * (plan.tile_n * body.out_dtype.nbytes + 16) > ctx.lds_bytes_per_cu:
        raise ScheduleError("the row epilogue works on the output tile staged in LDS, which this tile does not fit")


from deplodock_amd.emit.skinny import skinny_cols, skinny_waves  # noqa: E402


def pingpong_fits(plan: TilePlan, body: Contraction, ctx: Context, depth: int = 4, worthwhile: bool = True) -> bool:
    """Whether ``STAGE d<depth>/pp`` can be emitted for this tile, and (``worthwhile``) is worth it: eight waves own the tile (four
    more stage), a wave holds a whole slab's fragments beside its accumulators in the 168 registers a lane has at
    three waves a SIMD, the ring fits the LDS, the four staging waves' requests fit the six-bit counter, and a wave
    has at least 256 clocks of MFMA work a slab (the period's barrier costs about 120).  Measured against the
    default ``dl`` ring (us, same process): 2048x3072x1024 on the 128x192 tile 17.2 -> 13.6; 2048^3 on 128x128
    21.3 -> 19.6; shorter steps lose (1024^3 on 64x64: 4.8 -> 5.0, 512x4096x1024 on 64x128: 7.0 -> 7.7)."""
    if plan.block_threads != 512 or body.a_prologue is not None or body.row_epilogue is not None or body.k % plan.bk_elems:
        return False
    nb = 2 if body.gate_pair else 1
    fm, fn = plan.regs
    steps = plan.bk_elems // plan.atom.frag_k
    if plan.bk_elems % plan.atom.frag_k or steps < 1:
        return False
    mfma_per_step = (plan.atom.frag_k // plan.atom.k) * fm * fn * nb
    mfma_clocks = plan.atom.m * plan.atom.n * plan.atom.k * 2 // 1024  # 16 for a 16x16x32 16-bit atom, 32 for 32x32x16
    regs = steps * (nb * fn + fm) * 4 + fm * fn * nb * plan.atom.acc_per_lane
    chunks = (plan.tile_m + plan.tile_n * nb) * (plan.bk_elems * plan.atom.elem_bytes // 16)
    slab = (plan.tile_m + plan.tile_n * nb) * plan.bk_elems * plan.atom.elem_bytes
    return (
        regs <= 136 and slab * depth <= ctx.lds_bytes_per_cu and chunks % 256 == 0 and (plan.tile_m * plan.bk_elems * plan.atom.elem_bytes // 16) % 256 == 0
        and (depth - 1) * (chunks // 256) <= 63 and depth >= 3
        and (not worthwhile or (steps * mfma_per_step * mfma_clocks >= 256 and -(-body.k // plan.bk_elems) >= depth))
    )  # fmt: skip


#: The few-row form is the default up to this many rows and this many bytes of activation rows (it takes up to
#: ``skinny.MAX_ROWS`` rows when pinned).  Every workgroup reads all the rows, so they bound what a CU moves whatever the
#: column count: measured inside the decoder block (us, few-row form against the tiled ring), 16 rows: o_proj (K = 2048)
#: 3.5 / 3.9, down_proj (K = 3072) 4.5 / 5.0; 32 rows: gate / up (K = 1024, 64 KiB of rows) 5.3 / 6.0, o_proj (128 KiB)
#: 6.3 / 4.4, down_proj (192 KiB) 8.5 / 7.4; 48 rows: gate / up (96 KiB) 5.45 / 6.18; 64 rows: gate / up 7.7 / 6.0.
_FEW_ROWS = 48
_FEW_ROWS_BYTES = 96 * 1024


def _default_stage(plan: TilePlan, body: Contraction, ctx: Context) -> Stage:
    """Staging when nothing pins it.

    * A row-normalised operand is transformed in registers on its way to LDS: ``sync``
      (``mix`` sends the other operand direct to LDS; 12.7 / 15.8 us against 12.3 / 15.9 us).
    * Decode-size problems (M <= 16) are one pass over the weight matrix and cost memory round trips:
      where the shape allows, the k-split few-row form (``ks``: no slab loop, every wave requests all of
      its fragments at once; us back to back / with the weight streamed from HBM, 1024x3072:
      M = 1 3.03 / 4.40 -> 2.59 / 4.02, M = 16 3.10 / 4.56 -> 2.74 / 4.38).  Otherwise ``sync``
      through two register sets (measured with operands rotating through more memory
      than the caches hold: 4.4 / 4.5 / 6.2 us at M = 1 / 16 / 128 on 1024x3072, against
      5.2 / 5.4 / 6.9 through one set and 4.6 / 4.6 / 6.4 with a three-slab ``dl`` ring).
      At M = 128 the ring on the eight-wave 32x64 tile ties that when the weight comes from
      HBM (6.25 vs 6.27 us) and wins when it sits in the caches (4.02 vs 4.64 us); inside the
      decoder block at 64 tokens the ring wins on every projection (o: 4.11 vs 5.00 us).
    * Where :func:`pingpong_fits`: the wave-specialised ring (``d4/pp``).
    * Everything else: direct-to-LDS loads; a ring of three slabs where the LDS holds them
      and a slab is less than ~600 cycles of MFMA work, else two (us, ``d2/sync`` -> ``d2/dl`` -> ``d3/dl``: 512x1024x3072 12.2 -> 9.5 ->
      9.4; 512x1024x2048 7.4 -> 6.2 -> 6.2; 512x4096x1024 7.8 -> 6.8 -> 6.7; 2048x3072x1024
      17.2 -> 15.9 -> 16.1; 4096^3 136 -> 122; the block as one graph 66.9 -> 65.2 -> 62.8)."""
    steps = -(-body.k // plan.bk_elems)
    if skinny_waves(body) and body.m <= _FEW_ROWS and body.m * body.k * body.in_dtype.nbytes <= _FEW_ROWS_BYTES and (body.m <= 16 or body.k <= 1024):
        # (17-24 rows of K = 2048 fit the byte bound too, but two waves on 16x32 tiles are ahead there: 4.08 against 4.31 us)
        return Stage(depth=skinny_waves(body), transport="ks", cols=skinny_cols(body, ctx) % 16)
    if body.k % plan.bk_elems:
        return Stage(depth=2, transport="sync")  # the short last slab is zero-filled in registers
    if body.a_prologue is not None and body.a_prologue.scale is None:
        return Stage(depth=2, transport="sync")  # transformed in registers on its way to LDS
    if body.m <= 16:
        return Stage(depth=2, transport="sync", reg_depth=2 if steps >= 3 else 1)
    if body.k_split is None and body.in_dtype.nbytes == 2 and pingpong_fits(plan, body, ctx):
        return Stage(depth=4, transport="pp")
    if (plan.bk_elems // plan.atom.frag_k) % 2 == 0 and plan.bk_elems % plan.atom.frag_k == 0:
        # a slab that keeps the matrix pipe busy for long hides the next one's latency by itself
        mfma_cycles = plan.tile_m * plan.tile_n * (2 if body.gate_pair else 1) * plan.bk_elems * 2 // 4096
        for depth in (3, 2):
            if depth == 3 and (steps < 3 or mfma_cycles >= 600):
                continue
            if depth == 3 and body.in_dtype.name == "f32" and plan.block_threads <= 256 and plan.bk_elems >= 64:
                continue  # four-wave fp32 tiles: two slots leave the LDS to more workgroups a CU (see _fp32_even_rounds)
            try:
                _check_tile(plan, body, ctx, depth=depth, dl=True)
            except ScheduleError:
                continue
            loads = (plan.tile_m + plan.tile_n * (2 if body.gate_pair else 1)) * (plan.bk_elems // 8) // plan.block_threads
            if (depth - 1) * loads <= 63:  # the vector-memory counter has six bits
                # With eight and more MFMAs a step per wave the next slab's requests and the next step's fragment reads go
                # out one at a time between the MFMAs (``dlm``) instead of as a burst in front of them: 4096^3 on the 256x256
                # tile 111 -> 98.5 us; in the decoder block at 2 048 tokens q/k/v 31.4 -> 26.2, gate/up 29.9 -> 28.4 us.  Tiles
                # with fewer MFMAs a step have too little to spread over: four to six a step measured within +-4 % either
                # way depending on the box (gate/up at 512 tokens 10.4 -> 10.1 on one, 10.9 -> 11.4 on another), one a step
                # loses (down_proj at 512 tokens 8.0 -> 8.7 us): they keep the burst.
                spread = plan.regs[0] * plan.regs[1] * (2 if body.gate_pair else 1) >= 8
                return Stage(depth=depth, transport="dlm" if spread else "dl")
    return Stage(depth=2, transport="sync")


def _default_tile(body: Contraction, ctx: Context) -> TilePlan:
    atom_dtype = body.in_dtype.name
    re = body.row_epilogue
    plan = pick_tile(body.m, body.n, body.k, body.gate_pair, ctx, row_prologue=body.a_prologue is not None, group_cols=(re.cols, re.col_end) if re is not None else None,
                     copies=max(1, int(getattr(body, "batch", 1) or 1)))
    if atom_dtype == "f32" and all(isinstance(d, int) for d in (body.m, body.n, body.k)):
        # One even round of workgroups matters most at the fp32 matrix rate: 64x96 tiles (eight waves of 16x48) when they
        # make 0.9-1.0 workgroups per CU exactly (512x1024x3072: 30.6 us on 256 of them, 38.1 on 192 tiles of 64x128).
        groups = (body.m // 64) * (body.n // 96) * max(1, int(getattr(body, "batch", 1) or 1))
        if body.m % 64 == 0 and body.n % 96 == 0 and body.k % 64 == 0 and 0.9 * ctx.compute_units <= groups <= ctx.compute_units and not body.gate_pair and body.row_epilogue is None:
            return TilePlan(atom=ATOMS["mfma_16x16x4_f32"], units=(4, 2), regs=(1, 3), bk=16)
    if atom_dtype == "f32":
        # the fp32 tier keeps the candidate's tile and its slab's bytes per row: half the k-values, on the fp32 atom of the same m x n
        atom = ATOMS[{16: "mfma_16x16x4_f32", 32: "mfma_32x32x2_f32"}[plan.atom.m]]
        bk_elems = max(2 * atom.frag_k, plan.bk_elems // 2)
        while bk_elems > 2 * atom.frag_k and body.k % bk_elems:
            bk_elems //= 2
        plan = TilePlan(atom=atom, units=plan.units, regs=plan.regs, bk=bk_elems // atom.k)
        plan = _fp32_even_rounds(body, plan, ctx)
    elif plan.atom.dtype != atom_dtype:
        plan = TilePlan(atom=ATOMS[plan.atom.name.replace("bf16", atom_dtype)], units=plan.units, regs=plan.regs, bk=plan.bk)
    return plan


def _fp32_even_rounds(body: Contraction, plan: TilePlan, ctx: Context) -> TilePlan:
    """At the fp32 matrix rate a launch is as long as its fullest CU's MFMA work.  A tile whose workgroups fill the last
    round of CUs to less than 85 % gives way to four-wave 32x32 tiles when those make at least two rounds that come out
    more even (256 x 3072 x 1024: 192 tiles of 64x64 21.9 us, 768 of 32x32 17.6; 384 x 3072 x 1024: 144 tiles of 64x128
    1.4 times the 1 152 of 32x32).  That tile streams 64-deep slabs (128-deep
    beyond K = 2048) through two ring slots, which leaves the LDS for several workgroups a CU, one wave each a SIMD
    (256 x 1024 x 2048: 13.1 us against 15.0 with three 128-deep slabs; 256 x 1024 x 3072: 20.8 against 21.9)."""
    if not all(isinstance(d, int) for d in (body.m, body.n, body.k)) or body.gate_pair or body.row_epilogue is not None or body.a_prologue is not None:
        return plan
    cus = ctx.compute_units
    copies = max(1, int(getattr(body, "batch", 1) or 1))

    def evenness(tm: int, tn: int) -> tuple[int, float]:
        groups = -(-body.m // tm) * -(-body.n // tn) * copies
        return groups, groups / float(-(-groups // cus) * cus)

    small = (plan.units, plan.regs, plan.atom.name) == ((2, 2), (1, 1), "mfma_16x16x4_f32")
    if not small:
        _, even = evenness(plan.tile_m, plan.tile_n)
        groups32, even32 = evenness(32, 32)
        small = even < 0.85 and groups32 >= 2 * cus and even32 >= even + 0.1
    if not small:
        return plan
    bk = 16 if body.k <= 2048 else 32
    while bk > 8 and body.k % (bk * 4):
        bk //= 2
    return TilePlan(atom=ATOMS["mfma_16x16x4_f32"], units=(2, 2), regs=(1, 1), bk=bk)


def _fp32_underfilled(body: Contraction, plan: TilePlan, ctx: Context) -> tuple[TilePlan, int]:
    """The fp32 matrix pipe runs at a sixteenth of the 16-bit rate, so an fp32 problem is bound by how evenly its
    MFMA work spreads over the CUs long before memory matters: a 32 x 1024 x 3072 product on 128 one-wave tiles
    leaves half the CUs idle and each wave walks all of K alone (22.7 us).  When 32x32 tiles would not cover the
    CUs, the reduction axis is split across workgroups (partials workspace + combine kernel) until about two
    workgroups per CU run, on four-wave 32x32 tiles with 32-deep slabs.  Measured (us, the unsplit default ->
    this): 32x3072x1024 22.7 -> 5.8, 128x3072x1024 21.8 -> 10.7, 32x2048x1024 15.5 -> 4.9, 128x2048x1024 15.1 ->
    8.5, 32x1024x2048 6.5 -> 4.8, 32x1024x1024 6.7 -> 4.1, 128x1024x1024 6.6 -> 6.2; 16 rows and fewer likewise
    (16x1024x3072 19.9 -> 4.5 + 1.9, 16x4096x1024 7.7 -> 4.8 + 1.9; the fp32 decoder block at 1 / 16 tokens 71.1 / 72.5
    -> 46.8 / 49.1).  Problems whose 32x32 tiles already cover the CUs keep the unsplit default (128x1024x2048: 6.8
    unsplit, 8.4 split in two)."""
    plain = not (body.gate_pair or body.a_prologue is not None or body.row_epilogue is not None) and int(getattr(body, "batch", 1) or 1) == 1 and body.k_split is None
    sym = getattr(body, "sym", None)
    if sym is not None and sym.fields:
        return plan, 1  # the split's kernel pair bakes the row count in: a runtime-int kernel stays unsplit
    if body.in_dtype.name != "f32" or not plain or not all(isinstance(d, int) for d in (body.m, body.n, body.k)) or body.k % 32 or body.k < 256:
        return plan, 1
    if body.m <= 16 and body.k * body.n < (1 << 20):
        return plan, 1  # a small weight at decode sizes is one short launch: a second one would cost more than the idle CUs
    base = -(-body.m // 32) * -(-body.n // 32)
    if base >= ctx.compute_units:
        return plan, 1
    split = 1
    while split < 8 and base * split * 2 <= 2 * ctx.compute_units and (body.k // (split * 2)) % 32 == 0 and body.k // (split * 2) >= 128:
        split *= 2
    tile = TilePlan(atom=ATOMS["mfma_16x16x4_f32"], units=(2, 2), regs=(1, 1), bk=8)
    try:
        _check_tile(tile, body, ctx, depth=3, dl=True)
    except ScheduleError:
        return plan, 1
    return tile, split


def default_contraction_schedule(body: Contraction, ctx: Context) -> None:
    """Put the heuristic tile and staging on ``body``, whatever was pinned or tuned (the lowering's last
    resort for a pinned tile whose kernel only builds with register spills)."""
    body.tile = _default_tile(body, ctx)
    body.stage = _default_stage(body.tile, body, ctx)


def schedule_contraction(body: Contraction, ctx: Context) -> dict:
    tuned = _tuned(body, ctx)
    pinned = _pin("TILE", tuned)
    plan = None
    if pinned:
        try:
            plan = TilePlan.parse(pinned)
            if plan.atom.dtype != body.in_dtype.name:
                raise ScheduleError(f"atom {plan.atom.name} does not take {body.in_dtype} operands")
            if body.k % plan.bk_elems:
                raise ScheduleError(f"K={body.k} is not a multiple of the slab depth {plan.bk_elems}")
            if plan.atom.dtype == "f32" and (body.gate_pair or body.a_prologue is not None or body.row_epilogue is not None):
                raise ScheduleError("the fp32 tier takes a plain contraction")
            _check_tile(plan, body, ctx, depth=2)
        except ScheduleError as exc:
            logger.warning("EMMY_TILE=%r ignored: %s", pinned, exc)
            plan = None
    auto_split = 1
    if plan is None:
        plan = _default_tile(body, ctx)
        if not _pin("REDUCE", tuned):
            plan, auto_split = _fp32_underfilled(body, plan, ctx)
    body.tile = plan
    stage = None
    pinned_stage = _pin("STAGE", tuned)
    if pinned_stage:
        try:
            stage = Stage.parse(pinned_stage)
            if stage is not None and stage.transport in ("dl", "dli", "dlm") and ((plan.bk_elems // plan.atom.frag_k) % 2 or plan.bk_elems % plan.atom.frag_k):
                raise ScheduleError("direct-to-LDS staging needs an even number of MFMA steps per slab")
            if stage is not None and stage.transport == "ks":
                if not skinny_waves(body) or stage.depth not in (1, 2, 4, 8, 16) or body.k % (32 * stage.depth) or (stage.cols and (stage.cols % 4 or body.n % stage.cols)):
                    raise ScheduleError(f"the k-split few-row form does not fit M={body.m} N={body.n} K={body.k} with {stage.depth} waves and {stage.cols or 16} columns a workgroup")
            elif stage is not None and stage.transport == "pp":
                if not pingpong_fits(plan, body, ctx, depth=stage.depth, worthwhile=False):
                    raise ScheduleError("the wave-specialised ring takes a plain 16-bit contraction on an eight-wave tile whose slab fragments fit a lane's registers, and a ring of at least three that fits the LDS")
            elif stage is not None:
                _check_tile(plan, body, ctx, depth=max(2, stage.depth), dl=stage.transport in ("dl", "dlm"))
        except ScheduleError as exc:
            logger.warning("EMMY_STAGE=%r ignored: %s", pinned_stage, exc)
            stage = None
    if stage is not None and body.a_prologue is not None and body.a_prologue.scale is None and stage.transport in ("dl", "dlm"):
        logger.warning("STAGE=%s ignored: the row-normalised operand is transformed in registers (sync or mix staging only)", stage.spell())
        stage = None
    if stage is None:
        stage = _default_stage(plan, body, ctx)
    body.stage = stage
    knobs = {"TILE": plan.spell(), "STAGE": stage.spell()}
    # Cross-workgroup split of the reduction axis (``REDUCE=g<n>k`` workspace + combine, ``g<n>a`` atomic adds
    # into a zeroed workspace + combine).  Only a pin asks for it: on the measured shapes the second launch costs
    # more than the idle CUs (see ``deplodock_amd.emit.splitk``).  A ``b<n>`` / ``r<n>`` pin is a row kernel's.
    body.reduce = ReducePlan()
    pinned_reduce = _pin("REDUCE", tuned)
    if auto_split > 1 and not pinned_reduce and stage.transport in ("dl", "dlm", "sync"):
        body.reduce = ReducePlan(cta=auto_split, finalize="kernel")
        knobs["REDUCE"] = body.reduce.spell()
    if pinned_reduce:
        try:
            rp = ReducePlan.parse(pinned_reduce)
            if rp.cta > 1:
                if body.gate_pair or body.a_prologue is not None or body.row_epilogue is not None or getattr(body, "batch", 1) > 1:
                    raise ScheduleError("a cross-workgroup split takes a plain single contraction (no gate/up pair, row prologue, row epilogue or batch)")
                if body.k % rp.cta or (body.k // rp.cta) % plan.bk_elems:
                    raise ScheduleError(f"K={body.k} does not split into {rp.cta} slices of whole {plan.bk_elems}-deep slabs")
                if stage.transport in ("ks", "mix"):
                    body.stage = stage = Stage(depth=2, transport="sync", reg_depth=2 if body.k // rp.cta // plan.bk_elems >= 3 else 1)
                    knobs["STAGE"] = stage.spell()
                if stage.transport in ("dl", "dli", "dlm") and ((plan.bk_elems // plan.atom.frag_k) % 2 or plan.bk_elems % plan.atom.frag_k):
                    raise ScheduleError("direct-to-LDS staging needs an even number of MFMA steps per slab")
                body.reduce = ReducePlan(cta=rp.cta, finalize=rp.finalize)
                knobs["REDUCE"] = body.reduce.spell()
        except ScheduleError as exc:
            logger.warning("EMMY_REDUCE=%r ignored for the contraction: %s", pinned_reduce, exc)
    return knobs


def _flash_lds(body: Flash, ctx: Context) -> int:
    from deplodock_amd.emit.flash import lds_plan

    return lds_plan(body.waves, body.kv_split, body.block_kv, body.head_dim, ctx.lds_bytes_per_cu, deep=body.deep)["bytes"]


def schedule_flash(body: Flash, ctx: Context) -> dict:
    """``EMMY_FLASH=w<row groups>/kv<keys per block>/s<key split>[/p][/k3]``.

    ``/k3`` (a pin only): a K ring of three slots, K blocks requested two steps ahead and a step's end waiting for
    the next V block alone.  Measured slower on the benchmark shape (S=2048, ``w2/kv32/s4/p``: 27.9 -> 31.8 us; the
    ring takes the whole LDS, so the Q fragments come from global memory).

    Default: eight waves per workgroup, two per SIMD — four 32-row groups x two
    key-split wave groups on 64-key blocks (``w4/kv64/s2``) when that many rows per
    workgroup still cover the CUs, else two (or one) row groups x four key-split
    groups on 32-key blocks.  A long causal self-attention whose mirrored
    query-block pairs (``/p``: block b then block n-1-b in one workgroup, equal
    key work for every workgroup) still cover the CUs is paired; below 2048 keys the
    second prologue and close of a pair cost more than the balance gains.
    Measured with 16 q / 8 kv heads of 128 (us, best three): S=512 ``w2/kv32/s4``
    8.7, ``w1/kv32/s4`` 8.8, ``w2/kv64/s2`` 11.0; S=1024 ``w2/kv32/s4`` 13.5,
    ``w1/kv32/s4/p`` 17.8; S=2048 ``w2/kv32/s4/p`` 27.8, ``w2/kv32/s4`` 28.5,
    ``w4/kv64/s2`` 32.7; S=2048 unmasked ``w4/kv64/s2`` 36.5, ``w4/kv32/s2`` 41.3;
    32 q heads S=4096 ``w4/kv64/s2/p`` 157, ``w2/kv32/s4/p`` 186.
    Where 256-row workgroups still cover the CUs they win (``w8/kv64/s1``: S=8192 unmasked
    560 against 637 for ``w4/kv64/s2``, causal 303 against 351; S=16384 causal 1087 / 1239;
    batch 4 S=2048 causal ``w8/kv64/s1/p`` 104 / 117; 16 heads S=4096 causal, 256 such
    workgroups unpaired: 122 against 94, hence the 2x cover asked of an unpaired triangle)."""
    from deplodock_amd.emit.flash_f32 import on_f32_atoms

    if on_f32_atoms(body):
        return _schedule_flash_f32(body, ctx)
    pinned = _pin("FLASH", _tuned(body, ctx))
    if pinned:
        try:
            body.pair = body.deep = body.ws = body.sp = body.mfma_sum = body.private = False
            for tok in pinned.split("/"):
                if tok == "pv":
                    body.private = True
                elif tok == "p":
                    body.pair = True
                elif tok == "ms":
                    body.mfma_sum = True
                elif tok == "ws":
                    body.ws = True
                elif tok == "sp":
                    body.sp = True
                elif tok == "k3":
                    body.deep = True
                elif tok.startswith("w"):
                    body.waves = int(tok[1:])
                elif tok.startswith("kv"):
                    body.block_kv = int(tok[2:])
                elif tok.startswith("s"):
                    body.kv_split = int(tok[1:])
                else:
                    raise ScheduleError(f"cannot parse {tok!r} (expect w<groups> / kv<keys> / s<split> / p / k3 / ms / ws / sp / pv)")
            if body.ws and body.sp:
                raise ScheduleError("ws and sp are two forms: pin one")
            if body.private:
                from deplodock_amd.emit.flash_pv import max_key_split as pv_max_split
                from deplodock_amd.emit.flash_pv import pv_supported

                why = pv_supported(body)
                if why is not None:
                    raise ScheduleError(f"the key-split-waves form needs {why}")
                if body.waves != 1 or body.block_kv != 32 or body.kv_split not in (2, 4, 8) or body.kv_split > pv_max_split(body.head_dim, ctx.lds_bytes_per_cu) or body.pair or body.deep or body.ws or body.sp or body.mfma_sum:
                    raise ScheduleError("the key-split-waves form is w1/kv32/s<2|4|8>/pv within the LDS")
            if body.ws or body.sp:
                from deplodock_amd.emit.flash_ws import ws_supported

                body.block_kv = 32
                why = ws_supported(body, ctx)
                if why is not None:
                    raise ScheduleError(f"the software-pipelined forms need {why}")
            chunks = body.block_kv * body.head_dim // 8
            if body.waves < 1 or body.kv_split < 1 or body.block_kv % 32 or (not (body.ws or body.sp or body.private) and chunks % (body.waves * body.kv_split * 64)):
                raise ScheduleError("unrealisable workgroup shape")
            if not (body.ws or body.sp or body.private) and _flash_lds(body, ctx) > ctx.lds_bytes_per_cu:
                raise ScheduleError("the double-buffered K/V blocks of all key-split groups exceed the LDS")
            if (body.head_dim // 32 * 16) % (4 * body.kv_split):
                raise ScheduleError("the key-split groups cannot share a lane's output registers")
            if body.pair and not (body.causal and -(-body.q_len // (32 * body.waves)) % 2 == 0):
                raise ScheduleError("pairing mirrored query blocks needs a causal mask and an even block count")
        except (ValueError, ScheduleError) as exc:
            logger.warning("EMMY_FLASH=%r ignored: %s", pinned, exc)
            pinned = None
    if not pinned:
        heads = body.batch * body.q_heads
        fill = _FILL_FRACTION * ctx.compute_units

        def blocks(w: int) -> int:
            return -(-body.q_len // (32 * w))

        body.pair = body.deep = body.ws = body.sp = body.private = False
        body.waves = 0
        if body.head_dim <= 128 and body.kv_len >= 2048:
            # Enough rows to give every CU a 256-row workgroup: eight query waves share each
            # K/V block (the blocks come out of the L2s at ~32 B/clk per CU whoever asks, so rows
            # per block is what counts) and no key split is needed to put two waves on a SIMD.
            cus = ctx.compute_units
            if body.causal and body.q_len == body.kv_len:
                if body.kv_len <= 4096 and blocks(8) % 2 == 0 and heads * blocks(8) // 2 >= cus:
                    body.waves, body.pair = 8, True
                elif heads * blocks(8) >= 2 * cus:
                    body.waves = 8  # twice the CUs: the heaviest-first order balances the triangle
            elif heads * blocks(8) >= cus:
                body.waves = 8
        if not body.waves and body.causal and body.q_len == body.kv_len and body.kv_len >= 2048:
            for w in (4, 2):
                if blocks(w) % 2 == 0 and heads * blocks(w) // 2 >= fill:
                    body.waves, body.pair = w, True
                    break
        if not body.waves:
            # (two row groups pay down to half the CUs: 512 tokens x 16 heads, 128 workgroups of `w2` 8.81 us, 256 of `w1` 9.10;
            # and wherever there are more than two of their 64-row blocks, however few the workgroups: they share each K / V
            # block's way into the LDS: 160 / 192 / 384 tokens x 16 heads 6.15 / 6.16 / 7.32 us against 6.42 / 6.45 / 7.48)
            body.waves = next((w for w in (4, 2) if heads * blocks(w) >= (fill if w == 4 else 0.5 * ctx.compute_units) or (w == 2 and blocks(2) > 2)), 1)
        body.block_kv, body.kv_split = {8: (64, 1), 4: (64, 2)}.get(body.waves, (32, 4))
        while body.kv_split > 1 and -(-body.kv_len // body.block_kv) <= body.kv_split // 2:
            body.kv_split //= 2  # half the key-split groups would have no block (three blocks keep four groups: 96 keys 4.71 us, two groups 6.05)
        # wider heads: shrink the key block, then the key split, until the double-buffered K/V blocks fit the LDS
        while _flash_lds(body, ctx) > ctx.lds_bytes_per_cu:
            if body.block_kv > 32:
                body.block_kv //= 2
            elif body.kv_split > 1:
                body.kv_split //= 2
            else:
                break
        # narrower heads: a key block's 16-byte chunks are dealt over all threads of the workgroup, so it must
        # hold at least one chunk per thread: grow the block while the LDS allows, else give up key-split groups
        while (body.block_kv * body.head_dim // 8) % (body.waves * body.kv_split * 64):
            body.block_kv *= 2
            if _flash_lds(body, ctx) > ctx.lds_bytes_per_cu:
                body.block_kv //= 2
                if body.kv_split == 1:
                    break
                body.kv_split //= 2
    if getattr(body, "sym", None) is not None and body.sym.fields:
        body.pair = False  # pairing mirrored query blocks needs the block count when the kernel is built
    if body.private:
        body.kv_ctas = 1
        return {"FLASH": f"w1/kv32/s{body.kv_split}/pv"}
    knobs = _schedule_flash_split(body, ctx, tuned if (tuned := _tuned(body, ctx)) else None)
    return {**knobs, "FLASH": f"w{body.waves}/kv{body.block_kv}/s{body.kv_split}" + ("/p" if body.pair else "") + ("/k3" if body.deep else "") + ("/ws" if body.ws else "") + ("/sp" if body.sp else "")}


#: the key-split fp32 attention form runs its software-pipelined order unless pinned ``/np``
_F32_PIPELINED = False


def _schedule_flash_f32(body: Flash, ctx: Context) -> dict:
    """``EMMY_FLASH=f32/w<row groups>`` or ``f32/s<key-split waves>``.

    ``w<n>``: 1, 2 or 4 groups of 32 query rows per 256-thread workgroup share each K / V block (the other waves only stage).
    ``s<k>``: one group of 32 rows per workgroup whose 2, 4 or 8 waves split the key blocks and stage for themselves.
    ``s<k>/o``: the same with a wave's K and V blocks taking turns in one LDS region — half the LDS a wave, two waves a SIMD.
    ``s<k>/sp``: the software-pipelined order (a tie, kept as a pin).
    Default: the one-region key-split form wherever rows are whole aligned pairs of 16-byte chunks of at most 128 values —
    eight waves where a row group has eight key blocks and more and the launch is under four workgroups per CU, else four
    (measured, 16 / 8 heads of 128, causal, us, ``w4`` / ``s2`` / ``s4`` / ``s4/o`` / ``s8/o``: S=128 25.1 / 15.1 / 11.2 /
    10.6 / 12.1, 512: 82.5 / 44.2 / 26.4 / 24.9 / 24.7, 1024: 159 / 84.7 / 56.3 / 74.8 / 52.8, 2048: 313 / 180 / 193 / 179 /
    182, 4096: 713 / 699 / 711 / 621 / 664, 8192: 2625 / 2562 / 2641 / 2255 / 2351) — except for a single key block,
    where there is nothing to split (S=32: 7.4 against 9.9); else the most row groups that still give every CU a
    workgroup."""
    from deplodock_amd.emit.flash_f32 import max_key_split, whole_chunk_rows

    body.pair = body.deep = body.ws = body.sp = body.mfma_sum = False
    body.kv_ctas, body.block_kv = 1, 32
    heads = body.batch * body.q_heads
    can_split = body.dtype.name == "f32" and all(whole_chunk_rows(body)) and body.head_dim % 8 == 0
    most = max_key_split(body.head_dim, ctx.lds_bytes_per_cu, one_region=True) if can_split else 1
    symbolic = getattr(body, "sym", None) is not None and bool(body.sym.fields)
    body.one_region = False
    if most > 1 and (body.kv_len > 32 or symbolic):
        wide = most >= 8 and (symbolic or body.kv_len >= 8 * 32) and heads * -(-body.q_len // 32) < 4 * ctx.compute_units
        body.waves, body.kv_split, body.one_region = 1, (8 if wide else min(4, most)), True
    else:
        body.waves, body.kv_split = next((w for w in (4, 2) if heads * -(-body.q_len // (32 * w)) >= ctx.compute_units), 1), 1
    pinned = _pin("FLASH", _tuned(body, ctx))
    body.sp = body.kv_split > 1 and _F32_PIPELINED and not body.one_region
    if pinned and pinned.split("/")[0] == "f32":
        try:
            tok, *rest = pinned.split("/")[1:]
            n = int(tok[1:])
            if rest not in ([], ["sp"], ["np"], ["o"]):
                raise ValueError(rest)
            if tok[0] == "w" and n in (1, 2, 4) and not rest:
                body.waves, body.kv_split, body.sp, body.one_region = n, 1, False, False
            elif tok[0] == "s" and n in (2, 4, 8) and can_split and n <= max_key_split(body.head_dim, ctx.lds_bytes_per_cu, rest == ["o"]):
                body.waves, body.kv_split = 1, n
                body.sp = rest == ["sp"] or (not rest and _F32_PIPELINED)
                body.one_region = rest == ["o"]
            else:
                raise ValueError(tok)
        except ValueError:
            logger.warning("EMMY_FLASH=%r ignored: expect f32/w1, f32/w2, f32/w4 or f32/s2, f32/s4, f32/s8[/sp|/o] (rows of whole 16-byte chunks, regions within the LDS)", pinned)
    flash = (f"f32/s{body.kv_split}" + ("/sp" if body.sp else "") + ("/o" if body.one_region else "")) if body.kv_split > 1 else f"f32/w{body.waves}"
    knobs: dict = {}
    if body.kv_split > 1 and body.dtype.name == "f32" and not body.causal and body.mask is None and not symbolic and body.head_dim % 4 == 0:
        # decode-size queries over a long cache: the keys are also split across workgroups (partial kernel + combine)
        knobs = _schedule_flash_split(body, ctx, tuned if (tuned := _tuned(body, ctx)) else None)
    elif _pin("REDUCE", _tuned(body, ctx)):
        logger.warning("EMMY_REDUCE ignored for this fp32 attention: the cross-workgroup key split takes the key-split form without masks or symbolic lengths")
    return {**knobs, "FLASH": flash}


def _schedule_flash_split(body: Flash, ctx: Context, tuned: dict | None, min_keys: int = 256) -> dict:
    """``REDUCE=g<n>[k]`` on attention: ``n`` workgroups per query block split the keys and a combine kernel merges their
    ``(m, l, O)`` (the reference's cross-CTA finalize of the twisted carrier is kernel-only, tests/compiler/e2e/
    test_reduce_coverage.py:280-315; ``g<n>a`` is taken as ``g<n>k``).  Unpinned: where the query blocks cover less than
    half the CUs and the keys are long — decode-size queries over a long cache — the keys are split until the launch covers
    the CUs, in slices of at least ``min_keys`` keys (us, slices of 256 against 512 keys: one bf16 query over 2 048 / 4 096 keys
    7.98 / 9.16 against 9.92 / 10.20, 16 queries over 4 096 keys 9.94 against 10.44; in fp32 19.1 against 26.5)."""
    body.kv_ctas = 1
    plain = body.mask is None and not (getattr(body, "sym", None) is not None and body.sym.fields) and not (body.ws or body.sp)
    pinned = _pin("REDUCE", tuned)
    n = 1
    if pinned:
        try:
            plan = ReducePlan.parse(pinned)
            if plan.cta > 1:
                if not plain:
                    raise ScheduleError("the cross-workgroup key split takes no mask operand, symbolic lengths or software-pipelined form")
                if plan.finalize == "atomic":
                    logger.warning("EMMY_REDUCE=%r: the (m, l, O) carrier has no atomic finalize: g%dk instead", pinned, plan.cta)
                n = plan.cta
        except ScheduleError as exc:
            logger.warning("EMMY_REDUCE=%r ignored for attention: %s", pinned, exc)
    elif plain and not body.causal:
        groups = body.batch * body.q_heads * -(-body.q_len // (32 * body.waves))
        if 2 * groups <= ctx.compute_units and body.kv_len >= 2048:
            n = 1
            while n < 16 and groups * n * 2 <= ctx.compute_units and body.kv_len // (2 * n) >= min_keys:
                n *= 2
    if n > 1:
        step = body.kv_split * body.block_kv
        chunk = -(-(-(-body.kv_len // n)) // step) * step
        n = -(-body.kv_len // chunk)
    if n > 1:
        body.kv_ctas, body.pair = n, False
        return {"REDUCE": f"g{n}k"}
    return {}


def schedule(graph: Graph, ctx: Context | None = None) -> Graph:
    """Stamp a plan on every ``TileOp`` in ``graph`` (in place) and return it."""
    ctx = ctx or Context()
    for node in graph.nodes.values():
        op = node.op
        if not isinstance(op, TileOp):
            continue
        body = op.body
        if isinstance(body, RowReduce):
            op.knobs.update(schedule_row_reduce(body, ctx))
        elif isinstance(body, Contraction):
            op.knobs.update(schedule_contraction(body, ctx))
        elif isinstance(body, Flash):
            op.knobs.update(schedule_flash(body, ctx))
        elif isinstance(body, (Map, LoopNest, StridedCopy, IndexRows)):
            pass  # nothing to plan: a map is sized by its extent, a loop nest by its outer loops
        else:
            raise TypeError(f"unknown tile body {type(body).__name__}")
    return graph
