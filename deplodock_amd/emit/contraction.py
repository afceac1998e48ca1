"""MFMA contraction emitter: ``out[m, n] = epilogue(sum_k a[m, k] * b[n, k])``.

Replaces the reference's warp-MMA contraction (``_MmaOps``, ``_contract_kloop``
and ``_staged`` in emmy/compiler/pipeline/passes/lowering/kernel/_atom.py:397-715,
the cp.async ring of _stage.py:400-450, ``LdmatrixLoad`` / ``MmaSyncPtx`` /
``RegStore`` in emmy/compiler/ir/kernel/ir.py:1076-1529).  The design is for
CDNA4, not a translation:

* **Operand roles are swapped** relative to the math: the weight tile (rows =
  output features ``n``) feeds the MFMA *A* port and the activation tile (rows
  = ``m``) the *B* port, so the fp32 accumulator fragment holds, per lane, four
  *consecutive n* of one output row ``m``.  The epilogue therefore packs and
  stores 8-byte bf16x4 runs straight from registers — no shared-memory
  transpose, no 2-byte scatter.
* Both operands are K-contiguous in memory, which is exactly what an MFMA lane
  wants (8 consecutive k of one row = one 16-byte chunk), so LDS holds plain
  row-major slabs and fragments are single ``ds_read_b128``.
* LDS slabs are XOR-swizzled at 16-byte granularity so the 16 rows a quarter
  wave reads of one k-chunk land in 16 distinct 16-byte bank groups (64 banks).
* ``STAGE=d<n>/sync`` software-pipelines global → VGPR → LDS one slab ahead
  with one barrier per slab; ``STAGE=d<n>/dl`` issues global loads that write
  LDS directly (no VGPR hop), ``n - 1`` slabs ahead.
* Workgroup ids are remapped so the 8 XCDs (hardware round-robins consecutive
  ids over them) each own a compact block of output tiles and keep their
  operand rows in their own L2.
"""

from __future__ import annotations

from deplodock_amd.context import Context
from deplodock_amd.dtype import BF16, F16, F32
from deplodock_amd.emit import prelude
from deplodock_amd.render_target import rt
from deplodock_amd.emit.errors import LoweringError
from deplodock_amd.ir import expr as E
from deplodock_amd.ir.hip import HipOp
from deplodock_amd.ir.schedule import Stage
from deplodock_amd.ir.sym import XcdRounds, c_value, param_name
from deplodock_amd.ir.tile import Contraction



def _frag_t(dtype_name: str) -> str:
    """The 16-byte MFMA operand fragment (eight 16-bit elements) of ``dtype_name``."""
    return rt.vector_type(dtype_name, 8)[0]


def _pack4_t(dtype_name: str) -> str:
    """Four consecutive output elements, the run an accumulator group converts to."""
    return rt.vector_type(dtype_name, 4)[0]


def xcd_block(tiles_m: int, tiles_n: int, tile_m: int, tile_n: int, xcds: int) -> tuple[int, int]:
    """Shape ``(gm, gn)`` of the tile block one XCD owns: ``gm*gn`` as close to
    ``tiles/xcds`` as the grid allows, minimising operand rows touched
    (``gm*tile_m + gn*tile_n``) so the block's working set fits its L2."""
    per = max(1, (tiles_m * tiles_n) // xcds)
    best = None
    for gm in range(1, tiles_m + 1):
        if tiles_m % gm:
            continue
        gn = max(1, min(tiles_n, per // gm))
        while gn > 1 and tiles_n % gn:
            gn -= 1
        if gm * gn > per and not (gm == 1 and gn == 1):
            continue
        cost = (gm * tile_m + gn * tile_n, -(gm * gn))
        if best is None or (-(gm * gn), cost[0]) < (-(best[0] * best[1]), best[2]):
            best = (gm, gn, cost[0])
    return (best[0], best[1]) if best else (1, 1)


def _emit_row_epilogue_tables(a, re, re_args: list[str], EPC: int, m_guard: bool, mods: list | None = None) -> None:
    """Fetch, at kernel start, the table chunks the row epilogue of this thread will
    need (they depend on the output coordinates only): the k loop hides the latency."""
    d = re.cols
    vt_chunk = rt.vector_type(re.row_operands[0].dtype.name if re.row_operands else "bf16", EPC)[0]
    a(f"  constexpr int RE_IT = (TM * (TN / {EPC})) / T;")
    for nm, ro in zip(re_args, re.row_operands):
        a(f"  {vt_chunk} {nm}_v[RE_IT];")
    a(f"  if (n0 < {re.col_end}) {{")
    a("    #pragma unroll")
    a("    for (int it = 0; it < RE_IT; ++it) {")
    a(f"      const int q = tid + it * T, row = q / (TN / {EPC}), cc = q % (TN / {EPC});")
    a(f"      const int m = m0 + row, n = n0 + cc * {EPC}, gc = n % {d};")
    mrow = "(m < M ? m : M - 1)" if m_guard else "m"
    a(f"      const long rr = (long){mrow} * {re.col_end // d} + n / {d};  // the row number a separate row kernel would use")
    for i_, (nm, ro) in enumerate(zip(re_args, re.row_operands)):
        mod = c_value(mods[i_]) if mods is not None else str(ro.mod)
        a(f"      const {rt.type_name(ro.dtype.name)}* {nm}_row = {nm} + {ro.offset}L + ((rr / {ro.div}) % {mod}) * {d};")
        a(f"      {nm}_v[it] = *(const {vt_chunk}*)({nm}_row + gc);")
    a("    }")
    a("  }")


def _emit_row_epilogue(a, body: Contraction, re, re_args: list[str], EPC: int, vt_chunk: str, out_c: str, m_guard: bool, n_guard: bool) -> None:
    """The store loop of the tiles that hold row-epilogue columns: every thread
    owns one 16-byte chunk of an output row at a time; the ``HC`` threads that
    share a column group are consecutive lanes, so the group statistic is a
    butterfly over them, and the half-rotated partner chunk is read from the tile
    in LDS.  Leaves the ``else`` of the tile test open for the plain store loop."""
    d = re.cols
    HC = d // EPC
    if HC & (HC - 1) or HC > 32 or HC < 2:
        raise LoweringError(f"contraction: row-epilogue groups of {d} columns do not map onto lanes")
    stat_names = [st.name for st in re.stats]
    op_names = [ro.name for ro in re.row_operands]
    for st in re.stats:
        if E.variables(st.pre) - {"x"} or st.monoid not in ("sum", "max") or st.keep:
            raise LoweringError(f"contraction: row-epilogue statistic {st.name!r} is not a plain sum/max over the group")
    in_project = E.variables(re.project)
    in_rotate = E.variables(re.rotate.expr) if re.rotate is not None else set()
    unknown = (in_project - ({"x"} | set(stat_names) | set(op_names))) | (in_rotate - ({"y", "yr"} | set(stat_names) | set(op_names)))
    if unknown:
        raise LoweringError(f"contraction: row epilogue uses unknown names {sorted(unknown)}")
    cast = "" if body.out_dtype is F32 else f"({out_c})"
    a(f"  if (n0 < {re.col_end}) {{  // tiles of column groups that take the row epilogue")
    a(r"""  #pragma unroll
  for (int it = 0; it < (TM * CPRC) / T; ++it) {
    const int q = tid + it * T;
    const int row = q / CPRC, cc = q % CPRC;""")
    a(f"    const int m = m0 + row, n = n0 + cc * {EPC};")
    a(f"    const {vt_chunk} xv = *(const {vt_chunk}*)(emh_lds + row * CSTRIDE + cc * 16);")
    for st in re.stats:
        ident = "0.0f" if st.monoid == "sum" else "-__builtin_inff()"
        a(f"    float {st.name} = {ident};")
        a("    #pragma unroll")
        a(f"    for (int r = 0; r < {EPC}; ++r) {{ const float x_ = (float)xv[r]; const float t_ = {E.render(st.pre, {'x': 'x_'})}; {st.name} = " + (f"{st.name} + t_" if st.monoid == "sum" else f"fmaxf({st.name}, t_)") + "; }")
        a(f"    {st.name} = emh_wave_reduce<{prelude.MONOID_STRUCT[st.monoid]}, {HC}>({st.name});  // the group's chunks sit in {HC} consecutive lanes")
    env_stats = {n_: n_ for n_ in stat_names}
    if re.rotate is None:
        a(f"    {vt_chunk} yo;")
        a("    #pragma unroll")
        a(f"    for (int r = 0; r < {EPC}; ++r) {{")
        env = dict(env_stats, x="(float)xv[r]", **{ro.name: f"(float){nm}_v[it][r]" for nm, ro in zip(re_args, re.row_operands)})
        a(f"      yo[r] = {cast}({E.render(re.project, env)});")
        a("    }")
    else:
        # The half-rotated partner of a chunk is the chunk HC/2 further on in the same group,
        # i.e. the projected values of the lane HC/2 away: fetched across lanes, not recomputed.
        fetch = "emh_dpp<0x128>(yv[r])" if HC == 16 else f"__shfl_xor(yv[r], {HC // 2}, 64)"  # row_ror:8 inside a 16-lane row
        a(f"    const float sgn = (cc % {HC}) < {HC // 2} ? -1.0f : 1.0f;")
        a(f"    float yv[{EPC}];")
        a("    #pragma unroll")
        env_own = dict(env_stats, x="(float)xv[r]", **{ro.name: f"(float){nm}_v[it][r]" for nm, ro in zip(re_args, re.row_operands) if ro.name in in_project})
        a(f"    for (int r = 0; r < {EPC}; ++r) yv[r] = {E.render(re.project, env_own)};")
        a(f"    {vt_chunk} yo;")
        a("    #pragma unroll")
        a(f"    for (int r = 0; r < {EPC}; ++r) {{")
        a(f"      const float yr_ = sgn * {fetch};")
        env_rot = dict(env_stats, y="yv[r]", yr="yr_", **{ro.name: f"(float){nm}_v[it][r]" for nm, ro in zip(re_args, re.row_operands) if ro.name in in_rotate})
        a(f"      yo[r] = {cast}({E.render(re.rotate.expr, env_rot)});")
        a("    }")
    conds = (["m < M"] if m_guard else []) + (["n < N"] if n_guard else [])
    a(f"    if ({' && '.join(conds) if conds else 'true'}) *({vt_chunk}*)(O + {body.out_offset}L + (long)m * LDO + n) = yo;")
    a("  }")
    a("  } else {")


PP_PRODUCER_THREADS = 256  # the four request-issuing waves of STAGE .../pp (one per SIMD)


def _emit_pingpong_loop(a, *, KT: int, KS: int, depth: int, parts: list[str]) -> None:
    """The k loop of ``STAGE .../pp``: twelve waves, three on every SIMD, in three roles, one workgroup barrier a slab.

    Waves 0-3 and 4-7 (one of each on every SIMD; every wave owns its own part of the output tile) are two
    *consumer* groups that run half a slab apart.  In period j group 0 issues the MFMAs of slab j (at raised
    priority) and then reads slab j + 1's fragments into registers; group 1 first reads slab j's fragments and
    then issues its MFMAs.  So while one wave of a SIMD computes, the other reads, and LDS latency is paid by the
    wave with nothing to compute.  Waves 8-11 are *producers*: they issue every direct-to-LDS request (``parts``:
    the statements of one slab's requests of a producer thread, format strings over ``slab`` and ``buf``), wait
    for them in issue order and publish them.  A request blocks its wave at issue while the memory pipeline is
    full — which, with operands streaming from L2 at the rate this tile needs them, is most of the time; on a
    producer wave that costs nothing, on a consumer it would stall the MFMAs queued behind it.

        period j   group 0: MFMAs of slab j, read slab j + 1     group 1: read slab j, MFMAs of slab j
                   producers: request slab j + DEPTH - 1 (into the buffer of slab j - 1, whose last reader, group 1
                   in period j - 1, is done), then wait until slab j + 2 is complete and publish it;  barrier.

    Slab j + 1 is read inside period j, so it has to be complete at the barrier that *starts* the period: a slab
    requested in period q is waited for at the end of period q + DEPTH - 3, which needs DEPTH >= 4 to leave it
    more than the rest of its own period.

    (A wave gets about 32 bytes a clock out of LDS and issues in order, so group 1's MFMAs start some 400 clocks
    into the period, when group 0 is about done with its own.  Moving part of the reads between the MFMAs, in
    either group, measured slower: a read that blocks at issue holds back the MFMAs behind it.)"""
    R = depth

    def request(q: str) -> None:
        for st in parts:
            a("      " + st.format(slab=f"(({q}) + {R - 1})", buf=f"((({q}) + {R - 1}) % DEPTH)"))

    def fetch(j: str) -> None:
        for kk in range(KS):
            a(f"      EMH_READ({kk}, ({j}) % DEPTH, {kk});")

    def compute() -> None:
        a("      __builtin_amdgcn_s_setprio(1);")
        for kk in range(KS):
            a(f"      EMH_MMA({kk});")
        a("      __builtin_amdgcn_s_setprio(0);")

    def allowed(q: int) -> int:
        """Requests a producer thread may still have outstanding at the end of period q (-1: the period before
        the first) with every slab up to q + 2 complete: what it issued after slab q + 2 (they retire in order)."""
        last = min(q + R - 1, KT - 1) if q >= 0 else min(R - 2, KT - 1)
        return max(0, last - (q + 2)) * len(parts)

    a("  // a period ends when every wave is here")
    a('  #define EMH_PHASE_END() { asm volatile("" ::: "memory"); __builtin_amdgcn_s_barrier(); asm volatile("" ::: "memory"); }')
    steady = max(0, KT - R + 1)  # periods q for which slab q + R - 1 exists
    a("  if (role == 2) {  // ---- producers")
    a(f"    EMH_SLAB_SYNC({allowed(-1)});  // period -1")
    if steady:
        a(f"    for (int kt = 0; kt < {steady}; ++kt) {{")
        request("kt")
        a(f"      EMH_SLAB_SYNC({allowed(0)});")
        a("    }")
    for q in range(steady, KT):
        a(f"    EMH_SLAB_SYNC({allowed(q)});")
    a("  } else if (role == 0) {  // ---- consumer group 0")
    a("    {")
    fetch("0")
    a("      EMH_PHASE_END(); }  // period -1")
    a(f"    for (int kt = 0; kt < {KT}; ++kt) {{")
    compute()
    a("      EMH_STAMP_AT(0)  // this group's MFMAs issued")
    a(f"      if (kt + 1 < {KT}) {{")
    fetch("kt + 1")
    a("      }")
    a("      EMH_STAMP_AT(1)  // the next slab's fragment reads issued")
    a("      EMH_PHASE_END();")
    a("      EMH_STAMP_AT(2)  // the period's barrier")
    a("    }")
    a("  } else {  // ---- consumer group 1")
    a("    EMH_PHASE_END();  // period -1")
    a(f"    for (int kt = 0; kt < {KT}; ++kt) {{")
    fetch("kt")
    compute()
    a("      EMH_PHASE_END();")
    a("    }")
    a("  }")


#: fraction of the last step's MFMAs the ``dlm`` requests are spread over, and of a step's MFMAs the next step's fragment reads are
_SPREAD = 1.0
_READ_SPREAD = 0.5


def emit_contraction(body: Contraction, name: str, ctx: Context = Context()) -> HipOp:
    plan = body.tile
    if plan is None:
        raise LoweringError("contraction: no TilePlan stamped")
    if body.in_dtype.name not in ("bf16", "f16", "f32") or plan.atom.dtype != body.in_dtype.name:
        raise LoweringError(f"contraction: atom {plan.atom.name} does not take {body.in_dtype} operands")
    ES = body.in_dtype.nbytes  # operand element size
    EPCK = 16 // ES  # operand elements per 16-byte chunk (what a lane's fragment read fetches: consecutive k of one row)
    fp32_tier = body.in_dtype is F32
    if fp32_tier and (body.a_prologue is not None or body.gate_pair or body.row_epilogue is not None):
        raise LoweringError("contraction: row prologues, gate/up pairs and row epilogues are written for 16-bit operands")
    stage = body.stage or Stage(depth=2, transport="sync")
    if stage.transport == "ks":
        from deplodock_amd.emit.skinny import emit_contraction_skinny

        return emit_contraction_skinny(body, name, ctx)
    if body.reduce.cta != 1:
        raise LoweringError("contraction: a cross-workgroup split (REDUCE=g<n>) is lowered as a partial kernel plus a combine (deplodock_amd.emit.splitk.lower_split_contraction), not by this emitter alone")
    split = body.k_split
    batch = int(getattr(body, "batch", 1) or 1)
    if batch > 1:
        if split is not None or body.bias is not None or body.a_prologue is not None or body.row_epilogue is not None or body.epilogue_operands or body.gate_pair:
            raise LoweringError("contraction: a batch of products takes plain products only (no split, bias, prologue, row epilogue, epilogue operands or gate pair)")
        if batch > 65535:
            raise LoweringError(f"contraction: {batch} products exceed the launch's second dimension")
        if (body.a_batch * ES) % 16 or (body.b_batch * ES) % 16 or body.out_batch % 4:
            raise LoweringError("contraction: batch strides must keep 16-byte operand alignment and whole 4-element output runs")
    if split is not None:
        if body.epilogue is not None or body.post is not None or body.bias is not None or body.gate_pair or body.a_prologue is not None or body.row_epilogue is not None or body.out_dtype is not F32:
            raise LoweringError("contraction: the partial kernel of a split stores bare fp32 accumulators; bias, epilogue and rounding belong to the combine")
        if stage.transport not in ("sync", "dl", "dli", "dlm", "pp"):
            raise LoweringError(f"contraction: STAGE .../{stage.transport} does not combine with a cross-workgroup split")
    M, N, K = body.m, body.n, body.k
    lda = body.lda or K
    ldb = body.ldb or K
    ldo = body.ldo or N
    AM = plan.atom.m  # 32 or 16 (square atoms)
    KG = 64 // AM  # lane groups along k
    # k per fragment read: every lane fetches one 16-byte chunk, the KG lane groups of a row fetch neighbouring chunks.
    # A 16-bit atom consumes that in one MFMA (atom.k = 8 * KG); an fp32 atom takes one element of the chunk per MFMA
    # (atom.k = KG: lane group g feeds k = g), so a fragment feeds four MFMAs, element e of every lane's chunk in MFMA e —
    # a contraction does not care in which order its k terms are paired, as long as both operands use the same one.
    KSTEP = EPCK * KG
    MPF = KSTEP // plan.atom.k  # MFMAs per fragment pair
    if KSTEP % plan.atom.k or MPF not in (1, EPCK):
        raise LoweringError(f"contraction: atom {plan.atom.name} does not consume 16-byte k chunks")
    ACC = plan.atom.acc_per_lane
    WM, WN = plan.units
    FM, FN = plan.regs
    TM, TN = plan.tile_m, plan.tile_n
    BK = plan.bk_elems
    T = plan.block_threads
    k_guard = K % BK != 0  # the last slab is short: its missing chunks are staged as zeros (both operands)
    if k_guard and (K % EPCK or body.a_prologue is not None or stage.transport != "sync"):
        raise LoweringError(f"contraction: K={K} is not a multiple of the slab depth {BK} (a short last slab needs whole 16-byte chunks, register staging and no row prologue)")
    if BK % EPCK or BK * ES > 512:
        raise LoweringError(f"contraction: slab depth {BK} must be whole 16-byte chunks and at most 512 bytes a row")
    if lda % EPCK or ldb % EPCK or ldo % 4 or body.a_offset % EPCK or body.b_offset % EPCK or body.out_offset % 8:
        raise LoweringError("contraction: leading dimensions must keep 16-byte operand / 8-byte output alignment")
    CPR = BK // EPCK  # 16-byte chunks per slab row
    if CPR & (CPR - 1):
        raise LoweringError(f"contraction: slab depth {BK} must give a power-of-two chunk count")
    RPL = max(1, 16 // CPR)  # slab rows per 256-byte bank line
    gate = body.gate_pair
    NB = 2 if gate else 1  # weight matrices consumed per pass
    a_chunks = TM * CPR
    b_chunks = TN * CPR * NB
    # STAGE .../pp: the tile's waves compute; four more waves (one per SIMD) do all the staging
    ST = PP_PRODUCER_THREADS if stage.transport == "pp" else T  # threads that stage operands
    TT = T + PP_PRODUCER_THREADS if stage.transport == "pp" else T  # threads launched
    if a_chunks % ST or b_chunks % ST:
        raise LoweringError(f"contraction: tile {TM}x{TN}x{BK} does not divide over {ST} threads")
    A_PER_T, B_PER_T = a_chunks // ST, b_chunks // ST
    slab_bytes = (TM + TN * NB) * BK * ES
    depth = 2 if stage.transport == "mix" else max(2, stage.depth)
    RS = 1 if stage.transport in ("dl", "dli", "dlm", "pp", "mix") else max(1, stage.reg_depth)  # register sets a slab travels through on the sync path
    lds_bytes = slab_bytes * depth
    if lds_bytes > ctx.lds_bytes_per_cu:
        raise LoweringError(f"contraction: {lds_bytes} B of LDS exceeds {ctx.lds_bytes_per_cu} B per CU")
    acc_regs = FM * FN * ACC * NB
    if acc_regs > 384:
        raise LoweringError(f"contraction: {acc_regs} accumulator registers per lane exceed the register file")
    tiles_m, tiles_n = -(-M // TM), -(-N // TN)
    n_tiles = tiles_m * tiles_n
    gm, gn = xcd_block(tiles_m, tiles_n, TM, TN, ctx.xcds)
    KT = -(-K // BK)
    m_guard = M % TM != 0
    # Symbolic row count (``body.sym`` marks ``m`` as ``a * seq_len + b``): M, the tile counts and the launch size
    # become expressions over the kernel's trailing ``int`` parameter, rows are always guarded, and an XCD owns
    # one-tile-row blocks (the compact block shape above is a function of the tile counts).
    sym = getattr(body, "sym", None)
    m_sym = sym.fields.get("m") if sym is not None else None
    if m_sym is not None:
        if split is not None or stage.transport == "ks":
            raise LoweringError("contraction: a symbolic row count does not combine with a cross-workgroup split or the few-row form")
        m_guard = True
        gm = 1
        while tiles_n % gn:
            gn -= 1
    n_guard = N % TN != 0
    dli = stage.transport == "dli"  # direct to LDS, requests issued between the MFMAs of the slab before (see below)
    dlm = stage.transport == "dlm"  # direct to LDS as ``dl``, the steady-state requests spread among the MFMAs of the slab's last step
    pp = stage.transport == "pp"  # direct to LDS, the two waves of a SIMD in opposite phases (one computes, one fetches)
    spec = pp  # specialised waves: the tile's own compute, four more stage
    dl = stage.transport in ("dl", "dli", "dlm", "pp")
    mix = stage.transport == "mix"  # a through registers (it is transformed on the way), b direct to LDS
    if mix and b_chunks % 64:
        raise LoweringError("contraction: direct-to-LDS staging needs whole-wave chunk counts")
    if dl and (a_chunks % 64 or b_chunks % 64):
        raise LoweringError("contraction: direct-to-LDS staging needs whole-wave chunk counts")

    frag_t = rt.vector_type(body.in_dtype.name, EPCK)[0]
    in_c = rt.type_name(body.in_dtype.name)
    out_c = rt.type_name(body.out_dtype.name)
    epi_names = [n for n, _ in body.epilogue_operands]
    epi = body.epilogue if body.epilogue is not None else E.Var("acc")
    allowed = {"acc"} | ({"acc2"} if gate else set()) | ({"bias"} if body.bias is not None else set())
    if body.bias is not None and gate:
        raise LoweringError("contraction: a bias on a gate/up pair is not supported")
    unknown = E.variables(epi) - allowed
    if unknown:
        raise LoweringError(f"contraction epilogue uses unknown names {sorted(unknown)} (operands belong in `post`)")

    pro = body.a_prologue
    deferred = pro is not None and pro.scale is not None
    if deferred and (pro.weight is not None or E.variables(pro.scale) - {"ss"}):
        raise LoweringError("contraction: a deferred row scale is an expression over the row statistic; the column weight belongs in the b operand")
    if pro is not None:
        if dl and not deferred:
            raise LoweringError("contraction: a row prologue transforms the operand in registers; it needs STAGE .../sync")
        if body.in_dtype.nbytes != 2 or (pro.weight is not None and pro.weight_dtype.nbytes != 2):
            raise LoweringError("contraction: the row prologue is written for 16-bit operands")
        bad = (E.variables(pro.stat_pre) - {"x"}) | (set() if deferred else E.variables(pro.project) - ({"x", "ss"} | ({"w"} if pro.weight else set())))
        if bad:
            raise LoweringError(f"contraction: row prologue uses unknown names {sorted(bad)}")
        if CPR > 64:
            raise LoweringError("contraction: a row's slab chunks must sit in one wave for the prologue's row sum")
    params = [f"const {in_c}* __restrict__ A", f"const {in_c}* __restrict__ B"]
    if pro is not None and pro.weight is not None:
        params.append(f"const {rt.type_name(pro.weight_dtype.name)}* __restrict__ NW")
    if body.bias is not None:
        params.append(f"const {rt.type_name(body.bias_dtype.name)}* __restrict__ BIAS")
    params += [f"const {rt.type_name(dt.name)}* __restrict__ e{i}" for i, (_, dt) in enumerate(body.epilogue_operands)]
    rowepi = body.row_epilogue
    re_args = [f"re{i}" for i in range(len(rowepi.row_operands))] if rowepi is not None else []
    if rowepi is not None:
        if body.post is not None or gate or TN % rowepi.cols or rowepi.col_end % TN or rowepi.col_end > N:
            raise LoweringError("contraction: the row epilogue needs a plain result and output tiles of whole column groups")
        params += [f"const {rt.type_name(ro.dtype.name)}* __restrict__ {nm}" for nm, ro in zip(re_args, rowepi.row_operands)]
    params.append(f"{out_c}* __restrict__ O")
    sym_for_params = getattr(body, "sym", None)
    if sym_for_params is not None and sym_for_params.fields:
        params.append(f"int {param_name(sym_for_params.name)}")

    D = dict(
        name=name, T=T, ST=ST, TT=TT, M=M, N=N, K=K, LDA=lda, LDB=ldb, LDO=ldo, TM=TM, TN=TN, BK=BK, WM=WM, WN=WN, FM=FM, FN=FN,
        AM=AM, KG=KG, KSTEP=KSTEP, ACC=ACC, ES=ES, EPCK=EPCK, MPF=MPF, CPR=CPR, RPL=RPL, NB=NB, A_PER_T=A_PER_T, B_PER_T=B_PER_T,
        SLAB=slab_bytes, DEPTH=depth, RS=RS, KT=KT, TILES_M=tiles_m, TILES_N=tiles_n, NTILES=n_tiles, GM=gm, GN=gn,
        XCDS=ctx.xcds, frag_t=frag_t, in_c=in_c, out_c=out_c, params=", ".join(params), builtin=plan.atom.builtin,
        acc_t=rt.vector_type("f32", ACC)[0], G=ACC // 4,
    )  # fmt: skip

    o: list[str] = []
    a = o.append
    a(f"// {name}: M={M} N={N} K={K} TILE={plan.spell()} STAGE={stage.spell()} xcd-block={gm}x{gn}")
    if m_sym is not None:
        D.update(M=m_sym.c(), TILES_M="((M + TM - 1) / TM)", NTILES="(TILES_M * TILES_N)")
    for k_, v_ in D.items():
        if isinstance(v_, int) or (m_sym is not None and k_ in ("M", "TILES_M", "NTILES")):
            a(f"#define {k_} {v_}")
    a(r"""
EMH_DEV int emh_swz(int row, int c) { return c ^ ((row / RPL) % CPR); }
""")
    a(f'extern "C" __global__ __launch_bounds__({TT}) void {name}({D["params"]}) {{')
    a(r"""  extern __shared__ __attribute__((aligned(16))) unsigned char emh_lds[];
  // ---- tile ownership: consecutive workgroup ids rotate over the XCDs ----
  const int bid = blockIdx.x;
  const int xcd = bid % XCDS;
  const int slot = bid / XCDS;
  constexpr int PER_BLOCK = GM * GN;
  constexpr int BLOCKS_N = TILES_N / GN;
  const int NBLOCKS = (TILES_M / GM) * BLOCKS_N;
  int tm, tn;
  {
    // XCD x owns tile blocks x, x+XCDS, ...; `slot` walks the tiles of those blocks.
    const int blk = xcd + (slot / PER_BLOCK) * XCDS;
    const int in_blk = slot % PER_BLOCK;
    if (blk < NBLOCKS) {
      tm = (blk / BLOCKS_N) * GM + in_blk / GN;
      tn = (blk % BLOCKS_N) * GN + in_blk % GN;
    } else {
      return;  // padding workgroup of a launch rounded up to whole XCD rounds
    }
  }
  const int m0 = tm * TM, n0 = tn * TN;
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  // Measurement build (-DEMH_STAMP=1 or 2 among the compiler options): the first thread of workgroup 0 sums the clocks
  // its slabs spend per phase of the k loop (1, averaged per slab) or the kernel spends per part (2: prologue / k loop /
  // epilogue arithmetic / stores) and leaves four floats over the first 16 bytes of its output tile; the rest of the
  // output is the product as usual.
#ifndef EMH_STAMP
#define EMH_STAMP 0
#endif
#define EMH_STAMP_AT(i) if (EMH_STAMP == 1) { const unsigned long long now_ = __builtin_readcyclecounter(); st_acc[i] += (unsigned)(now_ - st_last); st_last = now_; st_acc[4 + (i)] += 1u; }
#define EMH_PHASE_AT(i) if (EMH_STAMP == 2) { const unsigned long long now_ = __builtin_readcyclecounter(); st_acc[i] += (unsigned)(now_ - st_last); st_last = now_; st_acc[4 + (i)] = 1u; }
  unsigned st_acc[8] = {0u, 0u, 0u, 0u, 0u, 0u, 0u, 0u};
  unsigned long long st_last = EMH_STAMP ? __builtin_readcyclecounter() : 0ull;
  const int stid = tid >= T ? tid - T : tid;  // staging thread id (the waves past the tile's own only stage)
  const int wm = (wave / WN) % WM, wn = wave % WN;
  const int lr = lane % AM, lk = lane / AM;  // fragment row, k-group
""")
    if split is not None:
        a("  // cross-workgroup split of the reduction axis: workgroup row blockIdx.y owns slice blockIdx.y (K is the slice length)")
        a("  const long ASL = (long)blockIdx.y * K, BSL = ASL;")
        a("  const long OSL = " + ("(long)blockIdx.y * M * LDO;" if split[1] == "kernel" else "0;  // every slice adds into the one zeroed plane"))
    elif batch > 1:
        a("  // independent products: workgroup row blockIdx.y owns product blockIdx.y")
        a(f"  const long ASL = (long)blockIdx.y * {body.a_batch}L, BSL = (long)blockIdx.y * {body.b_batch}L, OSL = (long)blockIdx.y * {body.out_batch}L;")
    else:
        a("  constexpr long ASL = 0, BSL = 0, OSL = 0;")
    # ---- staging ------------------------------------------------------------
    a(f"  const {in_c}* ga[A_PER_T]; int la[A_PER_T];" + (" int ca[A_PER_T];" if pro is not None else "") + (" int ka[A_PER_T], kb[B_PER_T];" if k_guard else ""))
    a(f"  const {in_c}* gb[B_PER_T]; int lb[B_PER_T];")
    if dli or dlm or spec:
        if max(M * lda, N * NB * ldb) * ES >= 2**32:
            raise LoweringError("contraction: STAGE .../dli addresses operands with 32-bit byte offsets; this operand is larger than 4 GiB")
        a("  unsigned va[A_PER_T], vb[B_PER_T];  // byte offset of each request's chunk from the operand base (the k position is added to the base, in scalar registers)")
        # Request i of a thread is request 0 moved down ST / CPR rows (the chunk column is the same): where no row is
        # clamped that is a constant added to the scalar base, and one lane offset serves every request of an operand.
        lin_a = not m_guard and not dli
        lin_b = not n_guard and not gate and not dli
        # (... and the same swizzled chunk: the swizzle repeats every RPL * CPR rows)
        lin = "(ST % CPR == 0 && (ST / CPR) % (RPL * CPR) == 0)"
        a(f"  constexpr bool LIN_A = {lin if lin_a else 'false'}, LIN_B = {lin if lin_b else 'false'};")
        a("  constexpr long STEP_A = LIN_A ? (long)(ST / CPR) * LDA * ES : 0, STEP_B = LIN_B ? (long)(ST / CPR) * LDB * ES : 0;")
        a("  const int wave_u = __builtin_amdgcn_readfirstlane(stid / 64);  // wave-uniform by construction; says so to the compiler")
        a("  const unsigned lds0 = emh_lds_addr(emh_lds);")
    a(r"""  #pragma unroll
  for (int i = 0; i < A_PER_T; ++i) {
    const int q = stid + i * ST;""")
    if dl:
        a("    const int row = q / CPR, c = emh_swz(row, q % CPR);  // lane order fixes the LDS slot; pick the chunk that belongs there")
        a("    la[i] = q * 16;")
    else:
        a("    const int row = q / CPR, c = q % CPR;")
        a("    la[i] = row * (BK * ES) + emh_swz(row, c) * 16;")
    a(f"    int gr = m0 + row;{' if (gr > M - 1) gr = M - 1;' if m_guard else ''}")
    a(f"    ga[i] = A + {body.a_offset}L + ASL + (long)gr * LDA + c * EPCK;")
    if dli or dlm or spec:
        a("    va[i] = ((unsigned)gr * LDA + c * EPCK) * (unsigned)ES;")
    if pro is not None:
        a("    ca[i] = c * EPCK;")
    if k_guard:
        a("    ka[i] = c * EPCK;")
    a("  }")
    a(r"""  #pragma unroll
  for (int i = 0; i < B_PER_T; ++i) {
    const int q = stid + i * ST;""")
    if dl or mix:
        a("    const int row = q / CPR, c = emh_swz(row, q % CPR);")
        a("    lb[i] = TM * BK * ES + q * 16;")
    else:
        a("    const int row = q / CPR, c = q % CPR;")
        a("    lb[i] = TM * BK * ES + row * (BK * ES) + emh_swz(row, c) * 16;")
    if gate:
        a("    int gr = (row < TN) ? (n0 + row) : (N + n0 + row - TN);  // second half of the slab: the paired matrix")
        if n_guard:
            a("    { const int lim = (row < TN) ? (N - 1) : (2 * N - 1); if (gr > lim) gr = lim; }")
    else:
        a(f"    int gr = n0 + row;{' if (gr > N - 1) gr = N - 1;' if n_guard else ''}")
    a(f"    gb[i] = B + {body.b_offset}L + BSL + (long)gr * LDB + c * EPCK;")
    if dli or dlm or spec:
        a("    vb[i] = ((unsigned)gr * LDB + c * EPCK) * (unsigned)ES;")
    if k_guard:
        a("    kb[i] = c * EPCK;")
    a("  }")

    a(f"  {D['acc_t']} acc[NB][FM][FN];")
    a(r"""  #pragma unroll
  for (int h = 0; h < NB; ++h)
  #pragma unroll
  for (int i = 0; i < FM; ++i)
  #pragma unroll
  for (int j = 0; j < FN; ++j)
  #pragma unroll
  for (int r = 0; r < ACC; ++r) acc[h][i][j][r] = 0.0f;
""")
    a("  #define EMH_OPND(f, e) " + ("((f)[e])  /* one element of the chunk per MFMA */" if MPF > 1 else "(f)"))
    KS = BK // KSTEP
    frag_decl = f"  {frag_t} fw[{max(2, KS) if pp else 2}][NB][FN], fx[{max(2, KS) if pp else 2}][FM];"
    a(frag_decl)
    a(r"""  // Fragments are double-buffered in registers: the reads for step s+1 are
  // issued before the MFMAs of step s and complete in their shadow.  The
  // sched_barriers pin that order (the scheduler otherwise sinks the reads to
  // just before their use).
  #define EMH_READ(P, buf, kk) { \
    const unsigned char* sA_ = emh_lds + (buf) * SLAB; \
    const unsigned char* sB_ = sA_ + TM * BK * ES; \
    const int c_ = (kk) * KG + lk; \
    _Pragma("unroll") for (int h = 0; h < NB; ++h) \
    _Pragma("unroll") for (int j = 0; j < FN; ++j) { \
      const int row_ = h * TN + (wn * FN + j) * AM + lr; \
      fw[P][h][j] = *(const FRAG_T*)(sB_ + row_ * (BK * ES) + emh_swz(row_, c_) * 16); } \
    _Pragma("unroll") for (int i = 0; i < FM; ++i) { \
      const int row_ = (wm * FM + i) * AM + lr; \
      fx[P][i] = *(const FRAG_T*)(sA_ + row_ * (BK * ES) + emh_swz(row_, c_) * 16); } \
    __builtin_amdgcn_sched_barrier(0); }
  #define EMH_READ_W(P, buf, kk, h, j) { const int row_ = (h) * TN + (wn * FN + (j)) * AM + lr; \
    fw[P][h][j] = *(const FRAG_T*)(emh_lds + (buf) * SLAB + TM * BK * ES + row_ * (BK * ES) + emh_swz(row_, (kk) * KG + lk) * 16); }
  #define EMH_READ_X(P, buf, kk, i) { const int row_ = (wm * FM + (i)) * AM + lr; \
    fx[P][i] = *(const FRAG_T*)(emh_lds + (buf) * SLAB + row_ * (BK * ES) + emh_swz(row_, (kk) * KG + lk) * 16); }
  #define EMH_MMA(P) { \
    _Pragma("unroll") for (int e = 0; e < MPF; ++e) \
    _Pragma("unroll") for (int h = 0; h < NB; ++h) \
    _Pragma("unroll") for (int i = 0; i < FM; ++i) \
    _Pragma("unroll") for (int j = 0; j < FN; ++j) \
      acc[h][i][j] = BUILTIN(EMH_OPND(fw[P][h][j], e), EMH_OPND(fx[P][i], e), acc[h][i][j], 0, 0, 0); \
    __builtin_amdgcn_sched_barrier(0); }
""".replace("FRAG_T", frag_t).replace("BUILTIN", plan.atom.builtin))
    if not dl:
        # global -> VGPR -> LDS, one slab ahead, one barrier per slab.  With the
        # mixed transport only the a operand takes that road (it may be transformed on
        # the way); the b slab is requested direct-to-LDS at the same moment and is
        # waited for, and published, where the a slab is written.
        if mix:
            b_gload = '{ unsigned char* sd_ = emh_lds + ((kt) % DEPTH) * SLAB; _Pragma("unroll") for (int i = 0; i < B_PER_T; ++i) emh_dma16(gb[i] + (kt) * BK, sd_ + lb[i] - lane * 16); }'
            b_lstore = "__builtin_amdgcn_s_waitcnt(EMH_WAIT_VM_LGKM0(0)); emh_lds_publish(emh_lds + tid * 4);"
        else:
            b_gload = '_Pragma("unroll") for (int i = 0; i < B_PER_T; ++i) rb[S][i] = *(const u32x4*)(gb[i] + (kt) * BK);'
            if k_guard:
                b_gload = '_Pragma("unroll") for (int i = 0; i < B_PER_T; ++i) { rb[S][i] = u32x4{0u, 0u, 0u, 0u}; if ((kt) * BK + kb[i] < K) rb[S][i] = *(const u32x4*)(gb[i] + (kt) * BK); }'
            b_lstore = '_Pragma("unroll") for (int i = 0; i < B_PER_T; ++i) *(u32x4*)(s_ + lb[i]) = rb[S][i];'
        if pro is not None:
            # Row statistic over the full k extent of this thread's rows: the chunks of
            # a row's slab sit in CPR consecutive lanes, so a lane sums its own chunk
            # column over all slabs and a butterfly over those lanes finishes the row.
            unroll = max(1, min(KT, 32 // max(1, A_PER_T)))
            a("  float ss[A_PER_T];")
            a("  #pragma unroll")
            a("  for (int i = 0; i < A_PER_T; ++i) ss[i] = 0.0f;")
            if not deferred:
                a(f"  #pragma unroll {unroll}")
                a("  for (int kt = 0; kt < KT; ++kt) {")
                a("    #pragma unroll")
                a("    for (int i = 0; i < A_PER_T; ++i) {")
                a(f"      const {frag_t} xv = *(const {frag_t}*)(ga[i] + kt * BK);")
                a("      #pragma unroll")
                a("      for (int e = 0; e < 8; ++e) { const float x_ = (float)xv[e]; ss[i] += " + E.render(pro.stat_pre, {"x": "x_"}) + "; }")
                a("    }")
                a("  }")
                a("  #pragma unroll")
                a("  for (int i = 0; i < A_PER_T; ++i)")
                a("  #pragma unroll")
                a("  for (int msk = 1; msk < CPR; msk *= 2) ss[i] += __shfl_xor(ss[i], msk, 64);")
            wdecl = f" {frag_t} rw[RS][A_PER_T];" if pro.weight is not None else ""
            a(f"  u32x4 ra[RS][A_PER_T], rb[RS][B_PER_T];{wdecl}")
            wload = " rw[S][i] = *(const FRAG_T*)(NW + (kt) * BK + ca[i]);".replace("FRAG_T", frag_t) if pro.weight is not None else ""
            a("  #define EMH_GLOAD(kt, S) { \\")
            a(f'    _Pragma("unroll") for (int i = 0; i < A_PER_T; ++i) {{ ra[S][i] = *(const u32x4*)(ga[i] + (kt) * BK);{wload} }} \\')
            a("    " + b_gload + " }")
            env = {"x": "(float)xv_[e]", "ss": "ss[i]"}
            if pro.weight is not None:
                env["w"] = "(float)rw[S][i][e]"
            a("  #define EMH_LSTORE(buf, S) { \\")
            a("    unsigned char* s_ = emh_lds + (buf) * SLAB; \\")
            a('    _Pragma("unroll") for (int i = 0; i < A_PER_T; ++i) { \\')
            a(f"      {frag_t} xv_ = __builtin_bit_cast({frag_t}, ra[S][i]); \\")
            if deferred:  # the slab goes to LDS as it is; its share of the row statistic is taken on the way
                a('      _Pragma("unroll") for (int e = 0; e < 8; ++e) { const float x_ = (float)xv_[e]; ss[i] += ' + E.render(pro.stat_pre, {"x": "x_"}) + "; } \\")
            else:
                a(f'      _Pragma("unroll") for (int e = 0; e < 8; ++e) xv_[e] = ({in_c})({E.render(pro.project, env)}); \\')
            a(f"      *({frag_t}*)(s_ + la[i]) = xv_; }} \\")
            a("    " + b_lstore + " }")
        else:
            a(r"""  u32x4 ra[RS][A_PER_T], rb[RS][B_PER_T];
  #define EMH_GLOAD(kt, S) { \
    _Pragma("unroll") for (int i = 0; i < A_PER_T; ++i) A_GLOAD \
    B_GLOAD }
  #define EMH_LSTORE(buf, S) { \
    unsigned char* s_ = emh_lds + (buf) * SLAB; \
    _Pragma("unroll") for (int i = 0; i < A_PER_T; ++i) *(u32x4*)(s_ + la[i]) = ra[S][i]; \
    B_LSTORE }""".replace("B_GLOAD", b_gload).replace("B_LSTORE", b_lstore).replace(
                "A_GLOAD",
                "{ ra[S][i] = u32x4{0u, 0u, 0u, 0u}; if ((kt) * BK + ka[i] < K) ra[S][i] = *(const u32x4*)(ga[i] + (kt) * BK); }" if k_guard else "ra[S][i] = *(const u32x4*)(ga[i] + (kt) * BK);",
            ))
        # Slab j travels through register set j % RS: RS slabs are in flight from
        # global memory while one is computed on, so a load has RS steps to arrive.
        a(r"""  #pragma unroll
  for (int p = 0; p < RS; ++p) if (p < KT) EMH_GLOAD(p, p);
  EMH_LSTORE(0, 0);
  __syncthreads();
ROW_EPILOGUE_TABLES
  for (int kt0 = 0; kt0 < KT; kt0 += RS) {
  #pragma unroll
  for (int rs = 0; rs < RS; ++rs) {
    const int kt = kt0 + rs;
    if (KT % RS != 0 && kt >= KT) break;
    const int cur = kt % DEPTH;
    if (kt + RS < KT) EMH_GLOAD(kt + RS, rs);  // set rs held slab kt, which is in LDS by now
    EMH_READ(0, cur, 0);""")
        for kk in range(KS):
            if kk + 1 < KS:
                a(f"    EMH_READ({(kk + 1) & 1}, cur, {kk + 1});")
            a(f"    EMH_MMA({kk & 1});")
        a(r"""    if (kt + 1 < KT) EMH_LSTORE((kt + 1) % DEPTH, (rs + 1) % RS);
    __syncthreads();
  }
  }""")
    else:
        if KS % 2 and not pp:
            raise LoweringError(f"contraction: direct-to-LDS pipeline needs an even number of MFMA steps per slab (BK={BK}, step={KSTEP})")
        if pp and (T != 512 or deferred or rowepi is not None or depth < 3):
            raise LoweringError("contraction: STAGE .../pp takes a tile of eight waves (two groups of four alternate, four more waves stage), a ring of at least three, and no row prologue or row epilogue")
        loads_per_slab = A_PER_T + B_PER_T
        if (depth - 1) * loads_per_slab > 63:
            raise LoweringError("contraction: too many loads in flight for the 6-bit vmcnt counter; lower STAGE depth")
        if dli and depth < 3:
            raise LoweringError("contraction: STAGE .../dli fills one slab while another is computed on and needs a ring of at least three")
        a(r"""  // Each wave-level direct-to-LDS load fills 64 consecutive 16-byte LDS slots
  // (slot = lane); the per-lane *global* address selects which chunk lands there.
  #define EMH_DLOAD(kt, buf) { \
    unsigned char* s_ = emh_lds + (buf) * SLAB; \
    _Pragma("unroll") for (int i = 0; i < A_PER_T; ++i) \
      emh_dma16(ga[i] + (kt) * BK, s_ + la[i] - lane * 16); \
    _Pragma("unroll") for (int i = 0; i < B_PER_T; ++i) \
      emh_dma16(gb[i] + (kt) * BK, s_ + lb[i] - lane * 16); }
  // A plain s_barrier is used on purpose: a workgroup fence would drain every
  // outstanding direct-to-LDS load and serialise the pipeline.  Loads retire in
  // issue order, so "at most n outstanding" means the older slabs have landed.
  // vmcnt reaching its target does not yet make direct-to-LDS data visible to
  // other waves (measured: stale fragment reads right after the barrier); an LDS
  // read of this wave queues behind its own DMA writes, so waiting for it orders
  // them before the barrier.
  #define EMH_SLAB_SYNC(n) { \
    __builtin_amdgcn_s_waitcnt(EMH_WAIT_VM_LGKM0(n)); \
    emh_lds_publish(emh_lds + tid * 4); \
    asm volatile("" ::: "memory"); __builtin_amdgcn_s_barrier(); asm volatile("" ::: "memory"); }
  #pragma unroll
  for (int p = 0; p < DEPTH - DLI; ++p) if (p < KT STAGER) EMH_DLOAD(p, p);""".replace("DLI", "1" if dli or pp else "0").replace(" STAGER", " && tid >= T" if spec else ""))
        if dli or dlm or spec:
            a(f"""  // One request of slab kt into ring buffer buf: the operand base moves along k in scalar registers, the
  // lane's chunk offset is a loop-invariant 32-bit register, the LDS target a scalar: no vector arithmetic per request.
  #define EMH_DPART_A(kt, buf, i) emh_dma16s((const unsigned char*)(A + {body.a_offset}L + ASL) + (long)(kt) * (BK * ES) + (long)(i) * STEP_A, va[LIN_A ? 0 : (i)], lds0 + (buf) * SLAB + (wave_u * 64 + (i) * ST) * 16)
  #define EMH_DPART_B(kt, buf, i) emh_dma16s((const unsigned char*)(B + {body.b_offset}L + BSL) + (long)(kt) * (BK * ES) + (long)(i) * STEP_B, vb[LIN_B ? 0 : (i)], lds0 + (buf) * SLAB + TM * BK * ES + (wave_u * 64 + (i) * ST) * 16)""")
        if deferred:
            # the rows arrive in LDS untouched: every thread reads back the chunks it requested
            # (any chunk of the row will do for a row sum) while the slab is resident
            a("  float ss[A_PER_T];")
            a("  #pragma unroll")
            a("  for (int i = 0; i < A_PER_T; ++i) ss[i] = 0.0f;")
            a(f"  {frag_t} sx[A_PER_T];")
            a("  #define EMH_SUMSQ_READ(buf) { \\")
            a(f'    _Pragma("unroll") for (int i = 0; i < A_PER_T; ++i) sx[i] = *(const {frag_t}*)(emh_lds + (buf) * SLAB + la[i]); }}')
            a("  #define EMH_SUMSQ_ADD() { \\")
            a('    _Pragma("unroll") for (int i = 0; i < A_PER_T; ++i) \\')
            a('    _Pragma("unroll") for (int e = 0; e < 8; ++e) { const float x_ = (float)sx[i][e]; ss[i] += ' + E.render(pro.stat_pre, {"x": "x_"}) + "; } \\")
            a("    __builtin_amdgcn_sched_barrier(0); }")
        first_younger = min(depth - 1 - (1 if dli or pp else 0), KT - 1) * loads_per_slab
        a(f"  EMH_SLAB_SYNC({first_younger});")
        if not spec:
            a("  EMH_READ(0, 0, 0);")
        a("ROW_EPILOGUE_TABLES")
        a("  EMH_PHASE_AT(0)  // tile decode, first requests, first slab landed")
        a("  if (EMH_STAMP == 1) st_last = __builtin_readcyclecounter();")
        if pp:
            a("  const int role = __builtin_amdgcn_readfirstlane(tid / 256);  // 0, 1: the two consumer groups (waves 0-3, 4-7); 2: the producers")
            part_fmt = [f"EMH_DPART_A({{slab}}, {{buf}}, {i});" for i in range(A_PER_T)] + [f"EMH_DPART_B({{slab}}, {{buf}}, {i});" for i in range(B_PER_T)]
            _emit_pingpong_loop(a, KT=KT, KS=KS, depth=depth, parts=part_fmt)

        def frag_reads(P: int, buf: str, kk: int) -> list[str]:
            """One statement per fragment of step ``kk`` of the slab in ring buffer ``buf`` into register set ``P``."""
            return [f"EMH_READ_W({P}, {buf}, {kk}, {h}, {j});" for h in range(NB) for j in range(FN)] + [f"EMH_READ_X({P}, {buf}, {kk}, {i});" for i in range(FM)]

        def mma_interleaved(P: int, reads: list[str], requests: list[str]) -> None:
            """The MFMAs of a step with the next step's fragment reads (over the first ``_READ_SPREAD`` of them: the data
            has the rest of the step to arrive) and, in a slab's last step, the requests of slab ``kt + DEPTH`` (over the
            first ``_SPREAD`` of them) issued one at a time in between: the matrix pipe always has an MFMA of this wave
            queued behind whatever else the wave issues."""
            n = NB * FM * FN
            if 4 * n < 5 * len(reads):
                # about as many reads as MFMAs: spread out, the last ones would land after the step that needs them has
                # begun (512-token gate/up, six MFMAs and seven reads a step: 10.1 -> 11.2 us); they go out together
                a("    " + " ".join(reads) + " __builtin_amdgcn_sched_barrier(0);")
                reads = []
            r_after = [int(q * n * _READ_SPREAD) // max(len(reads), 1) for q in range(len(reads))]
            q_after = [int(q * n * _SPREAD) // max(len(requests), 1) for q in range(len(requests))]
            for e in range(MPF):  # (the MFMAs a fragment feeds are a pass over all accumulators each, as in EMH_MMA)
                idx = 0
                for h in range(NB):
                    for i in range(FM):
                        for j in range(FN):
                            a(f"    acc[{h}][{i}][{j}] = {plan.atom.builtin}(EMH_OPND(fw[{P}][{h}][{j}], {e}), EMH_OPND(fx[{P}][{i}], {e}), acc[{h}][{i}][{j}], 0, 0, 0);")
                            extra = [st for st, at in zip(reads, r_after) if at == idx] + [st for st, at in zip(requests, q_after) if at == idx] if e == 0 else []
                            if extra:
                                a("    __builtin_amdgcn_sched_barrier(0); " + " ".join(extra) + " __builtin_amdgcn_sched_barrier(0);")
                            idx += 1
            a("    __builtin_amdgcn_sched_barrier(0);")

        def slab_steps(kt: str, static_kt: int | None) -> None:
            """MFMA steps of slab ``kt``.  With ``static_kt`` the hand-over to the
            next slab is resolved at emit time (tail); otherwise it is the
            steady state, where every condition holds and the body is branch-free
            (so the wait-count pass can see that only the newest reads are pending)."""
            a(f"    {{ const int cur = ({kt}) % DEPTH;")
            if deferred:
                a("    EMH_SUMSQ_READ(cur);  // queued with the fragment reads; summed behind the first MFMAs")
            for kk in range(KS):
                P = kk & 1
                if kk + 1 < KS:
                    if dlm and static_kt is None:
                        mma_interleaved(P, frag_reads(P ^ 1, "cur", kk + 1), [])
                        if deferred and kk == 0:
                            a("    EMH_SUMSQ_ADD();")
                        continue
                    a(f"    EMH_READ({P ^ 1}, cur, {kk + 1});")
                elif static_kt is None:
                    a("    EMH_STAMP_AT(0)  // the steps before the hand-over issued")
                    a(f"    EMH_SLAB_SYNC({(depth - 2) * loads_per_slab});")
                    a("    EMH_STAMP_AT(1)  // requests waited for, published, barrier")
                    if dlm:
                        # the buffer is free from here on (the last step's fragments are in registers): its next slab is
                        # requested one request at a time between this step's MFMAs instead of as a burst in front of them
                        parts = [f"EMH_DPART_A(({kt}) + DEPTH, cur, {i});" for i in range(A_PER_T)] + [f"EMH_DPART_B(({kt}) + DEPTH, cur, {i});" for i in range(B_PER_T)]
                        mma_interleaved(P, frag_reads(P ^ 1, f"((({kt}) + 1) % DEPTH)", 0), parts)
                        a("    EMH_STAMP_AT(2)  // the last step and the next slab's requests issued")
                        continue
                    a(f"    EMH_DLOAD(({kt}) + DEPTH, cur);")
                    a(f"    EMH_READ({P ^ 1}, (({kt}) + 1) % DEPTH, 0);")
                elif static_kt + 1 < KT:
                    younger = min(KT - static_kt - 2, depth - 2)
                    a(f"    EMH_SLAB_SYNC({younger * loads_per_slab});")
                    if static_kt + depth < KT:
                        a(f"    EMH_DLOAD({static_kt + depth}, cur);")
                    a(f"    EMH_READ({P ^ 1}, {(static_kt + 1) % depth}, 0);")
                a(f"    EMH_MMA({P});")
                if static_kt is None and kk + 1 == KS:
                    a("    EMH_STAMP_AT(2)  // the last step issued")
                if deferred and kk == 0:
                    a("    EMH_SUMSQ_ADD();")
            a("    }")

        # ``dli``: the requests of slab kt + DEPTH - 1 are issued *between the MFMAs* of slab kt, into the buffer
        # slab kt - 1 was read from (free since the barrier that ended it).  Issued as one burst behind the
        # barrier, as ``dl`` does, every wave sits in the request queue at the same moment and the matrix pipe
        # drains: load time and MFMA time add up instead of overlapping.
        n_mma = NB * FM * FN
        part_list = [("A", i) for i in range(A_PER_T)] + [("B", i) for i in range(B_PER_T)]
        slot_of = [(q * KS * n_mma) // len(part_list) for q in range(len(part_list))]  # after which MFMA of the slab a request goes
        n_pre = sum(1 for sl in slot_of if sl < (KS - 1) * n_mma)  # requests issued before the slab's closing barrier

        def mma_with_parts(P: int, kk: int, kt: str | None) -> None:
            idx = 0
            for h in range(NB):
                for i in range(FM):
                    for j in range(FN):
                        for e in range(MPF):
                            a(f"    acc[{h}][{i}][{j}] = {plan.atom.builtin}(EMH_OPND(fw[{P}][{h}][{j}], {e}), EMH_OPND(fx[{P}][{i}], {e}), acc[{h}][{i}][{j}], 0, 0, 0);")
                        if kt is not None:
                            for q, (which, pi) in enumerate(part_list):
                                if slot_of[q] == kk * n_mma + idx:
                                    a(f"    __builtin_amdgcn_sched_barrier(0); EMH_DPART_{which}(({kt}) + DEPTH - 1, (({kt}) + DEPTH - 1) % DEPTH, {pi}); __builtin_amdgcn_sched_barrier(0);")
                        idx += 1
            a("    __builtin_amdgcn_sched_barrier(0);")

        def slab_steps_dli(kt: str, static_kt: int | None) -> None:
            a(f"    {{ const int cur = ({kt}) % DEPTH;")
            if deferred:
                a("    EMH_SUMSQ_READ(cur);")
            issuing = static_kt is None
            for kk in range(KS):
                P = kk & 1
                if kk + 1 < KS:
                    a(f"    EMH_READ({P ^ 1}, cur, {kk + 1});")
                elif static_kt is None:
                    # outstanding and younger than slab kt + 1: the whole slabs kt + 2 .. kt + DEPTH - 2 and what has been requested of slab kt + DEPTH - 1
                    a(f"    EMH_SLAB_SYNC({(depth - 3) * loads_per_slab + n_pre});")
                    a(f"    EMH_READ({P ^ 1}, (({kt}) + 1) % DEPTH, 0);")
                elif static_kt + 1 < KT:
                    a(f"    EMH_SLAB_SYNC({max(0, KT - 2 - static_kt) * loads_per_slab});")
                    a(f"    EMH_READ({P ^ 1}, {(static_kt + 1) % depth}, 0);")
                mma_with_parts(P, kk, kt if issuing else None)
                if deferred and kk == 0:
                    a("    EMH_SUMSQ_ADD();")
            a("    }")

        if spec:
            pass
        elif dli:
            steady = max(0, KT - depth + 1)
            if steady:
                a(f"  for (int kt = 0; kt < {steady}; ++kt) {{")
                slab_steps_dli("kt", None)
                a("  }")
            for kt_s in range(steady, KT):
                slab_steps_dli(str(kt_s), kt_s)
        else:
            steady = max(0, KT - depth)
            if steady:
                a(f"  for (int kt = 0; kt < {steady}; ++kt) {{")
                slab_steps("kt", None)
                a("  }")
            for kt_s in range(steady, KT):
                slab_steps(str(kt_s), kt_s)

    a("  EMH_PHASE_AT(1)  // the k loop")
    # ---- epilogue ------------------------------------------------------------------
    esz = body.out_dtype.nbytes
    EPC = 16 // esz  # output elements per 16-byte chunk
    c_stride = TN * esz + 16
    staged = (N % EPC == 0) and (TN % EPC == 0) and (TM * c_stride <= ctx.lds_bytes_per_cu) and ((TM * (TN // EPC)) % T == 0)
    vt4 = _pack4_t(body.out_dtype.name)
    cast = "" if body.out_dtype is F32 else f"({out_c})"
    post = body.post if body.post is not None else E.Var("y")
    unknown = E.variables(post) - ({"y"} | set(epi_names))
    if unknown:
        raise LoweringError(f"contraction post-epilogue uses unknown names {sorted(unknown)}")
    a(r"""  // Accumulator lane layout: column (l % AM) is the output row m; the registers
  // of group g hold four consecutive n starting at g*4*KG + (l / AM)*4.""")
    if staged:
        lds_bytes = max(lds_bytes, TM * c_stride)
    # The deferred row scales sit behind the output tile, inside the slab area: every step of the
    # k loop ends with a barrier, so the slabs are dead when the scales are written.
    rs_off = TM * c_stride if staged else 0
    if deferred:
        lds_bytes = max(lds_bytes, rs_off + TM * 4)
        a("  // Row statistic: finish it over the lanes that hold a row's chunks, turn it into the row's")
        a("  // scale factor and hand it to the lanes that own the row's accumulators.")
        if dl:
            a("  __syncthreads();  // the last slab's fragments have been read by every wave")
        a("  #pragma unroll")
        a("  for (int i = 0; i < A_PER_T; ++i) {")
        a("    #pragma unroll")
        a("    for (int msk = 1; msk < CPR; msk *= 2) ss[i] += __shfl_xor(ss[i], msk, 64);")
        a(f"    if ((tid + i * T) % CPR == 0) ((float*)(emh_lds + {rs_off}))[(tid + i * T) / CPR] = {E.render(pro.scale, {'ss': 'ss[i]'})};")
        a("  }")
        if not staged:
            a("  __syncthreads();")
    if staged:
        a(f"  constexpr int CSTRIDE = {c_stride};")
        a("  __builtin_amdgcn_s_waitcnt(EMH_WAIT_VM_LGKM0(0));" if dl else "")
        a("  __syncthreads();  // every wave is done with the operand slabs; reuse them for the output tile")
        if spec:
            a("  if (tid < T) {  // the staging waves hold no accumulators")
        a(r"""  #pragma unroll
  for (int i = 0; i < FM; ++i) {
    const int ml = (wm * FM + i) * AM + lr;""")
        if deferred:
            a(f"    const float rs_ = ((const float*)(emh_lds + {rs_off}))[ml];")
        a(r"""    #pragma unroll
    for (int j = 0; j < FN; ++j)
    #pragma unroll
    for (int g = 0; g < G; ++g) {
      const int nl = (wn * FN + j) * AM + g * 4 * KG + lk * 4;""")
        if body.bias is not None:
            bt4 = _pack4_t(body.bias_dtype.name)
            clamp = f"(n0 + nl < N ? n0 + nl : N - 4)" if n_guard else "(n0 + nl)"
            a(f"      const {bt4} bv = *(const {bt4}*)(BIAS + {clamp});")
        a(f"      {vt4} yo;")
        sc = " * rs_" if deferred else ""
        for r in range(4):
            env = {"acc": f"(acc[0][i][j][g * 4 + {r}]{sc})"}
            if gate:
                env["acc2"] = f"(acc[1][i][j][g * 4 + {r}]{sc})"
            if body.bias is not None:
                env["bias"] = f"(float)bv[{r}]"
            a(f"      yo[{r}] = {cast}({E.render(epi, env)});")
        a(f"      *({vt4}*)(emh_lds + ml * CSTRIDE + nl * {esz}) = yo;")
        a("    }")
        a("  }")
        if spec:
            a("  }")
        a("  __syncthreads();")
        if spec:
            a("  if (tid >= T) return;  // no barrier follows")
        a("  EMH_PHASE_AT(2)  // accumulators mapped, rounded and staged")
        vt_chunk = rt.vector_type(body.out_dtype.name, EPC)[0]
        a(f"  constexpr int CPRC = TN / {EPC};  // 16-byte chunks per output-tile row")
        if rowepi is not None:
            _emit_row_epilogue(a, body, rowepi, re_args, EPC, vt_chunk, out_c, m_guard, n_guard)
        a(r"""  #pragma unroll
  for (int it = 0; it < (TM * CPRC) / T; ++it) {
    const int q = tid + it * T;
    const int row = q / CPRC, cc = q % CPRC;""")
        a(f"    const int m = m0 + row, n = n0 + cc * {EPC};")
        conds = []
        if m_guard:
            conds.append("m < M")
        if n_guard:
            conds.append("n < N")
        a(f"    if ({' && '.join(conds) if conds else 'true'}) {{")
        a(f"      {vt_chunk} v = *(const {vt_chunk}*)(emh_lds + row * CSTRIDE + cc * 16);")
        if body.post is not None:
            for i, (_, dt) in enumerate(body.epilogue_operands):
                if dt.nbytes != esz:
                    raise LoweringError("contraction: post-epilogue operands must have the output dtype")
                a(f"      const {vt_chunk} ev{i} = *(const {vt_chunk}*)(e{i} + (long)m * LDO + n);")
            for r in range(EPC):
                env = {"y": f"(float)v[{r}]"}
                for i, (n_, _) in enumerate(body.epilogue_operands):
                    env[n_] = f"(float)ev{i}[{r}]"
                a(f"      v[{r}] = {cast}({E.render(post, env)});")
        if split is not None and split[1] == "atomic":
            a(f"      float* o_ = O + {body.out_offset}L + OSL + (long)m * LDO + n;")
            a("      #pragma unroll")
            a(f"      for (int r = 0; r < {EPC}; ++r) __builtin_amdgcn_global_atomic_fadd_f32((__attribute__((address_space(1))) float*)(o_ + r), v[r]);")
        else:
            a(f"      *({vt_chunk}*)(O + {body.out_offset}L + OSL + (long)m * LDO + n) = v;")
        a("    }")
        a("  }")
        if rowepi is not None:
            a("  }")
        a("  EMH_PHASE_AT(3)  // the tile stored")
        a("  if (EMH_STAMP && bid == 0 && tid == 0) {  // over the 16 bytes this thread stored first: the start of its tile's first row")
        a("    #pragma unroll")
        a(f"    for (int i = 0; i < 4; ++i) ((float*)(O + {body.out_offset}L + OSL + (long)m0 * LDO + n0))[i] = (float)st_acc[i] / (float)(st_acc[4 + i] ? st_acc[4 + i] : 1u);")
        a("  }")
    else:
        if rowepi is not None:
            raise LoweringError("contraction: the row epilogue works on the staged output tile, which this tile shape does not have")
        if spec:
            a("  if (tid >= T) return;  // the staging waves hold no accumulators, and no barrier follows")
        a(r"""  #pragma unroll
  for (int i = 0; i < FM; ++i) {
    const int m = m0 + (wm * FM + i) * AM + lr;""")
        if deferred:
            a(f"    const float rs_ = ((const float*)(emh_lds + {rs_off}))[(wm * FM + i) * AM + lr];")
        if m_guard:
            a("    if (m >= M) continue;")
        a(r"""    #pragma unroll
    for (int j = 0; j < FN; ++j)
    #pragma unroll
    for (int g = 0; g < G; ++g) {
      const int n = n0 + (wn * FN + j) * AM + g * 4 * KG + lk * 4;""")
        if n_guard:
            a("      if (n >= N) continue;  // N and tile widths are multiples of 4: a run is all in or all out")
        for i, (_, dt) in enumerate(body.epilogue_operands):
            vt = _pack4_t(dt.name)
            a(f"      const {vt} ev{i} = *(const {vt}*)(e{i} + (long)m * LDO + n);")
        if body.bias is not None:
            bt4 = _pack4_t(body.bias_dtype.name)
            a(f"      const {bt4} bv = *(const {bt4}*)(BIAS + n);")
        a(f"      {vt4} yo;")
        sc = " * rs_" if deferred else ""
        for r in range(4):
            env = {"acc": f"(acc[0][i][j][g * 4 + {r}]{sc})"}
            if gate:
                env["acc2"] = f"(acc[1][i][j][g * 4 + {r}]{sc})"
            if body.bias is not None:
                env["bias"] = f"(float)bv[{r}]"
            pre = E.render(epi, env)
            if body.post is not None:
                env2 = {"y": f"(float){cast}({pre})"}
                for i, (n_, _) in enumerate(body.epilogue_operands):
                    env2[n_] = f"(float)ev{i}[{r}]"
                pre = E.render(post, env2)
            a(f"      yo[{r}] = {cast}({pre});")
        if split is not None and split[1] == "atomic":
            a(f"      float* o_ = O + {body.out_offset}L + OSL + (long)m * LDO + n;")
            a("      #pragma unroll")
            a("      for (int r = 0; r < 4; ++r) __builtin_amdgcn_global_atomic_fadd_f32((__attribute__((address_space(1))) float*)(o_ + r), yo[r]);")
        else:
            a(f"      *({vt4}*)(O + {body.out_offset}L + OSL + (long)m * LDO + n) = yo;")
        a("    }")
        a("  }")
    a("}")

    vm_macro = r"""
// s_waitcnt immediate: vmcnt <= n and lgkmcnt == 0 (gfx9 encoding: vmcnt[3:0] in
// bits 3:0, vmcnt[5:4] in bits 15:14; expcnt left at its maximum, lgkmcnt = 0).
#define EMH_WAIT_VM_LGKM0(n) ((((n) & 0xF) | ((((n) >> 4) & 0x3) << 14)) | 0x0070)
"""
    # The row epilogue's table chunks are requested once the first slab is on its way (loads
    # retire in order: requested earlier, the cold tables would hold up the operands behind them)
    # and are not looked at before the k loop is over.
    tables: list[str] = []
    if rowepi is not None:
        mods = [sym.fields.get(f"row_epilogue.row_operands.{i_}.mod", ro.mod) for i_, ro in enumerate(rowepi.row_operands)] if sym is not None else None
        _emit_row_epilogue_tables(tables.append, rowepi, re_args, EPC, m_guard, mods)
    source = prelude.header(prelude.DMA, vm_macro, *((prelude.WAVE_REDUCE,) if rowepi is not None else ())) + "\n".join(o).replace("ROW_EPILOGUE_TABLES", "\n".join(tables)) + "\n"
    if N % 4 or TN % 4:
        raise LoweringError("contraction: N must be a multiple of 4 (8-byte output runs)")
    n_blocks = (tiles_m // gm) * (tiles_n // gn)
    rounds = -(-n_blocks // ctx.xcds)
    grid = rounds * ctx.xcds * gm * gn
    if m_sym is not None:
        grid = XcdRounds(m_sym, TM, tiles_n // gn, gn, ctx.xcds)
    return HipOp(
        kernel_source=source,
        kernel_name=name,
        arg_order=(
            body.a, body.b, *((pro.weight,) if pro is not None and pro.weight is not None else ()), *((body.bias,) if body.bias is not None else ()),
            *(body.operand_buffers.get(n, n) for n in epi_names), *(rowepi.operand_buffers.get(ro.name, ro.name) for ro in (rowepi.row_operands if rowepi is not None else ())), body.out,
        ),  # fmt: skip
        grid=((grid,), (split[0] if split is not None else batch,), (1,)),
        block=((TT,), (1,), (1,)),
        lds_bytes=lds_bytes,
        zero_outputs=(body.out,) if split is not None and split[1] == "atomic" else (),
        comment=(f"partial of a {split[0]}-way split ({split[1]}) " if split is not None else "") + f"contraction M={M} N={N} K={K} TILE={plan.spell()} STAGE={stage.spell()}" + ((" a=row-scaled-after" if deferred else " a=row-normalised") if pro is not None else "") + (f" row-epilogue={rowepi.col_end // rowepi.cols}x{rowepi.cols}" if rowepi is not None else ""),
        algo_bytes=body.algo_bytes(),
        algo_flops=body.algo_flops(),
        knobs={"TILE": plan.spell(), "STAGE": stage.spell()},
        runtime_args=(sym.name,) if sym is not None and sym.fields else (),
    )


__all__ = ["emit_contraction", "xcd_block", "BF16", "F16"]
