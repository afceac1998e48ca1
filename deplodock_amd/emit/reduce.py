"""Row-reduction emitter: fused statistic(s) + projection kernels for gfx950.

Covers what the reference builds from ``_tile_reduce_axis`` / ``emit_combine``
(emmy/compiler/pipeline/passes/lowering/kernel/_factor.py:467-521, 652-746)
plus ``WarpShuffle`` / ``TreeHalve`` (emmy/compiler/ir/kernel/ir.py:569-702),
designed for wave64 instead of translated:

* ``coop`` lanes own one row.  Each lane keeps its slice of the row **resident
  in registers** (16-byte vector loads, lane-interleaved so every wave-load is
  one contiguous run), so the row is read from HBM exactly once however many
  statistics are taken — the reference's cooperative form re-reads the row per
  pass (``StridedLoop`` per statistic, _factor.py:652-746).
* Lane partials combine with DPP / swizzle / permlane butterflies only
  (``prelude.WAVE_REDUCE``).  Rows wider than one wave add a single LDS
  hand-off of ``coop/64`` partials per statistic — never a log-tree of
  barriers.
* A statistic's pre-map may replace the resident element (``Stat.keep``):
  softmax stores ``exp(x - max)`` once and the projection only scales it.
"""

from __future__ import annotations

from deplodock_amd.context import Context
from deplodock_amd.dtype import BF16, F16, DType
from deplodock_amd.emit import prelude
from deplodock_amd.render_target import rt
from deplodock_amd.emit.errors import LoweringError
from deplodock_amd.ir import expr as E
from deplodock_amd.ir.hip import HipOp
from deplodock_amd.ir.sym import CeilDiv, c_value, param_name
from deplodock_amd.ir.tile import RowAddr, RowReduce

_MAX_RESIDENT = 64  # fp32 row elements a lane may keep in registers

def _vec_t(dt: DType, v: int) -> str:
    """C type of ``v`` elements of ``dt`` moved by one access."""
    got = rt.vector_type(dt.name, v)
    if got is None:
        raise LoweringError(f"row kernel: no {v}-wide vector of {dt}")
    return got[0]


def pick_vec(cols: int, dtypes: list[DType], addrs: list[RowAddr]) -> int:
    """Widest element count per access such that the widest dtype moves 16 bytes
    and every row start stays aligned."""
    v = 16 // max(d.nbytes for d in dtypes)
    while v > 1 and cols % v:
        v //= 2
    for a in addrs:
        v = a.max_vec(v)
    return v


def _row_offset(addr: RowAddr, row: str) -> str:
    if addr.div == 1:
        return f"{addr.offset}L + {row} * {addr.stride_hi}L"
    return f"{addr.offset}L + ({row} / {addr.div}) * {addr.stride_hi}L + ({row} % {addr.div}) * {addr.stride_lo}L"


def _load_vec(ptr: str, idx: str, dt: DType, v: int, dst: str, nontemporal: bool) -> list[str]:
    """Lines that load ``v`` elements of ``dt`` at vector index ``idx`` into ``float dst[v]``."""
    vt = _vec_t(dt, v)
    addr = f"((const {vt}*)({ptr}))[{idx}]" if v > 1 else f"({ptr})[{idx}]"
    if nontemporal:
        addr = f"__builtin_nontemporal_load(&{addr})"
    if v == 1:
        return [f"{dst}[0] = {rt.convert(addr, dt.name, 'f32')};"]
    lines = [f"{{ {vt} t_ = {addr};"]
    lines += [f"  {dst}[{j}] = {rt.convert(f't_[{j}]', dt.name, 'f32')};" for j in range(v)]
    lines.append("}")
    return lines


def _store_vec(ptr: str, idx: str, dt: DType, v: int, src: str, nontemporal: bool) -> list[str]:
    vt = _vec_t(dt, v)
    cast = lambda x: rt.convert(x, "f32", dt.name)  # noqa: E731
    if v == 1:
        tgt = f"({ptr})[{idx}]"
        val = cast(f"{src}[0]")
        return [f"__builtin_nontemporal_store({val}, &{tgt});" if nontemporal else f"{tgt} = {val};"]
    lines = [f"{{ {vt} t_;"]
    lines += [f"  t_[{j}] = {cast(f'{src}[{j}]')};" for j in range(v)]
    tgt = f"(({vt}*)({ptr}))[{idx}]"
    lines.append(f"  __builtin_nontemporal_store(t_, &{tgt});" if nontemporal else f"  {tgt} = t_;")
    lines.append("}")
    return lines


def emit_row_reduce(body: RowReduce, name: str, ctx: Context = Context()) -> HipOp:
    """Render ``body`` (schedule already stamped on ``body.reduce``) to a HipOp."""
    plan = body.reduce
    L = plan.coop
    nontemporal = body.nontemporal
    if plan.cta != 1:
        raise LoweringError("row reduce: cross-workgroup split (g<n>) is not defined for a projected row")
    x_addr = body.x_addr or RowAddr.uniform(body.cols)
    out_addr = body.out_addr or RowAddr.uniform(body.cols)
    col_dts = [dt for _, dt in body.col_operands]
    row_dts = [ro.dtype for ro in body.row_operands]
    V = pick_vec(body.cols, [body.x_dtype, body.out_dtype, *col_dts, *row_dts], [x_addr, out_addr])
    for ro in body.row_operands:
        while V > 1 and ro.offset % V:
            V //= 2
    if body.rotate is not None:
        while V > 1 and (body.cols // V) % 2:
            V //= 2  # each half of the row is whole vectors (head_dim 40 in bf16: ten chunks of four, not five of eight)
    C = body.cols // V  # vector chunks per row
    if body.rotate is not None:
        if C % 2:
            raise LoweringError("row reduce: rotate-half needs an even number of vector chunks per row")
        if (C // 2) % L:
            raise LoweringError(f"row reduce: rotate-half keeps both halves in one lane, which needs REDUCE b<n> with n dividing {C // 2}")
    NV = -(-C // L)  # chunks per lane
    if NV * V > _MAX_RESIDENT:
        raise LoweringError(
            f"row reduce: {body.cols} columns over {L} lanes needs {NV * V} resident elements per lane "
            f"(> {_MAX_RESIDENT}); widen REDUCE b<n>"
        )
    masked = C % L != 0
    T = max(L, min(256, ctx.max_threads_per_block))
    if body.rows_per_block is not None:
        T = L * body.rows_per_block
    if T > ctx.max_threads_per_block or T % L:
        raise LoweringError(f"row reduce: {T} threads per workgroup is not launchable")
    R = T // L
    # Symbolic row count (``body.sym``): rows and table extents become expressions over the kernel's trailing
    # ``int`` parameter, the row guard is always there and the grid is sized at launch.
    sym = getattr(body, "sym", None)
    symf = sym.fields if sym is not None else {}
    for key in symf:
        if key != "rows" and not (key.startswith("row_operands.") and key.endswith(".mod")):
            raise LoweringError(f"row reduce: {key} cannot follow a symbolic axis")
    rows_c = c_value(symf.get("rows", body.rows))
    # Do not spread fewer rows than one workgroup holds over idle lanes.
    while "rows" not in symf and R > 1 and R > body.rows and T > ctx.wave_size:
        R //= 2
        T = L * R
    grid = CeilDiv(symf["rows"], R) if "rows" in symf else -(-body.rows // R)
    row_guard = "rows" in symf or body.rows % R != 0
    NW = max(1, L // ctx.wave_size)  # waves per row
    W = min(L, ctx.wave_size)  # butterfly width

    stat_names = [s.name for s in body.stats]
    operand_names = [n for n, _ in body.col_operands] + [ro.name for ro in body.row_operands]
    for s_i, st in enumerate(body.stats):
        unknown = E.variables(st.pre) - ({"x"} | set(stat_names[:s_i]))
        if unknown:
            raise LoweringError(f"stat {st.name!r}: pre-map uses unknown names {sorted(unknown)}")
    unknown = E.variables(body.project) - ({"x"} | set(stat_names) | set(operand_names))
    if unknown:
        raise LoweringError(f"projection uses unknown names {sorted(unknown)}")
    if body.rotate is not None:
        unknown = E.variables(body.rotate.expr) - ({"y", "yr"} | set(stat_names) | set(operand_names))
        if unknown:
            raise LoweringError(f"rotate-half expression uses unknown names {sorted(unknown)}")

    params = [f"const {rt.type_name(body.x_dtype.name)}* __restrict__ x"]
    params += [f"const {rt.type_name(dt.name)}* __restrict__ c{ci}" for ci, (_, dt) in enumerate(body.col_operands)]
    params += [f"const {rt.type_name(ro.dtype.name)}* __restrict__ r{ri}" for ri, ro in enumerate(body.row_operands)]
    params.append(f"{rt.type_name(body.out_dtype.name)}* __restrict__ out")
    if symf:
        params.append(f"int {param_name(sym.name)}")

    o: list[str] = []
    a = o.append
    a(f"// {name}: rows={body.rows} cols={body.cols} REDUCE={plan.spell() or 'serial'} vec={V} rows/wg={R}")
    a(f'extern "C" __global__ __launch_bounds__({T}) void {name}({", ".join(params)}) {{')
    a(f"  const int lane = threadIdx.x % {L};")
    a(f"  const int rib = threadIdx.x / {L};")
    a(f"  long row = (long)blockIdx.x * {R} + rib;")
    if row_guard:
        a(f"  const bool row_ok = row < (long){rows_c};")
        a(f"  if (!row_ok) row = (long){rows_c} - 1;")
    a(f"  const {rt.type_name(body.x_dtype.name)}* xr = x + ({_row_offset(x_addr, 'row')});")
    a(f"  float xv[{NV}][{V}];")
    if masked:
        a(f"  bool ok[{NV}];")
    for i in range(NV):
        idx = f"{i * L} + lane"
        if masked and (i + 1) * L > C:
            a(f"  ok[{i}] = ({idx}) < {C};")
            a(f"  if (ok[{i}]) {{")
            o.extend("    " + ln for ln in _load_vec("xr", idx, body.x_dtype, V, f"xv[{i}]", nontemporal))
            a("  } else {")
            a(f"    for (int j = 0; j < {V}; ++j) xv[{i}][j] = 0.0f;")
            a("  }")
        else:
            if masked:
                a(f"  ok[{i}] = true;")
            o.extend("  " + ln for ln in _load_vec("xr", idx, body.x_dtype, V, f"xv[{i}]", nontemporal))

    if not body.scalar_out:
        for ri, ro in enumerate(body.row_operands):
            mod = c_value(symf.get(f"row_operands.{ri}.mod", ro.mod))
            a(f"  const {rt.type_name(ro.dtype.name)}* rrow{ri} = r{ri} + {ro.offset}L + ((row / {ro.div}) % {mod}) * {body.cols}L;")

    def operand_loads(i: int, indent: str, tag: str = "") -> None:
        idx = f"{i * L} + lane"
        for ci, (_, dt) in enumerate(body.col_operands):
            a(f"{indent}float cv{ci}{tag}[{V}];")
            o.extend(indent + ln for ln in _load_vec(f"c{ci}", idx, dt, V, f"cv{ci}{tag}", False))
        for ri, ro in enumerate(body.row_operands):
            a(f"{indent}float rv{ri}{tag}[{V}];")
            o.extend(indent + ln for ln in _load_vec(f"rrow{ri}", idx, ro.dtype, V, f"rv{ri}{tag}", False))

    def operand_env(j: int, tag: str = "") -> dict[str, str]:
        env = {n: f"cv{ci}{tag}[{j}]" for ci, (n, _) in enumerate(body.col_operands)}
        env.update({ro.name: f"rv{ri}{tag}[{j}]" for ri, ro in enumerate(body.row_operands)})
        return env

    # The projection's other operands do not depend on the statistics: requested here, with the row, they
    # arrive while the statistics are reduced instead of costing a second memory round trip after them.
    n_operands = len(body.col_operands) + len(body.row_operands)
    hoist = bool(body.stats) and not body.scalar_out and body.rotate is None and 0 < n_operands * NV * V <= 32
    if hoist:
        for i in range(NV):
            if masked and (i + 1) * L > C:
                for ci in range(len(body.col_operands)):
                    a(f"  float cv{ci}_{i}[{V}] = {{}};")
                for ri in range(len(body.row_operands)):
                    a(f"  float rv{ri}_{i}[{V}] = {{}};")
                a(f"  if (ok[{i}]) {{")
                mark = len(o)
                operand_loads(i, "    ", f"_{i}")
                o[mark:] = [ln for ln in o[mark:] if not ln.strip().startswith("float ")]
                a("  }")
            else:
                operand_loads(i, "  ", f"_{i}")

    if NW > 1 and body.stats:
        a(f"  __shared__ float emh_part[{len(body.stats)}][{R}][{NW}];")
        a(f"  const int wave_in_row = lane / {ctx.wave_size};")

    env_base = {s: f"s_{s}" for s in stat_names}
    for s_i, st in enumerate(body.stats):
        mono = prelude.MONOID_STRUCT[st.monoid]
        nacc = max(1, min(plan.reg, NV * V))
        a(f"  float acc_{st.name}[{nacc}];")
        a(f"  for (int r = 0; r < {nacc}; ++r) acc_{st.name}[r] = {mono}::identity();")
        e_idx = 0
        for i in range(NV):
            guard = f"if (ok[{i}]) " if masked and (i + 1) * L > C else ""
            a(f"  {guard}{{")
            for j in range(V):
                env = dict(env_base, x=f"xv[{i}][{j}]")
                val = E.render(st.pre, env)
                r = e_idx % nacc
                if st.keep:
                    a(f"    xv[{i}][{j}] = {val};")
                    val = f"xv[{i}][{j}]"
                a(f"    acc_{st.name}[{r}] = {mono}::op(acc_{st.name}[{r}], {val});")
                e_idx += 1
            a("  }")
        a(f"  float s_{st.name} = acc_{st.name}[0];")
        for r in range(1, nacc):
            a(f"  s_{st.name} = {mono}::op(s_{st.name}, acc_{st.name}[{r}]);")
        a(f"  s_{st.name} = emh_wave_reduce<{mono}, {W}>(s_{st.name});")
        if NW > 1:
            a(f"  if ((lane % {ctx.wave_size}) == 0) emh_part[{s_i}][rib][wave_in_row] = s_{st.name};")
            a("  __syncthreads();")
            a(f"  s_{st.name} = emh_part[{s_i}][rib][0];")
            for w in range(1, NW):
                a(f"  s_{st.name} = {mono}::op(s_{st.name}, emh_part[{s_i}][rib][{w}]);")

    if body.scalar_out:
        # plain row reduction: every lane holds the statistics; one of them stores the row's value
        bad = E.variables(body.project) - set(stat_names)
        if bad or body.rotate is not None or body.col_operands or body.row_operands:
            raise LoweringError(f"row reduce: a one-value-per-row output maps the statistics only (got {sorted(bad)})")
        cast_ = "" if body.out_dtype.name == "f32" else f"({rt.type_name(body.out_dtype.name)})"
        a(f"  if (lane == 0{' && row_ok' if row_guard else ''}) out[row] = {cast_}({E.render(body.project, env_base)});")
        a("}")
        return HipOp(
            kernel_source=prelude.header(prelude.WAVE_REDUCE) + "\n".join(o) + "\n",
            kernel_name=name,
            arg_order=(body.x, body.out),
            grid=((grid,), (1,), (1,)),
            block=((T,), (1,), (1,)),
            lds_bytes=0,
            comment=f"row_reduce rows={body.rows} cols={body.cols} REDUCE={plan.spell()} one value per row",
            algo_bytes=body.algo_bytes(),
            knobs={"REDUCE": plan.spell(), "VEC": V, "NT": int(nontemporal)},
            runtime_args=(sym.name,) if symf else (),
        )
    a(f"  {rt.type_name(body.out_dtype.name)}* orow = out + ({_row_offset(out_addr, 'row')});")

    if row_guard:
        a("  if (row_ok) {")
    if body.rotate is None:
        for i in range(NV):
            idx = f"{i * L} + lane"
            guard = f"if (ok[{i}]) " if masked and (i + 1) * L > C else ""
            a(f"  {guard}{{")
            a(f"    float y[{V}];")
            if not hoist:
                operand_loads(i, "    ")
            for j in range(V):
                env = dict(env_base, x=f"xv[{i}][{j}]", **operand_env(j, f"_{i}" if hoist else ""))
                a(f"    y[{j}] = {E.render(body.project, env)};")
            o.extend("    " + ln for ln in _store_vec("orow", idx, body.out_dtype, V, "y", nontemporal))
            a("  }")
    else:
        # Phase 1: project the whole resident row; phase 2: combine each element
        # with its half-rotated partner, which lives in the same lane (the lane
        # count divides half the chunks), NV/2 chunks away.
        half = NV // 2
        in_project = E.variables(body.project)
        in_rotate = E.variables(body.rotate.expr)
        a(f"  float yv[{NV}][{V}];")
        for i in range(NV):
            a("  {")
            for ci, (_, dt) in enumerate(body.col_operands):
                a(f"    float cv{ci}[{V}];")
                o.extend("    " + ln for ln in _load_vec(f"c{ci}", f"{i * L} + lane", dt, V, f"cv{ci}", False))
            for ri, ro in enumerate(body.row_operands):
                if ro.name in in_project:
                    a(f"    float rv{ri}[{V}];")
                    o.extend("    " + ln for ln in _load_vec(f"rrow{ri}", f"{i * L} + lane", ro.dtype, V, f"rv{ri}", False))
            for j in range(V):
                env = dict(env_base, x=f"xv[{i}][{j}]")
                env.update({n: f"cv{ci}[{j}]" for ci, (n, _) in enumerate(body.col_operands)})
                env.update({ro.name: f"rv{ri}[{j}]" for ri, ro in enumerate(body.row_operands) if ro.name in in_project})
                a(f"    yv[{i}][{j}] = {E.render(body.project, env)};")
            a("  }")
        for i in range(NV):
            idx = f"{i * L} + lane"
            a("  {")
            a(f"    float y[{V}];")
            for ri, ro in enumerate(body.row_operands):
                if ro.name in in_rotate:
                    a(f"    float rv{ri}[{V}];")
                    o.extend("    " + ln for ln in _load_vec(f"rrow{ri}", idx, ro.dtype, V, f"rv{ri}", False))
            for j in range(V):
                partner = f"(-yv[{i + half}][{j}])" if i < half else f"yv[{i - half}][{j}]"
                env = dict(env_base, y=f"yv[{i}][{j}]", yr=partner)
                env.update({ro.name: f"rv{ri}[{j}]" for ri, ro in enumerate(body.row_operands) if ro.name in in_rotate})
                a(f"    y[{j}] = {E.render(body.rotate.expr, env)};")
            o.extend("    " + ln for ln in _store_vec("orow", idx, body.out_dtype, V, "y", nontemporal))
            a("  }")
    if row_guard:
        a("  }")
    a("}")

    source = prelude.header(prelude.WAVE_REDUCE) + "\n".join(o) + "\n"
    return HipOp(
        kernel_source=source,
        kernel_name=name,
        arg_order=(
            body.x,
            *(body.operand_buffers.get(n, n) for n, _ in body.col_operands),
            *(body.operand_buffers.get(ro.name, ro.name) for ro in body.row_operands),
            body.out,
        ),
        grid=((grid,), (1,), (1,)),
        block=((T,), (1,), (1,)),
        lds_bytes=0,
        comment=f"row_reduce rows={body.rows} cols={body.cols} REDUCE={plan.spell()}",
        algo_bytes=body.algo_bytes(),
        knobs={"REDUCE": plan.spell(), "VEC": V, "NT": int(nontemporal)},
        runtime_args=(sym.name,) if symf else (),
    )


__all__ = ["emit_row_reduce", "pick_vec", "BF16", "F16"]
