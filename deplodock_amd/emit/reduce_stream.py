"""Streaming row-reduction emitter: rows too long to keep in registers.

The register-resident form (``emit.reduce``) holds a whole row in the lanes that
own it — at most 64 elements per lane x 1024 lanes.  Beyond that (a softmax over
a 150 k-entry vocabulary) the row is *streamed*: the lanes of one workgroup walk
the row in 16-byte chunks once per statistic level and once more for the
projection, as the reference's cooperative form does (``StridedLoop`` per pass,
emmy/compiler/pipeline/passes/lowering/kernel/_factor.py:652-746), and the
max / sum-of-exponentials pair of softmax is taken in **one** pass with the
online carrier the reference certifies (``m' = max(m, x)``,
``d' = d e^{m-m'} + e^{x-m'}``; emmy/compiler/ir/stmt/carrier.py:279-345,
passes/lowering/tile/_softmax.py:35-123): two reads and one write of the row
instead of three and one.

Lane partials of the online pair combine without a pairwise carrier merge: the
maxima are reduced first, every lane rescales its own ``d`` to the row maximum,
and the rescaled ``d`` are summed — two scalar butterflies.
"""

from __future__ import annotations

from deplodock_amd.context import Context
from deplodock_amd.emit import prelude
from deplodock_amd.render_target import rt
from deplodock_amd.emit.errors import LoweringError
from deplodock_amd.emit.reduce import _load_vec, _row_offset, _store_vec, pick_vec
from deplodock_amd.ir import expr as E
from deplodock_amd.ir.hip import HipOp
from deplodock_amd.ir.tile import RowAddr, RowReduce, Stat


def _online_pair(stats: tuple[Stat, ...], i: int) -> bool:
    """Is ``stats[i], stats[i+1]`` the pair ``m = max x`` / ``d = sum exp(x - m)``?"""
    if i + 1 >= len(stats):
        return False
    m, d = stats[i], stats[i + 1]
    if not (m.monoid == "max" and isinstance(m.pre, E.Var) and m.pre.name == "x" and d.monoid == "sum"):
        return False
    p = d.pre
    return (
        isinstance(p, E.Un) and p.op == "exp" and isinstance(p.a, E.Bin) and p.a.op == "sub"
        and isinstance(p.a.a, E.Var) and p.a.a.name == "x" and isinstance(p.a.b, E.Var) and p.a.b.name == m.name
    )  # fmt: skip


def emit_row_reduce_streaming(body: RowReduce, name: str, ctx: Context = Context()) -> HipOp:
    if getattr(body, "sym", None) is not None and body.sym.fields:
        return _emit_streaming_symbolic_rows(body, name, ctx)
    return _emit_streaming(body, name, ctx)


def _emit_streaming_symbolic_rows(body: RowReduce, name: str, ctx: Context) -> HipOp:
    """One workgroup per row whatever the row count: the kernel never reads it, only the launch size follows it."""
    sym = body.sym
    if set(sym.fields) != {"rows"}:
        raise LoweringError(f"streamed row reduce: {sorted(sym.fields)} cannot follow a symbolic axis")
    op = _emit_streaming(body, name, ctx)
    op.grid = ((sym.fields["rows"],), (1,), (1,))
    return op


def _emit_streaming(body: RowReduce, name: str, ctx: Context = Context()) -> HipOp:
    if body.rotate is not None or body.row_operands:
        raise LoweringError("row reduce: the streaming form has no rotate-half / per-row tables")
    x_addr = body.x_addr or RowAddr.uniform(body.cols)
    out_addr = body.out_addr or RowAddr.uniform(1 if body.scalar_out else body.cols)
    T = min(1024, ctx.max_threads_per_block)  # one workgroup per row
    V = pick_vec(body.cols, [body.x_dtype, body.out_dtype, *(dt for _, dt in body.col_operands)], [x_addr] + ([] if body.scalar_out else [out_addr]))
    C = body.cols // V
    NW = T // ctx.wave_size
    stat_names = [s.name for s in body.stats]
    for s_i, st in enumerate(body.stats):
        unknown = E.variables(st.pre) - ({"x"} | set(stat_names[:s_i]))
        if unknown:
            raise LoweringError(f"stat {st.name!r}: pre-map uses unknown names {sorted(unknown)}")
    col_names = [n for n, _ in body.col_operands]
    unknown = E.variables(body.project) - (set(stat_names) | (set() if body.scalar_out else {"x"} | set(col_names)))
    if unknown:
        raise LoweringError(f"projection uses unknown names {sorted(unknown)}")

    # Passes: statistics in dependency order; an online pair shares one pass.
    passes: list[list[int]] = []
    i = 0
    while i < len(body.stats):
        if _online_pair(body.stats, i):
            passes.append([i, i + 1])
            i += 2
            continue
        # independent statistics that only need already-finished ones ride together
        group = [i]
        done = set(stat_names[:i])
        j = i + 1
        while j < len(body.stats) and not _online_pair(body.stats, j) and E.variables(body.stats[j].pre) - {"x"} <= done:
            group.append(j)
            j += 1
        passes.append(group)
        i = j

    params = [f"const {rt.type_name(body.x_dtype.name)}* __restrict__ x"]
    params += [f"const {rt.type_name(dt.name)}* __restrict__ c{ci}" for ci, (_, dt) in enumerate(body.col_operands)]
    params.append(f"{rt.type_name(body.out_dtype.name)}* __restrict__ out")
    o: list[str] = []
    a = o.append
    a(f"// {name}: rows={body.rows} cols={body.cols} streamed by {T} lanes, vec={V}, {len(passes)} statistic pass(es)")
    a(f'extern "C" __global__ __launch_bounds__({T}) void {name}({", ".join(params)}) {{')
    a("  const int lane = threadIdx.x;")
    a(f"  const int wave = lane / {ctx.wave_size};")
    a("  const long row = blockIdx.x;")
    a(f"  const {rt.type_name(body.x_dtype.name)}* xr = x + ({_row_offset(x_addr, 'row')});")
    a(f"  __shared__ float emh_part[{NW}];")
    a("  float xv[%d];" % V)

    def block_reduce(var: str, mono: str) -> None:
        """All lanes end with the workgroup-wide reduction of ``var``."""
        a(f"  {var} = emh_wave_reduce<{mono}, {ctx.wave_size}>({var});")
        a(f"  if (lane % {ctx.wave_size} == 0) emh_part[wave] = {var};")
        a("  __syncthreads();")
        a(f"  {var} = emh_part[0];")
        a(f"  for (int w = 1; w < {NW}; ++w) {var} = {mono}::op({var}, emh_part[w]);")
        a("  __syncthreads();")

    env_done: dict[str, str] = {}
    for group in passes:
        stats = [body.stats[g] for g in group]
        online = len(group) == 2 and _online_pair(body.stats, group[0])
        for st in stats:
            mono = prelude.MONOID_STRUCT[st.monoid]
            a(f"  float s_{st.name} = {mono}::identity();")
        a(f"  for (int c = lane; c < {C}; c += {T}) {{")
        o.extend("    " + ln for ln in _load_vec("xr", "c", body.x_dtype, V, "xv", False))
        if online:
            m, d = stats
            a("    float cm = xv[0];")
            a(f"    for (int j = 1; j < {V}; ++j) cm = fmaxf(cm, xv[j]);")
            a(f"    const float m_new = fmaxf(s_{m.name}, cm);")
            a("    // -inf scores (masked logits) are legal: guard the inf - inf forms")
            a(f"    float acc = s_{d.name} * (s_{m.name} == m_new ? 1.0f : expf(s_{m.name} - m_new));")
            a(f"    if (m_new > -__builtin_inff()) for (int j = 0; j < {V}; ++j) acc += expf(xv[j] - m_new);")
            a(f"    s_{m.name} = m_new; s_{d.name} = acc;")
        else:
            for st in stats:
                mono = prelude.MONOID_STRUCT[st.monoid]
                for j in range(V):
                    xj = f"xv[{j}]"
                    for prev in body.stats:
                        if prev.keep and prev.name in env_done:
                            xj = f"({E.render(prev.pre, dict(env_done, x=xj))})"
                    env = dict(env_done, x=xj)
                    a(f"    s_{st.name} = {mono}::op(s_{st.name}, {E.render(st.pre, env)});")
        a("  }")
        if online:
            m, d = stats
            a(f"  const float lane_m_{m.name} = s_{m.name};")
            block_reduce(f"s_{m.name}", "EmhMax")
            a(f"  s_{d.name} *= (lane_m_{m.name} == s_{m.name} ? 1.0f : expf(lane_m_{m.name} - s_{m.name}));  // a lane that saw no chunk holds d = 0")
            block_reduce(f"s_{d.name}", "EmhSum")
        else:
            for st in stats:
                block_reduce(f"s_{st.name}", prelude.MONOID_STRUCT[st.monoid])
        for st in stats:
            env_done[st.name] = f"s_{st.name}"

    if body.scalar_out:
        cast = "" if body.out_dtype.name == "f32" else f"({rt.type_name(body.out_dtype.name)})"
        a(f"  if (lane == 0) out[{_row_offset(out_addr, 'row')}] = {cast}({E.render(body.project, env_done)});")
    else:
        a(f"  {rt.type_name(body.out_dtype.name)}* orow = out + ({_row_offset(out_addr, 'row')});")
        a(f"  for (int c = lane; c < {C}; c += {T}) {{")
        o.extend("    " + ln for ln in _load_vec("xr", "c", body.x_dtype, V, "xv", False))
        for ci, (_, dt) in enumerate(body.col_operands):
            a(f"    float cv{ci}[{V}];")
            o.extend("    " + ln for ln in _load_vec(f"c{ci}", "c", dt, V, f"cv{ci}", False))
        a(f"    float y[{V}];")
        for j in range(V):
            # a statistic that keeps its pre-map (softmax's exp(x - m)) redefines x for what follows
            for st in body.stats:
                if st.keep:
                    a(f"    xv[{j}] = {E.render(st.pre, dict(env_done, x=f'xv[{j}]'))};")
            env = dict(env_done, x=f"xv[{j}]")
            env.update({n: f"cv{ci}[{j}]" for ci, n in enumerate(col_names)})
            a(f"    y[{j}] = {E.render(body.project, env)};")
        o.extend("    " + ln for ln in _store_vec("orow", "c", body.out_dtype, V, "y", False))
        a("  }")
    a("}")
    reads = len(passes) + (0 if body.scalar_out else 1)
    return HipOp(
        kernel_source=prelude.header(prelude.WAVE_REDUCE) + "\n".join(o) + "\n",
        kernel_name=name,
        arg_order=(body.x, *(body.operand_buffers.get(n, n) for n in col_names), body.out),
        grid=((body.rows,), (1,), (1,)),
        block=((T,), (1,), (1,)),
        lds_bytes=0,
        comment=f"row_reduce rows={body.rows} cols={body.cols} streamed ({reads} reads of the row)",
        algo_bytes=body.algo_bytes(),
        knobs={"REDUCE": f"b{T}/stream", "VEC": V, "NT": 0},
    )
