"""Pointwise map emitter: ``out[i] = expr(operands[i])`` over a flat index space.

The per-cell ``Tile`` of the reference (one thread per output cell,
emmy/compiler/ir/kernel/ir.py:159-297; degenerate arm of ``_bind``,
passes/lowering/kernel/_factor.py:329-398) with 16-byte vector accesses and a
grid sized to the index space.
"""

from __future__ import annotations

from deplodock_amd.context import Context
from deplodock_amd.emit import prelude
from deplodock_amd.render_target import rt
from deplodock_amd.emit.errors import LoweringError
from deplodock_amd.emit.reduce import _load_vec, _store_vec
from deplodock_amd.ir import expr as E
from deplodock_amd.ir.hip import HipOp
from deplodock_amd.ir.sym import CeilDiv, c_value, param_name
from deplodock_amd.ir.tile import Map

_T = 256


def emit_map(body: Map, name: str, ctx: Context = Context()) -> HipOp:
    names = [o.name for o in body.operands]
    unknown = E.variables(body.expr) - set(names)
    if unknown:
        raise LoweringError(f"map expression uses unknown names {sorted(unknown)}")
    dts = [body.out_dtype, *(o.dtype for o in body.operands)]
    V = 16 // max(d.nbytes for d in dts)
    offs = [body.operand_offsets.get(o.name, 0) for o in body.operands]
    kinds = {o.index for o in body.operands}
    while V > 1 and (body.numel % V or ((kinds & {"col", "row"}) and body.inner % V) or any(off % V for off, o in zip(offs, body.operands) if o.index in ("flat", "col"))):
        V //= 2
    chunks = body.numel // V
    grid = max(1, -(-chunks // _T))
    # Symbolic extent (``body.sym``): the element count is an expression over the kernel's trailing ``int``
    # parameter; the vector width must divide it at every size, i.e. divide both coefficients.
    sym = getattr(body, "sym", None)
    symf = sym.fields if sym is not None else {}
    chunks_c = str(chunks) + "L"
    if symf:
        if set(symf) != {"numel"}:
            raise LoweringError(f"map: {sorted(symf)} cannot follow a symbolic axis")
        n_sym = symf["numel"]
        while V > 1 and (n_sym.a % V or n_sym.b % V):
            V //= 2
        chunks_c = f"((long){c_value(n_sym)} / {V})"
        grid = CeilDiv(n_sym, V * _T)
    params = [f"const {rt.type_name(o.dtype.name)}* __restrict__ p{i}" for i, o in enumerate(body.operands)]
    params.append(f"{rt.type_name(body.out_dtype.name)}* __restrict__ out")
    if symf:
        params.append(f"int {param_name(sym.name)}")
    o: list[str] = []
    a = o.append
    a(f"// {name}: numel={body.numel} vec={V}")
    a(f'extern "C" __global__ __launch_bounds__({_T}) void {name}({", ".join(params)}) {{')
    a(f"  const long c = (long)blockIdx.x * {_T} + threadIdx.x;")
    a(f"  if (c >= {chunks_c}) return;")
    for i, op in enumerate(body.operands):
        a(f"  float v{i}[{V}];")
        if op.index == "flat":
            o.extend("  " + ln for ln in _load_vec(f"p{i} + {offs[i]}L", "c", op.dtype, V, f"v{i}", False))
        elif op.index == "col":
            o.extend("  " + ln for ln in _load_vec(f"p{i} + {offs[i]}L", f"(c % {body.inner // V}L)", op.dtype, V, f"v{i}", False))
        elif op.index == "row":
            # one value per output row: a vector chunk never straddles rows (inner % V == 0)
            a(f"  {{ const float s_ = (float)p{i}[{offs[i]}L + (c * {V}L) / {body.inner}L]; for (int j = 0; j < {V}; ++j) v{i}[j] = s_; }}")
        elif op.index == "scalar":
            a(f"  {{ const float s_ = (float)p{i}[{offs[i]}L]; for (int j = 0; j < {V}; ++j) v{i}[j] = s_; }}")
        else:
            raise LoweringError(f"map operand index scheme {op.index!r} is not supported")
    a(f"  float y[{V}];")
    for j in range(V):
        env = {op.name: f"v{i}[{j}]" for i, op in enumerate(body.operands)}
        a(f"  y[{j}] = {E.render(body.expr, env)};")
    o.extend("  " + ln for ln in _store_vec("out", "c", body.out_dtype, V, "y", False))
    a("}")
    return HipOp(
        kernel_source=prelude.header() + "\n".join(o) + "\n",
        kernel_name=name,
        arg_order=(*(body.operand_buffers.get(n, n) for n in names), body.out),
        grid=((grid,), (1,), (1,)),
        block=((_T,), (1,), (1,)),
        comment=f"map numel={body.numel}",
        runtime_args=(sym.name,) if symf else (),
        algo_bytes=body.algo_bytes(),
    )
