"""Loop-nest emitter: a Loop-IR body rendered loop for loop, one wave per point of its outer loops.

This is the tier below the tiled kernels — the counterpart of what the reference does with a ``LoopOp`` it has no
tile plan for: render the statements as they stand (emmy/compiler/ir/loop/ir.py:193-221 renders them to plain
C++ loops).  It exists so that every kernel of the reference's on-disk corpus (``kernels/*.json``: post-fusion,
pre-tiling Loop IR) runs on this backend with the reference's semantics; nests that are a contraction or a row
normalisation in disguise are raised to the tiled kernels before they get here (``passes/raise_loops.py``).

Mapping onto the machine:

* the *outer chain* — loops that hold nothing but (pure statements and) one further loop, and fold nothing
  themselves — becomes the launch: one 64-lane wave per point, four waves to a workgroup, no LDS, no barrier;
* below the chain a loop that holds further loops runs on every lane alike; a *leaf* loop is dealt over the lanes
  (iteration ``lane, lane + 64, ...``), and what it folds (``Accum``) is combined across the wave by a butterfly,
  after which every lane holds the result;
* a leaf loop without folds that ends the nest is also dealt over several waves when the chain alone is too few
  points to fill the machine;
* a ``Write`` outside a dealt loop is done by lane 0.

Arithmetic is fp32 whatever the operand types (loads widen, the store rounds), index arithmetic is 32-bit with
floor division and modulo (emmy/compiler/ir/expr.py:125-148).  Every index expression is evaluated over its
iteration space on the host when the kernel is built, and a body that would read or write outside an operand is
refused there — nothing is left to fault on the GPU.
"""

from __future__ import annotations

import math

import numpy as np

from deplodock_amd.context import Context
from deplodock_amd.emit import prelude
from deplodock_amd.emit.errors import LoweringError
from deplodock_amd.ir import loopnest as L
from deplodock_amd.ir.expr import float_literal
from deplodock_amd.ir.hip import HipOp
from deplodock_amd.ir.tile import LoopNest
from deplodock_amd.render_target import rt

_WAVES = 4  # waves per workgroup
_MAX_INDEX_POINTS = 1 << 24  # host-side bounds check: the largest index space an expression is evaluated over (int64: 128 MiB a temporary)

_HELPERS = r"""
EMH_DEV int emh_fdiv(int a, int b) { const int q = a / b, r = a % b; return (r != 0 && ((r < 0) != (b < 0))) ? q - 1 : q; }
EMH_DEV int emh_fmod(int a, int b) { const int r = a % b; return (r != 0 && ((r < 0) != (b < 0))) ? r + b : r; }
EMH_DEV float emh_ln_add(float v) { for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64); return v; }
EMH_DEV float emh_ln_multiply(float v) { for (int o = 32; o > 0; o >>= 1) v *= __shfl_xor(v, o, 64); return v; }
EMH_DEV float emh_ln_maximum(float v) { for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64)); return v; }
EMH_DEV float emh_ln_minimum(float v) { for (int o = 32; o > 0; o >>= 1) v = fminf(v, __shfl_xor(v, o, 64)); return v; }
"""

_UNARY_C = {
    "negative": "(-{0})", "reciprocal": "(1.0f / {0})", "rsqrt": "(1.0f / sqrtf({0}))", "sqrt": "sqrtf({0})", "exp": "expf({0})", "log": "logf({0})",
    "tanh": "tanhf({0})", "sigmoid": "(1.0f / (1.0f + expf(-{0})))", "silu": "({0} / (1.0f + expf(-{0})))", "abs": "fabsf({0})", "relu": "fmaxf({0}, 0.0f)",
    "square": "({0} * {0})",
}  # fmt: skip
_BINARY_C = {"add": "({0} + {1})", "subtract": "({0} - {1})", "multiply": "({0} * {1})", "divide": "({0} / {1})", "maximum": "fmaxf({0}, {1})", "minimum": "fminf({0}, {1})"}
_IDENTITY_C = {"add": "0.0f", "multiply": "1.0f", "maximum": "(-__builtin_inff())", "minimum": "__builtin_inff()"}


def _is_leaf(loop: L.Loop) -> bool:
    return not any(isinstance(s, L.Loop) for s in loop.body)


def _folds(loop: L.Loop) -> list[L.Accum]:
    seen: dict[str, L.Accum] = {}
    for s in loop.body:
        if isinstance(s, L.Accum):
            seen.setdefault(s.name, s)
    return list(seen.values())


def _v(name: str) -> str:
    return "v_" + "".join(ch if ch.isalnum() or ch == "_" else "_" for ch in name)


def _ax(name: str) -> str:
    return "i_" + "".join(ch if ch.isalnum() or ch == "_" else "_" for ch in name)


def _index_c(e) -> str:
    if isinstance(e, L.Var):
        return _ax(e.name)
    if isinstance(e, L.Lit):
        if isinstance(e.value, float) and not float(e.value).is_integer():
            raise LoweringError(f"loop nest: index literal {e.value!r} is not an integer")
        return str(int(e.value))
    if isinstance(e, L.Ternary):
        return f"(({_index_c(e.cond)}) ? ({_index_c(e.if_true)}) : ({_index_c(e.if_false)}))"
    a, b = _index_c(e.left), _index_c(e.right)
    if e.op in ("/", "//"):
        return f"emh_fdiv({a}, {b})"
    if e.op == "%":
        return f"emh_fmod({a}, {b})"
    return f"(({a}) {e.op} ({b}))"


def _index_np(e, env):
    if isinstance(e, L.Var):
        return env[e.name]
    if isinstance(e, L.Lit):
        return int(e.value)
    if isinstance(e, L.Ternary):
        return np.where(_index_np(e.cond, env), _index_np(e.if_true, env), _index_np(e.if_false, env))
    a, b = _index_np(e.left, env), _index_np(e.right, env)
    ops = {"+": np.add, "-": np.subtract, "*": np.multiply, "/": np.floor_divide, "//": np.floor_divide, "%": np.mod, "<": np.less, "<=": np.less_equal,
           ">": np.greater, ">=": np.greater_equal, "==": np.equal, "&&": np.logical_and, "||": np.logical_or}  # fmt: skip
    return ops[e.op](a, b)


def _check_bounds(what: str, index: tuple, shape: tuple[int, ...], extents: dict[str, int]) -> None:
    """Every index of ``what`` stays inside ``shape`` over the whole iteration space (evaluated, not estimated)."""
    if len(index) != len(shape):
        raise LoweringError(f"loop nest: {what} has {len(index)} indices for a rank-{len(shape)} tensor")
    for d, (e, dim) in enumerate(zip(index, shape)):
        if isinstance(e, L.Var):  # a bare axis: no need to enumerate it
            lo, hi = 0, extents[e.name] - 1
        elif isinstance(e, L.Lit):
            lo = hi = int(e.value)
        else:
            names = sorted(L.expr_vars(e))
            points = math.prod(extents[n] for n in names)
            if points > _MAX_INDEX_POINTS:
                raise LoweringError(f"loop nest: {what} index {d} is an expression over {points} points; too many to check")
            env = {n: np.arange(extents[n], dtype=np.int64).reshape([extents[n] if m == n else 1 for m in names]) for n in names}
            vals = np.asarray(_index_np(e, env), dtype=np.int64)
            lo, hi = int(vals.min()), int(vals.max())
        if lo < 0 or hi >= dim:
            raise LoweringError(f"loop nest: {what} index {d} spans [{lo}, {hi}] outside [0, {dim})")
        if max(abs(lo), abs(hi)) * 2 >= 2**31:
            raise LoweringError(f"loop nest: {what} index {d} overflows 32-bit index arithmetic")


def _max_intermediate(e, extents: dict[str, int]) -> int:
    """Largest magnitude any sub-expression of ``e`` takes (interval bound), to keep index arithmetic in 32 bits."""
    if isinstance(e, L.Var):
        return extents[e.name] - 1
    if isinstance(e, L.Lit):
        return abs(int(e.value))
    if isinstance(e, L.Ternary):
        return max(_max_intermediate(e.if_true, extents), _max_intermediate(e.if_false, extents), _max_intermediate(e.cond, extents))
    a, b = _max_intermediate(e.left, extents), _max_intermediate(e.right, extents)
    if e.op in ("+", "-"):
        return a + b
    if e.op == "*":
        return a * b
    return max(a, b)


def emit_loop_nest(body: LoopNest, name: str, ctx: Context = Context()) -> HipOp:
    stmts = body.stmts
    L.check_body(stmts)
    operands = body.operands  # Load.input name -> (buffer id, shape, dtype)
    order = list(dict.fromkeys(buf for buf, _, _ in operands.values()))  # kernel parameters, one per distinct buffer
    param_of = {buf: f"p{i}" for i, buf in enumerate(order)}
    dtype_of = {buf: dt for buf, _, dt in operands.values()}

    # ---- the outer chain: loops that only wrap one further loop ------------------------------------------------
    chain: list[L.Loop] = []
    pre: list[list] = []  # pure statements in front of each chain loop (evaluated again by every wave)
    cur = stmts
    while True:
        loops = [s for s in cur if isinstance(s, L.Loop)]
        if len(loops) != 1 or cur[-1] is not loops[0] or any(isinstance(s, (L.Write, L.Accum)) for s in cur):
            break
        loop = loops[0]
        if _is_leaf(loop) or _folds(loop):
            break
        pre.append([s for s in cur if s is not loop])
        chain.append(loop)
        cur = loop.body
    tail = cur
    points = math.prod(l_.extent for l_ in chain)

    # a closing leaf loop without folds can be dealt over several waves
    split = 1
    last = tail[-1] if tail else None
    if isinstance(last, L.Loop) and _is_leaf(last) and not _folds(last) and sum(isinstance(s, L.Loop) for s in tail) == 1:
        want = -(-(ctx.compute_units * 8) // max(points, 1))  # about eight waves per CU
        split = max(1, min(want, -(-last.extent // 64)))
    waves = points * split
    if waves >= 2**31:
        raise LoweringError(f"loop nest: {waves} waves exceed the launch index range")

    # ---- host-side checks: every access in bounds, index arithmetic in 32 bits ---------------------------------
    def visit(bd, extents):
        for s in bd:
            if isinstance(s, L.Loop):
                visit(s.body, {**extents, s.axis: s.extent})
            elif isinstance(s, L.Load):
                if s.input in body.scalars:
                    continue
                if s.input not in operands:
                    raise LoweringError(f"loop nest: Load of {s.input!r}, which is not an operand of the kernel")
                _check_bounds(f"Load {s.name!r} of {s.input!r}", s.index, tuple(operands[s.input][1]), extents)
                for e in s.index:
                    if _max_intermediate(e, extents) >= 2**31:
                        raise LoweringError(f"loop nest: Load {s.name!r}: index arithmetic overflows 32 bits")
            elif isinstance(s, L.Write):
                if s.output != body.out_name:
                    raise LoweringError(f"loop nest: Write to {s.output!r}; the kernel's output is {body.out_name!r}")
                _check_bounds(f"Write to {s.output!r}", s.index, tuple(body.out_shape), extents)
                for e in s.index:
                    if _max_intermediate(e, extents) >= 2**31:
                        raise LoweringError("loop nest: Write: index arithmetic overflows 32 bits")
            elif isinstance(s, L.Select):
                for _, p in s.branches:
                    if _max_intermediate(p, extents) >= 2**31:
                        raise LoweringError(f"loop nest: Select {s.name!r}: predicate arithmetic overflows 32 bits")

    visit(stmts, {})

    # ---- rendering ------------------------------------------------------------------------------------------------
    o: list[str] = []
    a = o.append

    def flat(index: tuple, shape: tuple[int, ...]) -> str:
        expr = "(long)0"
        for e, dim in zip(index, shape):
            expr = f"({expr} * {dim} + (long)({_index_c(e)}))"
        return expr

    def render(bd, ind: str, dealt: bool, split_leaf: L.Loop | None) -> None:
        for s in bd:
            if isinstance(s, L.Load):
                if s.input in body.scalars:
                    a(f"{ind}const float {_v(s.name)} = {float_literal(body.scalars[s.input])};")
                else:
                    buf, shape, dt = operands[s.input]
                    a(f"{ind}const float {_v(s.name)} = {rt.convert(f'{param_of[buf]}[{flat(s.index, shape)}]', dt.name, 'f32')};")
            elif isinstance(s, L.Assign):
                args = [_v(x) for x in s.args]
                form = _UNARY_C[s.op] if s.op in _UNARY_C else _BINARY_C[s.op]
                a(f"{ind}const float {_v(s.name)} = {form.format(*args)};")
            elif isinstance(s, L.Select):
                expr = _v(s.branches[-1][0])  # the last branch is the catch-all
                for val, pred in reversed(s.branches[:-1]):
                    expr = f"(({_index_c(pred)}) ? {_v(val)} : {expr})"
                a(f"{ind}const float {_v(s.name)} = {expr};")
            elif isinstance(s, L.Accum):
                a(f"{ind}{_v(s.name)} = {_BINARY_C[s.op].format(_v(s.name), _v(s.value))};")
            elif isinstance(s, L.Write):
                store = f"out[{flat(s.index, tuple(body.out_shape))}] = {rt.convert(_v(s.value), 'f32', body.out_dtype.name)};"
                a(f"{ind}{store}" if dealt else f"{ind}if (lane == 0) {store}")
            elif isinstance(s, L.Loop):
                folds = _folds(s)
                for f in folds:
                    a(f"{ind}float {_v(f.name)} = {_IDENTITY_C[f.op]};")
                ax = _ax(s.axis)
                if _is_leaf(s) and not dealt:
                    if s is split_leaf and split > 1:
                        a(f"{ind}for (int {ax} = sp * 64 + lane; {ax} < {s.extent}; {ax} += {64 * split}) {{")
                    else:
                        a(f"{ind}for (int {ax} = lane; {ax} < {s.extent}; {ax} += 64) {{")
                    render(s.body, ind + "  ", True, None)
                    a(f"{ind}}}")
                    for f in folds:
                        a(f"{ind}{_v(f.name)} = emh_ln_{f.op}({_v(f.name)});")
                else:
                    a(f"{ind}for (int {ax} = 0; {ax} < {s.extent}; ++{ax}) {{")
                    render(s.body, ind + "  ", dealt, split_leaf)
                    a(f"{ind}}}")

    params = [f"const {rt.type_name(dtype_of[buf].name)}* __restrict__ {param_of[buf]}" for buf in order]
    params.append(f"{rt.type_name(body.out_dtype.name)}* __restrict__ out")
    a(f"// {name}: loop nest, one wave per point of {[(l_.axis, l_.extent) for l_ in chain]}" + (f", closing loop dealt over {split} waves" if split > 1 else ""))
    a(_HELPERS)
    a(f'extern "C" __global__ __launch_bounds__({_WAVES * 64}) void {name}({", ".join(params)}) {{')
    a("  const int lane = threadIdx.x % 64;")
    a(f"  long wv = (long)blockIdx.x * {_WAVES} + threadIdx.x / 64;")
    a("  wv = __builtin_amdgcn_readfirstlane((int)wv);  // uniform over the wave")
    a(f"  if (wv >= {waves}L) return;")
    if split > 1:
        a(f"  const int sp = (int)(wv % {split}); wv /= {split};")
    for loop in reversed(chain):
        a(f"  const int {_ax(loop.axis)} = (int)(wv % {loop.extent}); wv /= {loop.extent};")
    for level in pre:
        render(level, "  ", False, None)
    render(tail, "  ", False, last if split > 1 else None)
    a("}")
    grid = -(-waves // _WAVES)
    nbytes = int(math.prod(body.out_shape)) * body.out_dtype.nbytes + sum(int(math.prod(shape)) * dt.nbytes for _, shape, dt in {b: (b, s_, d) for b, s_, d in operands.values()}.values())
    return HipOp(
        kernel_source=prelude.header() + "\n".join(o) + "\n",
        kernel_name=name,
        arg_order=(*order, body.out),
        grid=((grid,), (1,), (1,)),
        block=((_WAVES * 64,), (1,), (1,)),
        lds_bytes=0,
        comment=f"loop nest points={points} split={split}",
        algo_bytes=nbytes,
        algo_flops=body.algo_flops(),
        knobs={"NEST": f"loops/w{points}" + (f"/s{split}" if split > 1 else "")},  # the route, then how it was dealt (informational)
    )
