"""Cross-workgroup split of a contraction's reduction axis: ``REDUCE=g<n>k`` / ``g<n>a``.

The reference realises a ``GRID`` reduce stage as a graph rewrite
(emmy/compiler/pipeline/passes/lowering/tile/030_split.py:135-334): a *partial* kernel
whose extra grid axis walks contiguous slices of the reduce axis and contributes its
carrier state, and either a sibling *finalize* kernel that folds a ``ws[cta, *free]``
workspace and projects the output (``"kernel"``, two nodes), or ``atomicAdd`` of the
additive state into a zero-initialised output (``"atomic"``).  Here:

* the partial kernel is the ordinary MFMA contraction over one slice of ``k``
  (``Contraction.k_split``): grid y = the split, bare fp32 accumulators out — plane
  ``blockIdx.y`` of an fp32 workspace (``"kernel"``), or ``global_atomic_add_f32`` into its
  single plane, which the runtime clears before the launch (``"atomic"``);
* the output type is 16-bit here, so the atomic arm cannot add into the output itself as the
  reference's fp32 kernels do: both arms end in the *combine* kernel below, which folds the
  planes in a fixed order, applies bias, epilogue and rounding exactly as the unsplit kernel's
  output stage does, and stores the result.  The workspace is a scratch tensor of the graph
  (planned into the program's slab like any intermediate).

It pays where the unsplit tiles do not cover the CUs (few rows, long reduction extent).
"""

from __future__ import annotations

from dataclasses import replace

from deplodock_amd.context import Context
from deplodock_amd.dtype import F32
from deplodock_amd.emit import prelude
from deplodock_amd.emit.errors import LoweringError
from deplodock_amd.ir import expr as E
from deplodock_amd.ir.hip import HipOp
from deplodock_amd.ir.schedule import ReducePlan
from deplodock_amd.ir.tile import Contraction
from deplodock_amd.render_target import rt

_T = 256


def split_planes(body: Contraction) -> int:
    """fp32 ``[m, n]`` planes the workspace of ``body``'s split holds."""
    return body.reduce.cta if body.reduce.finalize == "kernel" else 1


def partial_body(body: Contraction, ws: str) -> Contraction:
    """The contraction one slice of the split computes: same operands and tile, ``k`` = the slice,
    bare fp32 accumulators into the workspace."""
    n = body.reduce.cta
    if n < 2:
        raise LoweringError("contraction: not a cross-workgroup split")
    sym = getattr(body, "sym", None)
    if sym is not None and sym.fields:
        # ``sym`` is a plain attribute (``dataclasses.replace`` below would drop it) and the combine kernel bakes m in:
        # a split kernel pair serves the traced size only, so the caller must lower per size instead.
        raise LoweringError(f"contraction: a cross-workgroup split does not combine with a symbolic extent ({sorted(sym.fields)})")
    if body.gate_pair or body.a_prologue is not None or body.row_epilogue is not None:
        raise LoweringError("contraction: a cross-workgroup split takes a plain contraction (no gate/up pair, row prologue or row epilogue)")
    if body.k % n or (body.tile is not None and (body.k // n) % body.tile.bk_elems):
        raise LoweringError(f"contraction: K={body.k} does not split into {n} slices of whole slabs")
    return replace(
        body, k=body.k // n, lda=body.lda or body.k, ldb=body.ldb or body.k, out=ws, out_dtype=F32, ldo=body.n, out_offset=0,
        epilogue=None, post=None, epilogue_operands=(), operand_buffers={}, bias=None, bias_dtype=None,
        reduce=ReducePlan(), k_split=(n, body.reduce.finalize),
    )  # fmt: skip


def emit_splitk_combine(body: Contraction, ws: str, name: str, ctx: Context = Context()) -> HipOp:
    """``out[m, n] = post(round(epilogue(sum_s ws[s, m, n], bias)), operands)``: one thread per four
    consecutive columns, planes added in ascending order (bit-reproducible for the ``"kernel"`` arm)."""
    M, N = body.m, body.n
    planes = split_planes(body)
    if N % 4:
        raise LoweringError("contraction: N must be a multiple of 4 (8-byte output runs)")
    ldo = body.ldo or N
    epi = body.epilogue if body.epilogue is not None else E.Var("acc")
    post = body.post if body.post is not None else E.Var("y")
    epi_names = [n for n, _ in body.epilogue_operands]
    bad = (E.variables(epi) - ({"acc"} | ({"bias"} if body.bias is not None else set()))) | (E.variables(post) - ({"y"} | set(epi_names)))
    if bad:
        raise LoweringError(f"contraction: the split's combine uses unknown names {sorted(bad)}")
    out_t = rt.type_name(body.out_dtype.name)
    v4 = lambda dt: rt.vector_type(dt.name, 4)[0]  # noqa: E731
    params = ["const float* __restrict__ WS"]
    if body.bias is not None:
        params.append(f"const {rt.type_name(body.bias_dtype.name)}* __restrict__ BIAS")
    params += [f"const {rt.type_name(dt.name)}* __restrict__ e{i}" for i, (_, dt) in enumerate(body.epilogue_operands)]
    params.append(f"{out_t}* __restrict__ O")
    groups = M * (N // 4)
    o: list[str] = []
    a = o.append
    a(f"// {name}: combine of a {body.reduce.cta}-way split ({body.reduce.finalize}) M={M} N={N}: {planes} fp32 plane(s)")
    a(f'extern "C" __global__ __launch_bounds__({_T}) void {name}({", ".join(params)}) {{')
    a(f"  const long q = (long)blockIdx.x * {_T} + threadIdx.x;")
    a(f"  if (q >= {groups}L) return;")
    a(f"  const long m = q / {N // 4}, n = (q % {N // 4}) * 4;")
    a(f"  {v4(F32)} acc = *(const {v4(F32)}*)(WS + m * {N}L + n);")
    for s in range(1, planes):
        a(f"  {{ const {v4(F32)} t = *(const {v4(F32)}*)(WS + {s * M * N}L + m * {N}L + n); acc[0] += t[0]; acc[1] += t[1]; acc[2] += t[2]; acc[3] += t[3]; }}")
    if body.bias is not None:
        a(f"  const {v4(body.bias_dtype)} bv = *(const {v4(body.bias_dtype)}*)(BIAS + n);")
    for i, (_, dt) in enumerate(body.epilogue_operands):
        if dt.nbytes != body.out_dtype.nbytes:
            raise LoweringError("contraction: post-epilogue operands must have the output dtype")
        a(f"  const {v4(dt)} ev{i} = *(const {v4(dt)}*)(e{i} + m * {ldo}L + n);")
    a(f"  {v4(body.out_dtype)} yo;")
    for r in range(4):
        env = {"acc": f"acc[{r}]"}
        if body.bias is not None:
            env["bias"] = rt.convert(f"bv[{r}]", body.bias_dtype.name, "f32")
        val = E.render(epi, env)
        if body.post is not None:
            env2 = {"y": rt.convert(rt.convert(val, "f32", body.out_dtype.name), body.out_dtype.name, "f32")}
            for i, (n_, dt) in enumerate(body.epilogue_operands):
                env2[n_] = rt.convert(f"ev{i}[{r}]", dt.name, "f32")
            val = E.render(post, env2)
        a(f"  yo[{r}] = {rt.convert(val, 'f32', body.out_dtype.name)};")
    a(f"  *({v4(body.out_dtype)}*)(O + {body.out_offset}L + m * {ldo}L + n) = yo;")
    a("}")
    return HipOp(
        kernel_source=prelude.header() + "\n".join(o) + "\n",
        kernel_name=name,
        arg_order=(ws, *((body.bias,) if body.bias is not None else ()), *(body.operand_buffers.get(n, n) for n in epi_names), body.out),
        grid=((-(-groups // _T),), (1,), (1,)),
        block=((_T,), (1,), (1,)),
        comment=f"combine of a {body.reduce.cta}-way split ({body.reduce.finalize}) M={M} N={N}",
        algo_bytes=planes * M * N * 4 + M * N * body.out_dtype.nbytes * (1 + len(epi_names)),
        algo_flops=0,
        knobs={"REDUCE": body.reduce.spell()},
    )


__all__ = ["emit_splitk_combine", "partial_body", "split_planes"]
