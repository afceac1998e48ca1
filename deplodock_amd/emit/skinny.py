"""Few-row contraction emitter: ``out[m, n] = epilogue(sum_k a[m, k] * b[n, k])`` for ``m <= 16``.

The decode-size case of the reference's output-tiled contraction
(``_contract_kloop``, emmy/compiler/pipeline/passes/lowering/kernel/_atom.py:446-468;
its cooperative-K option is ``ReducePlan`` on a Contraction, schedule.py:447).  With
at most 16 rows the problem is one pass over the weight matrix, and what it costs is
memory round trips, not arithmetic.  So there is no slab loop:

* a workgroup owns 16 output columns (one ``16x16x32`` MFMA tile holds all rows);
* its ``KW`` waves split the reduction axis, and every wave requests *all* of its
  weight fragments straight from global memory into registers before the first
  MFMA — the whole weight matrix is in flight at once, one round trip deep;
* with more than one row the activation rows are fetched once per workgroup as whole
  lines, ahead of the weights, and handed to the waves through LDS while the weights
  are on their way (as fragments from global memory a wave's load would touch
  16 rows x 64 bytes);
* the waves' partial tiles meet in LDS (``KW`` x 1 KiB), and the first wave applies
  the epilogue and stores four consecutive ``n`` per lane.

``STAGE=d<KW>/ks`` selects it (``ks``: k-split over the waves of a workgroup).
"""

from __future__ import annotations

from deplodock_amd.context import Context
from deplodock_amd.dtype import F32
from deplodock_amd.emit import prelude
from deplodock_amd.render_target import rt
from deplodock_amd.emit.errors import LoweringError
from deplodock_amd.ir import expr as E
from deplodock_amd.ir.hip import HipOp
from deplodock_amd.ir.tile import Contraction



def _frag_t(dtype_name: str) -> str:
    """The 16-byte MFMA operand fragment (eight 16-bit elements) of ``dtype_name``."""
    return rt.vector_type(dtype_name, 8)[0]


def _pack4_t(dtype_name: str) -> str:
    """Four consecutive output elements, the run an accumulator group converts to."""
    return rt.vector_type(dtype_name, 4)[0]
_BUILTIN = {"bf16": "__builtin_amdgcn_mfma_f32_16x16x32_bf16", "f16": "__builtin_amdgcn_mfma_f32_16x16x32_f16"}

#: MFMA steps whose fragments a wave requests in one go (2 x 4 registers each)
MAX_STEPS_IN_FLIGHT = 16


def skinny_waves(body: Contraction) -> int:
    """Waves that split the reduction axis (0: the shape does not take this form)."""
    if body.m > 16 or body.gate_pair or body.a_prologue is not None or body.row_epilogue is not None or body.reduce.cta != 1 or getattr(body, "batch", 1) > 1:
        return 0
    if getattr(body, "sym", None) is not None and "m" in body.sym.fields:
        return 0  # the few-row form holds every row in one MFMA tile: not with a row count known only at launch
    if body.in_dtype.name not in ("bf16", "f16") or body.k % 32 or body.n % 4:
        return 0
    for kw in (8, 4, 2, 1):
        if body.k % (32 * kw) == 0:
            return kw
    return 0


def emit_contraction_skinny(body: Contraction, name: str, ctx: Context = Context()) -> HipOp:
    stage = body.stage
    KW = stage.depth
    M, N, K = body.m, body.n, body.k
    if not skinny_waves(body) or KW not in (1, 2, 4, 8, 16) or K % (32 * KW):
        raise LoweringError(f"contraction: M={M} N={N} K={K} does not take the k-split few-row form with {KW} waves")
    lda, ldb, ldo = body.lda or K, body.ldb or K, body.ldo or N
    if lda % 8 or ldb % 8 or ldo % 4 or body.a_offset % 8 or body.b_offset % 8 or body.out_offset % 4:
        raise LoweringError("contraction: leading dimensions must keep 16-byte operand / 8-byte output alignment")
    steps = K // KW // 32
    chunk = steps
    while chunk > MAX_STEPS_IN_FLIGHT:
        chunk = next(c for c in range(chunk - 1, 0, -1) if steps % c == 0)
    frag_t = _frag_t(body.in_dtype.name)
    in_c, out_c = rt.type_name(body.in_dtype.name), rt.type_name(body.out_dtype.name)
    vt4 = _pack4_t(body.out_dtype.name)
    cast = "" if body.out_dtype is F32 else f"({out_c})"
    epi_names = [n for n, _ in body.epilogue_operands]
    epi = body.epilogue if body.epilogue is not None else E.Var("acc")
    unknown = E.variables(epi) - ({"acc"} | ({"bias"} if body.bias is not None else set()))
    if unknown:
        raise LoweringError(f"contraction epilogue uses unknown names {sorted(unknown)} (operands belong in `post`)")
    post = body.post if body.post is not None else E.Var("y")
    unknown = E.variables(post) - ({"y"} | set(epi_names))
    if unknown:
        raise LoweringError(f"contraction post-epilogue uses unknown names {sorted(unknown)}")
    for _, dt in body.epilogue_operands:
        if dt is not body.out_dtype:
            raise LoweringError("contraction: post-epilogue operands must have the output dtype")

    params = [f"const {in_c}* __restrict__ A", f"const {in_c}* __restrict__ B"]
    if body.bias is not None:
        params.append(f"const {rt.type_name(body.bias_dtype.name)}* __restrict__ BIAS")
    params += [f"const {rt.type_name(dt.name)}* __restrict__ e{i}" for i, (_, dt) in enumerate(body.epilogue_operands)]
    params.append(f"{out_c}* __restrict__ O")
    T = 64 * KW
    o: list[str] = []
    a = o.append
    a(f"// {name}: M={M} N={N} K={K} few rows, k split over {KW} waves, {steps} MFMA steps per wave ({chunk} in flight)")
    a(f'extern "C" __global__ __launch_bounds__({T}) void {name}({", ".join(params)}) {{')
    # More than one row: the activation rows go through LDS.  Read as fragments from global memory, a
    # wave's load touches 16 rows x 64 bytes; staged, the workgroup fetches whole lines once, and the
    # requests go out ahead of the weight loads, so the staging runs under the weights' round trip.
    pitch = K * 2 + 16  # rows 16 bytes apart modulo the bank width: conflict-free 16-byte fragment reads
    x_lds = M > 1 and KW * 1024 + M * pitch <= min(ctx.lds_bytes_per_cu, 128 * 1024)
    x_chunks = M * K // 8
    x_per_t = -(-x_chunks // T)
    lds_bytes = KW * 1024 + (M * pitch if x_lds else 0)
    a("  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];")
    a("  f32x4* part = (f32x4*)lds;")
    a("  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;")
    a("  const int lr = lane % 16, lk = lane / 16;")
    a("  const int n0 = blockIdx.x * 16;")
    a(f"  const int nrow = n0 + lr < {N} ? n0 + lr : {N - 1};  // a ragged last tile re-reads the last row; its columns are not stored")
    a(f"  const int mrow = lr < {M} ? lr : {M - 1};")
    a(f"  const {in_c}* bp = B + {body.b_offset}L + (long)nrow * {ldb} + wave * {K // KW} + lk * 8;")
    if x_lds:
        a(f"  unsigned char* xs = lds + {KW * 1024};")
        a(f"  const unsigned char* xp = xs + mrow * {pitch} + (wave * {K // KW} + lk * 8) * 2;")
        a(f"  u32x4 xr[{x_per_t}];")
        a("  #pragma unroll")
        a(f"  for (int i = 0; i < {x_per_t}; ++i) {{")
        a(f"    const int q = tid + i * {T};")
        a(f"    if ({'true' if x_chunks % T == 0 else f'q < {x_chunks}'}) xr[i] = *(const u32x4*)(A + {body.a_offset}L + (long)(q / {K // 8}) * {lda} + (q % {K // 8}) * 8);")
        a("  }")
    else:
        a(f"  const {in_c}* ap = A + {body.a_offset}L + (long)mrow * {lda} + wave * {K // KW} + lk * 8;")

    def publish_x() -> None:
        a("  #pragma unroll")
        a(f"  for (int i = 0; i < {x_per_t}; ++i) {{")
        a(f"    const int q = tid + i * {T};")
        a(f"    if ({'true' if x_chunks % T == 0 else f'q < {x_chunks}'}) *(u32x4*)(xs + (q / {K // 8}) * {pitch} + (q % {K // 8}) * 16) = xr[i];")
        a("  }")
        a("  __syncthreads();")

    a("  // Operand roles: the weights take the A port, so accumulator register r of a lane is")
    a("  // out[m = lane % 16][n = n0 + 4 * (lane / 16) + r] - four consecutive n of one row.")
    a("  f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};")
    looped = chunk < steps
    if looped:
        if x_lds:
            publish_x()
        a("  #pragma unroll 1")
        a(f"  for (int s0 = 0; s0 < {steps}; s0 += {chunk}) {{")
        base = "(s0 + s) * 32"
    else:
        a("  {")
        base = "s * 32"
    a(f"    {frag_t} wf[{chunk}], xf[{chunk}];")
    a("    #pragma unroll")
    a(f"    for (int s = 0; s < {chunk}; ++s) wf[s] = *(const {frag_t}*)(bp + {base});")
    if x_lds and not looped:
        publish_x()
    a("    #pragma unroll")
    if x_lds:
        a(f"    for (int s = 0; s < {chunk}; ++s) xf[s] = *(const {frag_t}*)(xp + ({base}) * 2);")
    else:
        a(f"    for (int s = 0; s < {chunk}; ++s) xf[s] = *(const {frag_t}*)(ap + {base});")
    a("    #pragma unroll")
    a(f"    for (int s = 0; s < {chunk}; ++s) acc = {_BUILTIN[body.in_dtype.name]}(wf[s], xf[s], acc, 0, 0, 0);")
    a("  }")
    if KW > 1:
        a("  part[wave * 64 + lane] = acc;")
        a("  __syncthreads();")
        a("  if (wave != 0) return;")
        a("  #pragma unroll")
        a(f"  for (int w = 1; w < {KW}; ++w) acc += part[w * 64 + lane];")
    a("  const int m = lr, n = n0 + lk * 4;")
    a(f"  if (m >= {M} || n >= {N}) return;  // N is a multiple of 4: a run of four is all in or all out")
    for i, (_, dt) in enumerate(body.epilogue_operands):
        vt = _pack4_t(dt.name)
        a(f"  const {vt} ev{i} = *(const {vt}*)(e{i} + (long)m * {ldo} + n);")
    if body.bias is not None:
        bt4 = _pack4_t(body.bias_dtype.name)
        a(f"  const {bt4} bv = *(const {bt4}*)(BIAS + n);")
    a(f"  {vt4} yo;")
    for r in range(4):
        env = {"acc": f"acc[{r}]"}
        if body.bias is not None:
            env["bias"] = f"(float)bv[{r}]"
        pre = E.render(epi, env)
        if body.post is not None:
            env2 = {"y": f"(float){cast}({pre})"}
            for i, n_ in enumerate(epi_names):
                env2[n_] = f"(float)ev{i}[{r}]"
            pre = E.render(post, env2)
        a(f"  yo[{r}] = {cast}({pre});")
    a(f"  *({vt4}*)(O + {body.out_offset}L + (long)m * {ldo} + n) = yo;")
    a("}")
    return HipOp(
        kernel_source=prelude.header() + "\n".join(o) + "\n",
        kernel_name=name,
        arg_order=(body.a, body.b, *((body.bias,) if body.bias is not None else ()), *(body.operand_buffers.get(n, n) for n in epi_names), body.out),
        grid=((-(-N // 16),), (1,), (1,)),
        block=((T,), (1,), (1,)),
        lds_bytes=lds_bytes,
        comment=f"contraction M={M} N={N} K={K} few rows, k split over {KW} waves",
        algo_bytes=body.algo_bytes(),
        algo_flops=body.algo_flops(),
        knobs={"TILE": body.tile.spell() if body.tile is not None else "", "STAGE": stage.spell()},
    )


__all__ = ["emit_contraction_skinny", "skinny_waves"]
