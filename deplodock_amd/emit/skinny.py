"""Few-row contraction emitter: ``out[m, n] = epilogue(sum_k a[m, k] * b[n, k])`` for ``m <= 64``.

The decode-size case of the reference's output-tiled contraction
(``_contract_kloop``, emmy/compiler/pipeline/passes/lowering/kernel/_atom.py:446-468;
its cooperative-K option is ``ReducePlan`` on a Contraction, schedule.py:447).  With
a few rows the problem is one pass over the weight matrix, and what it costs is
memory round trips, not arithmetic.  So there is no slab loop:

* a workgroup owns ``C`` output columns (4, 8, 12 or 16: one ``16x16x32`` MFMA tile per
  16 rows holds them; with fewer than 16 the spare weight rows of the tile repeat the
  first ones and are not stored).  ``C`` is chosen so that the workgroups cover the CUs:
  what a CU moves is the activation rows once plus its share of the weights;
* its ``KW`` waves split the reduction axis, and every wave requests *all* of its
  weight fragments straight from global memory into registers before the first
  MFMA — the whole weight matrix is in flight at once, one round trip deep;
* with more than one row the activation rows are fetched once per workgroup as whole
  lines, ahead of the weights, and handed to the waves through LDS while the weights
  are on their way (as fragments from global memory a wave's load would touch
  16 rows x 64 bytes); rows that do not fit the LDS are read as fragments;
* more than 16 rows are further row tiles against the same weight fragments;
* a gate / up pair (``gate_pair``) is two weight fragment sets and two accumulators per
  row tile, met in the epilogue;
* a deferred row normalisation (``RowPrologue.scale``: the column weight is already
  folded into ``b``) accumulates its statistic from the fragments each lane holds: the
  lanes of a row meet through a butterfly, the waves through LDS beside the partial
  tiles, and the accumulators are scaled before the epilogue;
* the waves' partial tiles meet in LDS, and wave ``t`` finishes row tile ``t``: epilogue,
  then four consecutive ``n`` per lane stored.

``STAGE=d<KW>/ks[/c<C>]`` selects it (``ks``: k-split over the waves of a workgroup).
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

#: MFMA steps whose fragments a wave requests in one go (4 registers each; a gate / up pair holds two sets)
MAX_STEPS_IN_FLIGHT = 16
#: rows the form takes: up to four 16-row MFMA tiles against one set of weight fragments
MAX_ROWS = 64


def skinny_waves(body: Contraction) -> int:
    """Waves that split the reduction axis (0: the shape does not take this form)."""
    if body.m > MAX_ROWS or body.row_epilogue is not None or body.reduce.cta != 1 or getattr(body, "batch", 1) > 1 or body.k_split is not None:
        return 0
    pro = body.a_prologue
    if pro is not None and (pro.scale is None or pro.weight is not None or E.variables(pro.scale) - {"ss"} or E.variables(pro.stat_pre) - {"x"}):
        return 0  # only the deferred normalisation: a per-row factor on the accumulators
    if getattr(body, "sym", None) is not None and "m" in body.sym.fields:
        return 0  # the few-row form holds every row in a fixed number of MFMA tiles: not with a row count known only at launch
    if body.in_dtype.name not in ("bf16", "f16") or body.k % 32 or body.n % 4:
        return 0
    # at least 256 values of the reduction axis a wave (eight MFMA steps): in the decoder block at 1-32 rows, K = 1024
    # takes 2.74-2.96 us on two or four waves against 2.89-3.12 on eight; K = 3072 is 3.72 on eight, 4.39 on four
    for kw in (8, 4, 2, 1):
        if body.k % (32 * kw) == 0 and (body.k // kw >= 256 or kw == 1):
            return kw
    return 0


def skinny_cols(body: Contraction, ctx: Context = Context()) -> int:
    """Output columns per workgroup: what a CU moves is the activation rows (once per workgroup) plus ``C`` weight rows
    (two sets for a gate / up pair), times the workgroups it is dealt; the ``C`` with the least of that wins."""
    nb = 2 if body.gate_pair else 1
    x_bytes = body.m * body.k * body.in_dtype.nbytes

    def per_cu(c: int) -> int:
        rounds = -(-(-(-body.n // c)) // ctx.compute_units)
        return rounds * (x_bytes + c * body.k * body.in_dtype.nbytes * nb)

    if -(-body.n // 16) >= 0.75 * ctx.compute_units:
        # whole 16-wide MFMA tiles already cover the machine: fewer, fuller workgroups ask the L2s for the rows less often
        # (gate / up pair, N = 3072, 8-32 rows: 3.93 / 3.98 / 4.65 us on 192 workgroups of 16 against 4.21 / 4.24 / 5.13 on 256 of 12)
        return 16
    return min((c for c in (16, 12, 8, 4) if body.n % c == 0 or c == 16), key=lambda c: (per_cu(c), -c))


def emit_contraction_skinny(body: Contraction, name: str, ctx: Context = Context()) -> HipOp:
    stage = body.stage
    KW = stage.depth
    M, N, K = body.m, body.n, body.k
    if not skinny_waves(body) or KW not in (1, 2, 4, 8, 16) or K % (32 * KW):
        raise LoweringError(f"contraction: M={M} N={N} K={K} does not take the k-split few-row form with {KW} waves")
    C = getattr(stage, "cols", 0) or 16
    if C not in (4, 8, 12, 16) or (C != 16 and N % C):
        raise LoweringError(f"contraction: {C} columns per workgroup do not tile N={N} (4, 8, 12 or 16, dividing N)")
    lda, ldb, ldo = body.lda or K, body.ldb or K, body.ldo or N
    if lda % 8 or ldb % 8 or ldo % 4 or body.a_offset % 8 or body.b_offset % 8 or body.out_offset % 4:
        raise LoweringError("contraction: leading dimensions must keep 16-byte operand / 8-byte output alignment")
    gate = bool(body.gate_pair)
    NB = 2 if gate else 1
    MT = -(-M // 16)  # row tiles
    pro = body.a_prologue
    deferred = pro is not None
    steps = K // KW // 32
    chunk = steps
    in_flight = MAX_STEPS_IN_FLIGHT // NB
    while chunk > in_flight:
        chunk = next(c for c in range(chunk - 1, 0, -1) if steps % c == 0)
    frag_t = _frag_t(body.in_dtype.name)
    in_c, out_c = rt.type_name(body.in_dtype.name), rt.type_name(body.out_dtype.name)
    vt4 = _pack4_t(body.out_dtype.name)
    cast = "" if body.out_dtype is F32 else f"({out_c})"
    epi_names = [n for n, _ in body.epilogue_operands]
    epi = body.epilogue if body.epilogue is not None else E.Var("acc")
    unknown = E.variables(epi) - ({"acc"} | ({"acc2"} if gate else set()) | ({"bias"} if body.bias is not None else set()))
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
    a(f"// {name}: M={M} N={N} K={K} few rows ({MT} row tile(s), {C} columns a workgroup{', gate / up pair' if gate else ''}), k split over {KW} waves, {steps} MFMA steps per wave ({chunk} in flight)")
    a(f'extern "C" __global__ __launch_bounds__({T}) void {name}({", ".join(params)}) {{')
    # LDS: the partial tiles [wave][row tile][gate | up] of 1 KiB, the waves' row statistics, then the activation rows.
    # More than one row: the activation rows go through LDS.  Read as fragments from global memory, a
    # wave's load touches 16 rows x 64 bytes; staged, the workgroup fetches whole lines once, and the
    # requests go out ahead of the weight loads, so the staging runs under the weights' round trip.
    part_bytes = KW * MT * NB * 1024 if KW > 1 else 0
    ss_off = part_bytes
    ss_bytes = KW * MT * 16 * 4 if deferred and KW > 1 else 0
    x_off = -(-(ss_off + ss_bytes) // 16) * 16
    pitch = K * 2 + 16  # rows 16 bytes apart modulo the bank width: conflict-free 16-byte fragment reads
    x_lds = M > 1 and x_off + M * pitch <= min(ctx.lds_bytes_per_cu, 128 * 1024)
    x_chunks = M * K // 8
    x_per_t = -(-x_chunks // T)
    if x_lds and x_per_t > 24:
        x_lds = False  # the staged rows pass through registers: too many of them would crowd out the weight fragments
    lds_bytes = max(x_off + (M * pitch if x_lds else 0), 16)
    a("  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];")
    a("  f32x4* part = (f32x4*)lds;")
    a("  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;")
    a("  const int lr = lane % 16, lk = lane / 16;")
    a(f"  const int n0 = blockIdx.x * {C};")
    a(f"  const int nrow = n0 + lr < {N} ? n0 + lr : {N - 1};  // a ragged last tile re-reads the last row; its columns are not stored")
    a(f"  const {in_c}* bp = B + {body.b_offset}L + (long)nrow * {ldb} + wave * {K // KW} + lk * 8;")
    if gate:
        a(f"  const {in_c}* bp2 = bp + {N}L * {ldb};  // the up projection's rows follow the gate's")
    if x_lds:
        a(f"  unsigned char* xs = lds + {x_off};")
        a(f"  u32x4 xr[{x_per_t}];")
        a("  #pragma unroll")
        a(f"  for (int i = 0; i < {x_per_t}; ++i) {{")
        a(f"    const int q = tid + i * {T};")
        a(f"    if ({'true' if x_chunks % T == 0 else f'q < {x_chunks}'}) xr[i] = *(const u32x4*)(A + {body.a_offset}L + (long)(q / {K // 8}) * {lda} + (q % {K // 8}) * 8);")
        a("  }")

    def publish_x() -> None:
        a("  #pragma unroll")
        a(f"  for (int i = 0; i < {x_per_t}; ++i) {{")
        a(f"    const int q = tid + i * {T};")
        a(f"    if ({'true' if x_chunks % T == 0 else f'q < {x_chunks}'}) *(u32x4*)(xs + (q / {K // 8}) * {pitch} + (q % {K // 8}) * 16) = xr[i];")
        a("  }")
        a("  __syncthreads();")

    a("  // Operand roles: the weights take the A port, so accumulator register r of a lane is")
    a("  // out[m = 16 * tile + lane % 16][n = n0 + 4 * (lane / 16) + r] - four consecutive n of one row.")
    a(f"  f32x4 acc[{MT}][{NB}];")
    a("  #pragma unroll")
    a(f"  for (int t = 0; t < {MT}; ++t)")
    a("  #pragma unroll")
    a(f"  for (int b = 0; b < {NB}; ++b) acc[t][b] = (f32x4){{0.0f, 0.0f, 0.0f, 0.0f}};")
    if deferred:
        a(f"  float ss[{MT}];")
        a("  #pragma unroll")
        a(f"  for (int t = 0; t < {MT}; ++t) ss[t] = 0.0f;")
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
    a(f"    {frag_t} wf[{NB}][{chunk}];")
    if C < 16:
        # the tile's spare weight rows request nothing (a repeated address would still be a request) and count as zeros
        a("    #pragma unroll")
        a(f"    for (int b = 0; b < {NB}; ++b)")
        a("    #pragma unroll")
        a(f"    for (int s = 0; s < {chunk}; ++s)")
        a("    #pragma unroll")
        a(f"    for (int e = 0; e < 8; ++e) wf[b][s][e] = ({in_c})0.0f;")
        a(f"    if (lr < {C}) {{")
    a("    #pragma unroll")
    a(f"    for (int s = 0; s < {chunk}; ++s) wf[0][s] = *(const {frag_t}*)(bp + {base});")
    if gate:
        a("    #pragma unroll")
        a(f"    for (int s = 0; s < {chunk}; ++s) wf[1][s] = *(const {frag_t}*)(bp2 + {base});")
    if C < 16:
        a("    }")
    if x_lds and not looped:
        publish_x()
    a("    #pragma unroll")
    a(f"    for (int t = 0; t < {MT}; ++t) {{")
    a(f"      const int mrow = 16 * t + lr < {M} ? 16 * t + lr : {M - 1};")
    a(f"      {frag_t} xf[{chunk}];")
    a("      #pragma unroll")
    if x_lds:
        a(f"      for (int s = 0; s < {chunk}; ++s) xf[s] = *(const {frag_t}*)(xs + mrow * {pitch} + (wave * {K // KW} + lk * 8 + {base}) * 2);")
    else:
        a(f"      for (int s = 0; s < {chunk}; ++s) xf[s] = *(const {frag_t}*)(A + {body.a_offset}L + (long)mrow * {lda} + wave * {K // KW} + lk * 8 + {base});")
    if deferred:
        a("      #pragma unroll")
        a(f"      for (int s = 0; s < {chunk}; ++s)")
        a("      #pragma unroll")
        a("      for (int e = 0; e < 8; ++e) { const float x_ = (float)xf[s][e]; ss[t] += " + E.render(pro.stat_pre, {"x": "x_"}) + "; }")
    a("      #pragma unroll")
    a(f"      for (int s = 0; s < {chunk}; ++s) {{")
    a(f"        acc[t][0] = {_BUILTIN[body.in_dtype.name]}(wf[0][s], xf[s], acc[t][0], 0, 0, 0);")
    if gate:
        a(f"        acc[t][1] = {_BUILTIN[body.in_dtype.name]}(wf[1][s], xf[s], acc[t][1], 0, 0, 0);")
    a("      }")
    a("    }")
    a("  }")
    if deferred:
        # a row's statistic: its four lane groups (k chunks of a step) meet through a butterfly, the waves through LDS
        a("  #pragma unroll")
        a(f"  for (int t = 0; t < {MT}; ++t) {{ ss[t] += emh_xor16(ss[t]); ss[t] += __shfl_xor(ss[t], 32); }}")
    if KW > 1:
        a("  #pragma unroll")
        a(f"  for (int t = 0; t < {MT}; ++t)")
        a("  #pragma unroll")
        a(f"  for (int b = 0; b < {NB}; ++b) part[((wave * {MT} + t) * {NB} + b) * 64 + lane] = acc[t][b];")
        if deferred:
            a(f"  float* ssp = (float*)(lds + {ss_off});")
            a("  if (lk == 0) {")
            a("    #pragma unroll")
            a(f"    for (int t = 0; t < {MT}; ++t) ssp[(wave * {MT} + t) * 16 + lr] = ss[t];")
            a("  }")
        a("  __syncthreads();")
        a(f"  if (wave >= {min(MT, KW)}) return;")
        tiles = f"for (int t = wave; t < {MT}; t += {KW})" if MT > KW else "{ const int t = wave;"
    else:
        tiles = f"for (int t = 0; t < {MT}; ++t)"
    if tiles.startswith("for"):
        a("  #pragma unroll")
        a(f"  {tiles} {{")
    else:
        a(f"  {tiles}")
    a(f"    f32x4 y[{NB}];")
    if KW > 1:
        a("    #pragma unroll")
        a(f"    for (int b = 0; b < {NB}; ++b) {{")
        a(f"      y[b] = part[(t * {NB} + b) * 64 + lane];")
        a("      #pragma unroll")
        a(f"      for (int w = 1; w < {KW}; ++w) y[b] += part[((w * {MT} + t) * {NB} + b) * 64 + lane];")
        a("    }")
        if deferred:
            a("    float st = 0.0f;")
            a("    #pragma unroll")
            a(f"    for (int w = 0; w < {KW}; ++w) st += ssp[(w * {MT} + t) * 16 + lr];")
    else:
        a("    #pragma unroll")
        a(f"    for (int b = 0; b < {NB}; ++b) y[b] = acc[t][b];")
        if deferred:
            a("    const float st = ss[t];")
    if deferred:
        a(f"    const float rs_ = {E.render(pro.scale, {'ss': 'st'})};")
    a("    const int m = 16 * t + lr, n = n0 + lk * 4;")
    a(f"    if (m < {M} && n < {N} && lk * 4 < {C}) {{  // N is a multiple of 4: a run of four is all in or all out")
    for i, (_, dt) in enumerate(body.epilogue_operands):
        vt = _pack4_t(dt.name)
        a(f"      const {vt} ev{i} = *(const {vt}*)(e{i} + (long)m * {ldo} + n);")
    if body.bias is not None:
        bt4 = _pack4_t(body.bias_dtype.name)
        a(f"      const {bt4} bv = *(const {bt4}*)(BIAS + n);")
    a(f"      {vt4} yo;")
    sc = " * rs_" if deferred else ""
    for r in range(4):
        env = {"acc": f"(y[0][{r}]{sc})"}
        if gate:
            env["acc2"] = f"(y[1][{r}]{sc})"
        if body.bias is not None:
            env["bias"] = f"(float)bv[{r}]"
        pre = E.render(epi, env)
        if body.post is not None:
            env2 = {"y": f"(float){cast}({pre})"}
            for i, n_ in enumerate(epi_names):
                env2[n_] = f"(float)ev{i}[{r}]"
            pre = E.render(post, env2)
        a(f"      yo[{r}] = {cast}({pre});")
    a(f"      *({vt4}*)(O + {body.out_offset}L + (long)m * {ldo} + n) = yo;")
    a("    }")
    a("  }")
    a("}")
    hip = HipOp(
        kernel_source=prelude.header(prelude.WAVE_REDUCE) + "\n".join(o) + "\n",
        kernel_name=name,
        arg_order=(body.a, body.b, *((body.bias,) if body.bias is not None else ()), *(body.operand_buffers.get(n, n) for n in epi_names), body.out),
        grid=((-(-N // C),), (1,), (1,)),
        block=((T,), (1,), (1,)),
        lds_bytes=lds_bytes,
        comment=f"contraction M={M} N={N} K={K} few rows, k split over {KW} waves, {C} columns a workgroup",
        algo_bytes=body.algo_bytes(),
        algo_flops=body.algo_flops(),
        knobs={"TILE": body.tile.spell() if body.tile is not None else "", "STAGE": stage.spell()},
    )
    if body.b_offset == 0 and N % C == 0:
        # workgroup j streams rows [C j, C j + C) of the weight (a gate / up pair: and the same rows of the second matrix,
        # N rows further on): what a kernel launched before this one needs to know to put them into the right XCD's L2
        hip.weight_slices = (body.b, C * ldb * body.in_dtype.nbytes, NB * N // C)
    return hip


__all__ = ["emit_contraction_skinny", "skinny_waves", "skinny_cols", "MAX_ROWS"]
