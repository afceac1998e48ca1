"""Dense copy of a strided view, axes permuted, with zero padding: the layout change a contraction operand needs.

Two kernels, chosen by where the source's unit-stride axis lands in the result:

* it is the result's last axis too (or the source has none): every lane writes consecutive result elements and
  reads the source at whatever stride that implies — both sides coalesced when the last axis has stride 1;
* it lands elsewhere (a transposition, e.g. a ``[K, N]`` weight read as ``[N, K]`` rows): 64 x 64 tiles go through
  LDS, read with lanes along the source's unit-stride axis and written with lanes along the result's last axis, so
  both sides move whole 256-byte (128-byte for 16-bit types) runs.  Rows of the LDS tile are an odd number of
  words apart, which keeps the transposed read free of bank conflicts.

Index arithmetic is unsigned 32-bit; the host refuses what does not fit, and checks the largest source index
against the buffer before anything is launched.
"""

from __future__ import annotations

from dataclasses import dataclass

from deplodock_amd.context import Context
from deplodock_amd.emit import prelude
from deplodock_amd.emit.errors import LoweringError
from deplodock_amd.ir.hip import HipOp
from deplodock_amd.ir.sym import Affine, c_value, param_name
from deplodock_amd.ir.tile import IndexRows, StridedCopy
from deplodock_amd.render_target import rt

_TILE = 64
_PER_THREAD = 4  # result elements per lane in the row kernel


def emit_strided_copy(body: StridedCopy, name: str, ctx: Context = Context()) -> HipOp:
    axes = body.axes  # result order: (result extent, source extent, source stride)
    if not axes or any(se > de or se < 1 for de, se, _ in axes):
        raise LoweringError("copy: every axis needs 1 <= source extent <= result extent")
    total = 1
    for de, _, _ in axes:
        total *= de
    reach = body.src_offset + sum((se - 1) * st for _, se, st in axes)
    if body.src_offset < 0 or any(st < 0 for _, _, st in axes) or reach >= body.src_numel:
        raise LoweringError(f"copy: the view reaches element {reach} of a buffer of {body.src_numel}")
    if total >= 1 << 31 or reach >= 1 << 31:
        raise LoweringError("copy: index arithmetic is 32-bit; the tensor is too large")
    T = rt.type_name(body.dtype.name)
    zero = rt.literal("0.0f", body.dtype.name)
    dstrides = []
    acc = 1
    for de, _, _ in reversed(axes):
        dstrides.append(acc)
        acc *= de
    dstrides.reverse()
    last = len(axes) - 1
    unit = [i for i, (_, se, st) in enumerate(axes) if st == 1 and se > 1]
    s_ax = unit[-1] if unit else None
    o: list[str] = []
    a = o.append
    a(f'extern "C" __global__ __launch_bounds__(256) void {name}(const {T}* __restrict__ src, {T}* __restrict__ dst) {{')
    if s_ax is None or s_ax == last or axes[last][0] == 1:
        mode = "rows"
        per_block = 256 * _PER_THREAD
        a(f"  const unsigned lin0 = blockIdx.x * {per_block}u + threadIdx.x;")
        a("  #pragma unroll")
        a(f"  for (int u = 0; u < {_PER_THREAD}; ++u) {{")
        a("    const unsigned lin = lin0 + u * 256u;")
        a(f"    if (lin >= {total}u) break;")
        a(f"    unsigned rest = lin, at = {body.src_offset}u;")
        a("    bool inside = true;")
        for i in range(last, -1, -1):
            de, se, st = axes[i]
            if de == 1:
                continue
            a(f"    {{ const unsigned i{i} = rest % {de}u; rest /= {de}u; at += i{i} * {st}u;" + (f" inside = inside && i{i} < {se}u;" if se < de else "") + " }")
        a(f"    {T} v = {zero};")
        a("    if (inside) v = src[at];")
        a("    dst[lin] = v;")
        a("  }")
        grid = -(-total // per_block)
        lds = 0
    else:
        mode = "tile64"
        pad = 1 if body.dtype.nbytes == 4 else 2 if body.dtype.nbytes == 2 else None
        if pad is None:
            raise LoweringError(f"copy: no tile layout for {body.dtype.nbytes}-byte elements")
        (d_de, d_se, d_st), (s_de, s_se, _) = axes[last], axes[s_ax]
        td, ts = -(-d_de // _TILE), -(-s_de // _TILE)
        a(f"  __shared__ {T} tile[{_TILE}][{_TILE + pad}];")
        a("  const unsigned tx = threadIdx.x & 63u, ty = threadIdx.x >> 6;")
        a("  unsigned b = blockIdx.x;")
        a(f"  const unsigned td = b % {td}u; b /= {td}u;")
        a(f"  const unsigned ts = b % {ts}u; b /= {ts}u;")
        a(f"  unsigned at = {body.src_offset}u, to = 0u;")
        a("  bool inside = true;")
        outer = 1
        for i in range(last - 1, -1, -1):
            if i == s_ax:
                continue
            de, se, st = axes[i]
            outer *= de
            if de == 1:
                continue
            a(f"  {{ const unsigned i{i} = b % {de}u; b /= {de}u; at += i{i} * {st}u; to += i{i} * {dstrides[i]}u;" + (f" inside = inside && i{i} < {se}u;" if se < de else "") + " }")
        a("  #pragma unroll")
        a(f"  for (unsigned r = ty; r < {_TILE}u; r += 4u) {{")
        a(f"    const unsigned di = td * {_TILE}u + r, si = ts * {_TILE}u + tx;")
        a(f"    {T} v = {zero};")
        a(f"    if (inside && di < {d_se}u && si < {s_se}u) v = src[at + di * {d_st}u + si];")
        a("    tile[r][tx] = v;")
        a("  }")
        a("  __syncthreads();")
        a("  #pragma unroll")
        a(f"  for (unsigned r = ty; r < {_TILE}u; r += 4u) {{")
        a(f"    const unsigned si = ts * {_TILE}u + r, di = td * {_TILE}u + tx;")
        a(f"    if (si < {s_de}u && di < {d_de}u) dst[to + si * {dstrides[s_ax]}u + di] = tile[tx][r];")
        a("  }")
        grid = td * ts * outer
        lds = 0  # the tile is static LDS, declared in the source
    a("}")
    src_elems = 1
    for _, se, _ in axes:
        src_elems *= se
    return HipOp(
        kernel_source=prelude.header() + "\n".join(o) + "\n",
        kernel_name=name,
        arg_order=(body.src, body.out),
        grid=((grid,), (1,), (1,)),
        block=((256,), (1,), (1,)),
        lds_bytes=lds,
        comment=f"strided copy {mode}",
        algo_bytes=(src_elems + total) * body.dtype.nbytes,
        algo_flops=0,
        knobs={"COPY": mode},
    )


def emit_index_rows(body: IndexRows, name: str, ctx: Context = Context()) -> HipOp:
    """One lane per result element, consecutive along ``inner``: the row index is read once per element (it sits in
    cache for the whole row) and clamped into the table, so no value of ``idx`` can send a load outside ``src``.

    Symbolic form (``body.sym``): the number of looked-up rows ``count`` is an expression over the kernel's trailing
    ``int`` parameter (token ids ``[batch, seq_len]`` into an embedding table); the table itself never follows the
    axis.  The 32-bit index arithmetic then bounds the result at run time: a launch whose result would not fit is
    refused by the grid factor (``_IndexRowsGrid``) before anything runs."""
    total = body.outer * body.count * body.inner
    if min(body.outer, body.n, body.inner, body.count) < 1:
        raise LoweringError("index rows: empty operand")
    if total >= 1 << 31 or body.outer * body.n * body.inner >= 1 << 31:
        raise LoweringError("index rows: index arithmetic is 32-bit; the tensor is too large")
    if body.idx_dtype.name not in ("i32", "i64"):
        raise LoweringError(f"index rows: indices must be int32 or int64, got {body.idx_dtype}")
    sym = getattr(body, "sym", None)
    symf = sym.fields if sym is not None else {}
    if symf and set(symf) != {"count"}:
        raise LoweringError(f"index rows: {sorted(symf)} cannot follow a symbolic axis (only the number of looked-up rows can)")
    count_c = f"(unsigned){c_value(symf['count'])}" if symf else f"{body.count}u"
    T, IT = rt.type_name(body.dtype.name), rt.type_name(body.idx_dtype.name)
    o: list[str] = []
    a = o.append
    a(f'extern "C" __global__ __launch_bounds__(256) void {name}(const {T}* __restrict__ src, const {IT}* __restrict__ idx, {T}* __restrict__ dst{f", int {param_name(sym.name)}" if symf else ""}) {{')
    a("  const unsigned lin = blockIdx.x * 256u + threadIdx.x;")
    a(f"  const unsigned count = {count_c};")
    a(f"  if (lin >= {body.outer * body.inner}u * count) return;")
    a(f"  const unsigned i = lin % {body.inner}u, j = (lin / {body.inner}u) % count, o = lin / ({body.inner}u * count);")
    a("  long long r = (long long)idx[j];")
    a(f"  r = r < 0 ? 0 : (r >= {body.n} ? {body.n - 1} : r);")
    a(f"  dst[lin] = src[(o * {body.n}u + (unsigned)r) * {body.inner}u + i];")
    a("}")
    return HipOp(
        kernel_source=prelude.header() + "\n".join(o) + "\n",
        kernel_name=name,
        arg_order=(body.src, body.idx, body.out),
        grid=((_IndexRowsGrid(symf["count"], body.outer * body.inner) if symf else -(-total // 256),), (1,), (1,)),
        block=((256,), (1,), (1,)),
        lds_bytes=0,
        runtime_args=(sym.name,) if symf else (),
        comment="index rows",
        algo_bytes=body.algo_bytes(),
        algo_flops=0,
        knobs={"COPY": "index"},
    )


@dataclass(frozen=True)
class _IndexRowsGrid:
    """Launch-time grid of a symbolic lookup: one lane per result element, refused when the element count leaves the
    kernel's 32-bit index arithmetic."""

    count: Affine
    per_row: int

    def __call__(self, env: dict) -> int:
        total = self.count.at(env) * self.per_row
        if total >= 1 << 31:
            raise ValueError(f"index rows: {total} result elements at {env} do not fit the kernel's 32-bit index arithmetic")
        return -(-total // 256)


__all__ = ["emit_strided_copy", "emit_index_rows"]
