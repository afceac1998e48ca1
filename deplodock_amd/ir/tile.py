"""Tile IR — one scheduled kernel per ``TileOp``.

The input contract of the gfx950 lowering, playing the role of the
reference's ``TileOp`` (emmy/compiler/ir/tile/ir.py:424-459) whose body is a
``Map`` (:392), ``Reduction`` (:89) or ``Contraction`` (:196) with the schedule
plans stamped on it (``ReducePlan`` / ``TilePlan`` / ``Stage``).  The emitters
apply a stamped plan verbatim and decide nothing.

Buffers are named by graph node id.  Element-wise pieces (statistic
pre-maps, projections, epilogues) are ``ir.expr`` trees over named scalars.
"""

from __future__ import annotations

from dataclasses import dataclass, field

from deplodock_amd.dtype import DType
from deplodock_amd.ir.base import Op
from deplodock_amd.ir.expr import Expr
from deplodock_amd.ir.schedule import ReducePlan, Stage, TilePlan


@dataclass(frozen=True)
class Stat:
    """One row statistic: ``name = monoid over columns of pre(x, earlier stats)``."""

    name: str
    monoid: str  # "sum" | "max" | "min"
    pre: Expr  # over Var("x") and earlier stat names
    keep: bool = False  # the pre-mapped value replaces the resident element ``x``


@dataclass(frozen=True)
class RowAddr:
    """Element offset of row ``r``: ``offset + (r // div) * stride_hi + (r % div) * stride_lo``.
    ``div == 1`` is the plain ``offset + r * stride_hi``; the two-level form walks
    e.g. the heads of a ``[tokens, heads * head_dim]`` buffer as rows."""

    offset: int = 0
    div: int = 1
    stride_hi: int = 0
    stride_lo: int = 0

    @classmethod
    def uniform(cls, stride: int, offset: int = 0) -> RowAddr:
        return cls(offset=offset, div=1, stride_hi=stride, stride_lo=0)

    def max_vec(self, v: int) -> int:
        """Largest power-of-two vector width <= ``v`` every row start is aligned to."""
        while v > 1 and (self.offset % v or self.stride_hi % v or (self.div > 1 and self.stride_lo % v)):
            v //= 2
        return v


@dataclass(frozen=True)
class RowOperand:
    """A per-(row-group, column) table such as RoPE ``cos`` / ``sin`` ``[positions, cols]``:
    row ``r`` reads table row ``(r // div) % mod``."""

    name: str
    dtype: DType
    div: int = 1
    mod: int = 1
    offset: int = 0


@dataclass(frozen=True)
class RotateHalf:
    """Second projection phase for rotary embeddings.  With ``y`` the projected
    row and ``yr`` its signed half-rotation (``-y[c + cols/2]`` for the first
    half, ``y[c - cols/2]`` for the second; the reference traces it as
    ``cat(neg(slice_hi), slice_lo)``), the output is ``expr(y, yr, row operands)``."""

    expr: Expr


@dataclass
class RowReduce:
    """``Map(source=Reduction)``: per-row statistics followed by a projection.

    ``x`` is ``[rows, cols]`` with the reduce axis innermost and contiguous;
    ``x_addr`` / ``out_addr`` place the rows.  ``project`` is evaluated per
    element over ``x``, the statistics, and the per-column operands
    (``col_operands``: vectors of length ``cols`` such as a norm weight).
    RMSNorm is ``stats=(ss = sum x*x)``, ``project = x * rsqrt(ss/cols + eps) * w``
    (emmy/compiler/ir/frontend/ir.py:309-312); softmax is ``m = max x``,
    ``d = sum exp(x - m)``, ``project = exp(x - m) / d`` (:354-358).  ``stats``
    may be empty (a pure row-wise map).  With ``scalar_out`` the kernel is a plain
    row reduction (``sum`` / ``mean`` over the last axis): one value per row."""

    rows: int
    cols: int
    x: str
    x_dtype: DType
    out: str
    out_dtype: DType
    stats: tuple[Stat, ...]
    project: Expr
    col_operands: tuple[tuple[str, DType], ...] = ()
    row_operands: tuple[RowOperand, ...] = ()
    rotate: RotateHalf | None = None
    x_addr: RowAddr | None = None
    out_addr: RowAddr | None = None
    reduce: ReducePlan = field(default_factory=ReducePlan)
    rows_per_block: int | None = None  # derived from the plan when None
    nontemporal: bool = False
    stream: bool = False  # walk the row once per statistic level instead of keeping it in registers
    scalar_out: bool = False  # the output is one value per row: ``project`` over the statistics only
    # expression name -> buffer (graph node id) for col/row operands; identity when absent
    operand_buffers: dict = field(default_factory=dict)

    def algo_bytes(self) -> int:
        b = self.rows * self.cols * self.x_dtype.nbytes + self.rows * (1 if self.scalar_out else self.cols) * self.out_dtype.nbytes
        for _, dt in self.col_operands:
            b += self.cols * dt.nbytes
        for ro in self.row_operands:
            b += ro.mod * self.cols * ro.dtype.nbytes
        return b


@dataclass(frozen=True)
class RowPrologue:
    """A row-wise normalisation applied to the ``a`` operand on its way into the
    contraction, so ``norm -> linear`` is one launch: every workgroup first
    folds ``stat_pre(x)`` over the full ``k`` extent of its rows (name ``ss``),
    then maps each element with ``project`` (names ``x``, ``ss`` and, when
    ``weight`` is set, ``w`` — a length-``k`` vector) while staging the slab.
    ``project`` carries the producer's own rounding points, so the operand the
    MFMAs see is bit-for-bit what the separate kernel would have written.

    With ``scale`` set the normalisation is *deferred*: when the projection is
    ``x * f(ss) * w`` — a per-row factor and a per-column weight, as in RMSNorm —
    then ``(x f(ss) w) @ W^T = f(ss) (x @ (W w)^T)``: the column weight is folded
    into the constant ``b`` operand once, at bind time, the ``a`` operand is staged
    untouched while its statistic is accumulated slab by slab, and the accumulators
    are multiplied by ``scale`` (an expression over ``ss``) before the epilogue.
    That drops the statistic pre-pass over the rows and the per-element transform
    every workgroup of a row block would repeat; the normalised operand is then
    never rounded to 16 bits, so the result is as close to the exact one as the
    eager module's, not bit-equal to it."""

    stat_pre: Expr
    project: Expr
    weight: str | None = None
    weight_dtype: DType | None = None
    scale: Expr | None = None


@dataclass
class RowEpilogue:
    """A row kernel folded into the contraction's output stage.  Columns
    ``[0, col_end)`` of the result are ``col_end / cols`` groups of ``cols``
    columns (the heads of a merged q/k projection); on every (output row, group)
    the statistics, projection and optional half-rotation of a ``RowReduce`` are
    applied to the rounded contraction result while the output tile sits in LDS,
    so ``linear -> head norm -> rotary embedding`` is one launch.  ``row_operands``
    index their tables with the row number ``m * (col_end / cols) + group``, as the
    separate kernel would; columns from ``col_end`` on are stored untouched."""

    cols: int
    col_end: int
    stats: tuple[Stat, ...]
    project: Expr
    rotate: RotateHalf | None = None
    row_operands: tuple[RowOperand, ...] = ()
    operand_buffers: dict = field(default_factory=dict)  # row operand name -> buffer id


@dataclass
class Contraction:
    """``out[m, n] = epilogue(sum_k a[m, k] * b[n, k])`` — both operands
    K-contiguous (the reference's ``b_trans`` layout for ``nn.Linear`` weights,
    emmy/compiler/ir/tile/ir.py:325).  ``epilogue`` is an expression over
    ``acc`` and the names in ``epilogue_operands`` (``[m, n]`` tensors such as a
    residual).  With ``gate_pair`` the weight holds two stacked matrices
    ``[2n, k]`` and the epilogue sees ``acc`` (rows ``0..n``) and ``acc2`` (rows
    ``n..2n``) — the SwiGLU gate/up pair computed in one pass over ``a``.

    The element-wise tail has two phases so a fused kernel can reproduce the
    rounding points of an eager module: ``epilogue`` maps the fp32 accumulator(s)
    (names ``acc``, ``acc2``) and is rounded to ``out_dtype``; ``post`` then maps
    that value (name ``y``) together with ``epilogue_operands`` (``[m, n]``
    tensors of ``out_dtype`` such as a residual) and is rounded again."""

    m: int
    n: int
    k: int
    a: str
    b: str
    out: str
    in_dtype: DType
    out_dtype: DType
    epilogue: Expr | None = None
    post: Expr | None = None
    epilogue_operands: tuple[tuple[str, DType], ...] = ()
    gate_pair: bool = False
    tile: TilePlan | None = None
    stage: Stage | None = None
    reduce: ReducePlan = field(default_factory=ReducePlan)  # split-K
    lda: int | None = None
    ldb: int | None = None
    ldo: int | None = None
    a_offset: int = 0
    b_offset: int = 0
    out_offset: int = 0
    operand_buffers: dict = field(default_factory=dict)  # epilogue operand name -> buffer id
    a_prologue: RowPrologue | None = None
    bias: str | None = None  # length-n vector the epilogue may name ``bias`` (added to the fp32 accumulator)
    bias_dtype: DType | None = None
    row_epilogue: RowEpilogue | None = None
    # Set by the lowering on the *partial* kernel of a cross-workgroup split (``REDUCE=g<n>a|k``): ``(n, mode)``.
    # ``k`` is then one slice of the reduction extent, workgroup ``blockIdx.y`` takes slice ``blockIdx.y`` of both
    # operands, and the fp32 accumulators go to plane ``blockIdx.y`` of the workspace (``"kernel"``) or are added
    # atomically into its single zeroed plane (``"atomic"``).
    k_split: tuple[int, str] | None = None
    # ``batch`` independent products in one launch (workgroup row ``blockIdx.y`` takes product ``blockIdx.y``): the
    # operands and the result of product ``p`` start ``p * a_batch`` / ``p * b_batch`` / ``p * out_batch`` elements
    # further on (``b_batch`` 0: every product reads the same ``b``).  Plain products only: no bias, prologue, row
    # epilogue or epilogue operands, no split.
    batch: int = 1
    a_batch: int = 0
    b_batch: int = 0
    out_batch: int = 0

    def algo_flops(self) -> int:
        return 2 * self.m * self.n * self.k * (2 if self.gate_pair else 1) * self.batch

    def algo_bytes(self) -> int:
        nb = self.n * (2 if self.gate_pair else 1)
        if self.batch > 1:
            return self.batch * (self.m * self.k * self.in_dtype.nbytes + self.m * self.n * self.out_dtype.nbytes) + (self.batch if self.b_batch else 1) * nb * self.k * self.in_dtype.nbytes
        b = (self.m * self.k + nb * self.k) * self.in_dtype.nbytes + self.m * self.n * self.out_dtype.nbytes
        for _, dt in self.epilogue_operands:
            b += self.m * self.n * dt.nbytes
        if self.a_prologue is not None and self.a_prologue.weight is not None:
            b += self.k * self.a_prologue.weight_dtype.nbytes
        if self.bias is not None:
            b += self.n * self.bias_dtype.nbytes
        if self.row_epilogue is not None:
            for ro in self.row_epilogue.row_operands:
                b += ro.mod * self.row_epilogue.cols * ro.dtype.nbytes
        return b


@dataclass
class Flash:
    """Fused attention ``softmax(q k^T * scale + causal) v`` with grouped KV
    heads (``kv head = q head // group``), streamed over keys with the online
    (m, l, O) carrier (emmy/compiler/pipeline/passes/lowering/kernel/_twist.py:229-363).

    Tensors are addressed as ``base + b*stride_b + h*stride_h + s*stride_s + d``
    (``d`` contiguous), so ``[B,H,S,D]`` and ``[B,S,H,D]`` both fit."""

    batch: int
    q_heads: int
    kv_heads: int
    q_len: int
    kv_len: int
    head_dim: int
    q: str
    k: str
    v: str
    out: str
    dtype: DType
    scale: float
    causal: bool
    q_strides: tuple[int, int, int]  # (batch, head, seq) in elements
    k_strides: tuple[int, int, int]
    v_strides: tuple[int, int, int]
    o_strides: tuple[int, int, int]
    q_offset: int = 0
    k_offset: int = 0
    v_offset: int = 0
    o_offset: int = 0
    block_q: int = 128
    block_kv: int = 64
    waves: int = 4  # 32-row query groups per workgroup
    kv_split: int = 1  # wave groups that split the key blocks of a query group between them
    pair: bool = False  # causal only: a workgroup takes query block b and its mirror QBLOCKS-1-b
    deep: bool = False  # a K ring of three slots (K blocks requested two steps ahead) beside a V ring of two
    pair_steps: bool = True  # key steps unrolled in pairs so ring slots are compile-time (the lowering clears it if that build spills)
    mfma_sum: bool = False  # the row sums come out of the matrix pipe (an all-ones operand against the P fragments) instead of one add per probability
    ws: bool = False  # wave-specialised form: four consumer waves (waves x kv_split = 4) and four staging waves
    sp: bool = False  # software-pipelined form without staging waves: eight consumer waves (waves x kv_split = 8) stage for themselves
    one_region: bool = False  # fp32 key-split form: a wave's K and V blocks take turns in one LDS region (half the LDS a wave, two waves a SIMD)
    private: bool = False  # short sequences: one row group whose kv_split waves each stage and stream their own key blocks (no barrier in the loop)
    # cross-workgroup split of the keys (``REDUCE=g<n>k``): ``kv_ctas`` workgroups per query block each take a contiguous
    # slice of the keys and leave their (m, l, O) in a workspace; a combine kernel merges the slices.  ``partials`` names
    # the workspace when this body is the partial kernel of such a pair.
    kv_ctas: int = 1
    partials: str | None = None
    # rows of the operands hold ``head_dim_real`` values when that is not one of the kernel's widths: ``head_dim`` is then
    # the next width up, the missing columns of q count as zeros (k's and v's are never looked at: their products with a
    # zero vanish, their output columns are not stored)
    head_dim_real: int | None = None
    # an additive bias on the scaled scores, ``[batch, head, query, key]`` addressed through (batch, head, query)
    # strides (0 = broadcast) with keys contiguous; ``None``: no mask operand
    mask: str | None = None
    mask_dtype: DType | None = None
    mask_strides: tuple[int, int, int] = (0, 0, 0)
    mask_offset: int = 0

    def algo_flops(self) -> int:
        if self.causal and self.q_len == self.kv_len:
            pairs = self.q_len * (self.q_len + 1) // 2
        else:
            pairs = self.q_len * self.kv_len
        return 4 * self.batch * self.q_heads * (self.head_dim_real or self.head_dim) * pairs

    def algo_bytes(self) -> int:
        e = self.dtype.nbytes
        q = self.batch * self.q_heads * self.q_len * (self.head_dim_real or self.head_dim)
        kv = self.batch * self.kv_heads * self.kv_len * (self.head_dim_real or self.head_dim)
        mask = 0
        if self.mask is not None:
            mb, mh, mq = self.mask_strides
            mask = (self.batch if mb else 1) * (self.q_heads if mh else 1) * (self.q_len if mq else 1) * self.kv_len * self.mask_dtype.nbytes
        return (2 * q + 2 * kv) * e + mask


@dataclass
class MapOperand:
    """One pointwise input.  ``index`` names the addressing scheme:
    ``"flat"`` (same linear index as the output), ``"col"`` (a vector along the
    innermost axis), ``"row"`` (one value per output row) or ``"scalar"``."""

    name: str
    dtype: DType
    index: str = "flat"


@dataclass
class Map:
    """Pointwise kernel: ``out[i] = expr(operands[i])`` over ``numel`` cells."""

    numel: int
    operands: tuple[MapOperand, ...]
    expr: Expr
    out: str
    out_dtype: DType
    inner: int = 1  # extent of the innermost axis, for "col" broadcasts
    operand_buffers: dict = field(default_factory=dict)  # operand name -> buffer id
    operand_offsets: dict = field(default_factory=dict)  # operand name -> element offset

    def algo_bytes(self) -> int:
        b = self.numel * self.out_dtype.nbytes
        for o in self.operands:
            b += {"flat": self.numel, "col": self.inner, "row": self.numel // max(self.inner, 1), "scalar": 1}[o.index] * o.dtype.nbytes
        return b


@dataclass
class StridedCopy:
    """A dense row-major tensor made from a strided view of ``src``: result axis ``i`` has ``axes[i] = (extent,
    source extent, source stride)``; where the result extends past the source it is zero (``emit/copy.py``)."""

    src: str
    out: str
    dtype: DType
    src_offset: int
    src_numel: int
    axes: tuple  # ((result extent, source extent, source stride), ...) in result order

    def algo_flops(self) -> int:
        return 0

    def algo_bytes(self) -> int:
        import math

        return int((math.prod(se for _, se, _ in self.axes) + math.prod(de for de, _, _ in self.axes)) * self.dtype.nbytes)


@dataclass
class IndexRows:
    """``out[o, j, i] = src[o, idx[j], i]`` over a dense ``src [outer, n, inner]`` and an integer vector ``idx [count]``
    (an embedding lookup, ``index_select``); an index outside ``[0, n)`` is clamped (``emit/copy.py``)."""

    src: str
    idx: str
    out: str
    dtype: DType
    idx_dtype: DType
    outer: int
    n: int
    inner: int
    count: int

    def algo_flops(self) -> int:
        return 0

    def algo_bytes(self) -> int:
        return int(2 * self.outer * self.count * self.inner * self.dtype.nbytes + self.count * self.idx_dtype.nbytes)


@dataclass
class LoopNest:
    """A Loop-IR body rendered as it stands (``emit/loopnest.py``): the statements of a reference ``LoopOp``
    (``ir/loopnest.py``), the tensors its ``Load`` statements name, and scalar constants folded into the text."""

    stmts: tuple
    operands: dict  # Load.input name -> (buffer id, shape, dtype)
    scalars: dict  # Load.input name -> python float (a shape-[1] constant with a recorded value)
    out: str  # buffer id of the result
    out_name: str  # the name ``Write`` statements use for it
    out_shape: tuple[int, ...]
    out_dtype: DType

    def _weights(self) -> tuple[int, int]:
        """``(arithmetic statements executed, elements loaded)`` over the whole iteration space."""
        from deplodock_amd.ir import loopnest as L

        def run(body, times):
            ops = loads = 0
            for s in body:
                if isinstance(s, L.Loop):
                    o, l_ = run(s.body, times * s.extent)
                    ops, loads = ops + o, loads + l_
                elif isinstance(s, (L.Assign, L.Accum)):
                    ops += times
                elif isinstance(s, L.Load):
                    loads += times
            return ops, loads

        return run(self.stmts, 1)

    def algo_flops(self) -> int:
        return self._weights()[0]

    def algo_bytes(self) -> int:
        import math

        seen = {buf: math.prod(shape) * dt.nbytes for buf, shape, dt in self.operands.values()}
        return int(sum(seen.values()) + math.prod(self.out_shape) * self.out_dtype.nbytes)


@dataclass
class TileOp(Op):
    """One kernel: a name plus a scheduled body."""

    name: str = ""
    body: object = None

    def pretty_body(self) -> str:
        return f"{self.name}: {self.body!r}"
