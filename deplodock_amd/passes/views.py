"""Strided views: layout ops collapse into addressing instead of kernels.

``view`` / ``transpose`` / ``permute`` / ``unsqueeze`` / ``squeeze`` / ``slice``
never move data here: a consumer kernel is handed ``(base buffer, offset,
strides)`` and addresses the producer's memory directly.  (The reference turns
the same ops into ``IndexMap`` nodes that fuse into their consumers' index
expressions, emmy/compiler/pipeline/passes/frontend/decomposition/ layout rules.)
"""

from __future__ import annotations

from dataclasses import dataclass

from deplodock_amd.dtype import DType
from deplodock_amd.graph import Graph
from deplodock_amd.ir import frontend as F


@dataclass(frozen=True)
class View:
    base: str  # id of the node that owns the memory
    offset: int  # elements
    shape: tuple[int, ...]
    strides: tuple[int, ...]  # elements
    dtype: DType

    @property
    def numel(self) -> int:
        n = 1
        for d in self.shape:
            n *= d
        return n

    def is_contiguous(self) -> bool:
        """Row-major dense; the stride of a size-1 dimension is irrelevant."""
        want = contiguous_strides(self.shape)
        return all(n == 1 or s == w for n, s, w in zip(self.shape, self.strides, want))

    def collapse_leading(self, keep: int) -> tuple[int, int] | None:
        """If all but the last ``keep`` dims form one uniformly strided run,
        return ``(count, stride)`` of that run, else ``None``."""
        lead_shape = self.shape[: len(self.shape) - keep]
        lead_strides = self.strides[: len(self.strides) - keep]
        dims = [(n, s) for n, s in zip(lead_shape, lead_strides) if n != 1]
        if not dims:
            return (1, 0)
        count, stride = dims[-1]
        for n, s in reversed(dims[:-1]):
            if s != stride * count:
                return None
            count *= n
        return (count, stride)


def contiguous_strides(shape: tuple[int, ...]) -> tuple[int, ...]:
    out = []
    acc = 1
    for d in reversed(shape):
        out.append(acc)
        acc *= d
    return tuple(reversed(out))


LAYOUT_OPS = (F.ViewOp, F.TransposeOp, F.PermuteOp, F.UnsqueezeOp, F.SqueezeOp, F.SliceOp, F.ExpandOp)


def _reshape_strides(shape: tuple[int, ...], strides: tuple[int, ...], new_shape: tuple[int, ...]) -> tuple[int, ...] | None:
    """Strides that present the same elements in ``new_shape`` without a copy, or ``None``."""
    old: list[tuple[int, int]] = []
    for n, s in zip(shape, strides):
        if n == 1:
            continue
        if old and old[-1][1] == s * n:
            old[-1] = (old[-1][0] * n, s)  # mutually contiguous neighbours are one run: any split of it is a view
        else:
            old.append((n, s))
    out: list[int] = []
    oi = 0
    ni = 0
    new = list(new_shape)
    while ni < len(new):
        n = new[ni]
        if n == 1:
            out.append(0)
            ni += 1
            continue
        if oi >= len(old):
            return None
        on, os = old[oi]
        if n == on:
            out.append(os)
            oi += 1
            ni += 1
        elif n < on:
            if on % n:
                return None
            # split the old dim: this new dim takes the slow part
            out.append(os * (on // n))
            old[oi] = (on // n, os)
            ni += 1
        else:
            # merge several old dims into this new dim: they must be mutually contiguous
            need = n
            run_stride = None
            while need > 1:
                if oi >= len(old):
                    return None
                on, os = old[oi]
                if need % on:
                    return None
                if run_stride is not None and run_stride != os * on:
                    return None
                run_stride = os
                need //= on
                oi += 1
            out.append(run_stride if run_stride is not None else 0)
            ni += 1
    if oi != len(old):
        return None
    return tuple(out)


def apply_layout(src: View, op, out_shape: tuple[int, ...], nid: str = "?") -> View:
    """The view that layout op ``op`` (producing ``out_shape``) presents of ``src``."""
    if isinstance(op, F.ViewOp):
        st = _reshape_strides(src.shape, src.strides, out_shape)
        if st is None:
            raise NotViewable(nid)
        return View(src.base, src.offset, out_shape, st, src.dtype)
    if isinstance(op, F.TransposeOp):
        sh, st = list(src.shape), list(src.strides)
        sh[op.dim0], sh[op.dim1] = sh[op.dim1], sh[op.dim0]
        st[op.dim0], st[op.dim1] = st[op.dim1], st[op.dim0]
        return View(src.base, src.offset, tuple(sh), tuple(st), src.dtype)
    if isinstance(op, F.PermuteOp):
        return View(src.base, src.offset, tuple(src.shape[d] for d in op.dims), tuple(src.strides[d] for d in op.dims), src.dtype)
    if isinstance(op, F.UnsqueezeOp):
        sh, st = list(src.shape), list(src.strides)
        sh.insert(op.dim, 1)
        st.insert(op.dim, 0)
        return View(src.base, src.offset, tuple(sh), tuple(st), src.dtype)
    if isinstance(op, F.ExpandOp):
        pad = len(out_shape) - len(src.shape)
        if pad < 0 or any(n not in (1, o) for n, o in zip(src.shape, out_shape[pad:])):
            raise NotViewable(nid)
        st = [0] * pad + [0 if n == 1 and o != 1 else s for n, o, s in zip(src.shape, out_shape[pad:], src.strides)]
        return View(src.base, src.offset, tuple(out_shape), tuple(st), src.dtype)
    if isinstance(op, F.SqueezeOp):
        sh, st = list(src.shape), list(src.strides)
        if sh[op.dim] == 1:
            del sh[op.dim]
            del st[op.dim]
        return View(src.base, src.offset, tuple(sh), tuple(st), src.dtype)
    if isinstance(op, F.SliceOp):
        if op.step != 1:
            raise NotViewable(nid)
        sh = list(src.shape)
        sh[op.dim] = op.end - op.start
        return View(src.base, src.offset + op.start * src.strides[op.dim], tuple(sh), src.strides, src.dtype)
    raise NotViewable(nid)


def resolve_view(g: Graph, nid: str) -> View:
    """Express node ``nid`` as a strided window into the nearest non-layout producer."""
    node = g.nodes[nid]
    shape = tuple(int(d) for d in node.output.shape)
    if not isinstance(node.op, LAYOUT_OPS):
        return View(nid, 0, shape, contiguous_strides(shape), node.output.dtype)
    return apply_layout(resolve_view(g, node.inputs[0]), node.op, shape, nid)


class NotViewable(ValueError):
    """A layout op cannot be expressed as strides over its producer (needs a copy)."""
