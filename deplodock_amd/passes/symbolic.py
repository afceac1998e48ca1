"""Finding what depends on a symbolic axis, by lowering the module at several sizes.

The fusion pass works on concrete shapes.  To get kernels that take the symbolic extent as a runtime ``int``,
the traced module is fused at three sizes of the axis — the traced size and two others, one of them odd so that
alignment-dependent decisions show — and the three tile graphs are compared node by node: an integer field that
changes must change affinely (``a * size + b``, the same ``a`` and ``b`` through all three points) and must be
one of the fields the emitters can take at run time (row counts, a contraction's ``m``, attention lengths, the
position count of a table, a pointwise extent); anything else that differs — another kernel boundary, a stride,
an offset, a fusion decision — makes the module not symbolisable, and the caller keeps lowering per size.
"""

from __future__ import annotations

import dataclasses

from deplodock_amd.graph import Graph
from deplodock_amd.ir.base import ConstantOp
from deplodock_amd.ir.sym import Affine, SymSpec
from deplodock_amd.ir.tile import Contraction, Flash, IndexRows, Map, RowReduce, TileOp


class SymbolicError(ValueError):
    """The module's lowering changes shape with the symbolic axis in a way a runtime ``int`` cannot express."""


# field paths (with tuple indices written as ``*``) that may follow the axis, per body type
_ALLOWED = {
    RowReduce: {"rows", "row_operands.*.mod"},
    Contraction: {"m", "row_epilogue.row_operands.*.mod"},
    # the batch stride of a [B, H, S, D] tensor follows S; so does the row stride of a mask [.., S, S] (its head and batch
    # strides are quadratic in S unless the mask is broadcast over them, and a quadratic field is refused by the fit)
    Flash: {"q_len", "kv_len", "q_strides.*", "k_strides.*", "v_strides.*", "o_strides.*", "mask_strides.*"},
    Map: {"numel"},
    IndexRows: {"count"},  # token ids [batch, seq_len] into a table that does not follow the axis
}


def _fit(name: str, sizes: list[int], values: list[int], what: str) -> Affine:
    (s0, s1, s2), (v0, v1, v2) = sizes, values
    if (v1 - v0) % (s1 - s0):
        raise SymbolicError(f"{what} is not affine in {name}: {values} at {sizes}")
    a = (v1 - v0) // (s1 - s0)
    b = v0 - a * s0
    if a * s2 + b != v2:
        raise SymbolicError(f"{what} is not affine in {name}: {values} at {sizes}")
    return Affine(name, a, b)


def _walk(objs: list, path: str, pattern: str, allowed: set, name: str, sizes: list[int], out: dict, what: str) -> None:
    first = objs[0]
    if any(type(o) is not type(first) for o in objs):
        raise SymbolicError(f"{what}.{path} changes type with {name}")
    if dataclasses.is_dataclass(first) and not isinstance(first, type):
        for f in dataclasses.fields(first):
            sub = f"{path}.{f.name}" if path else f.name
            subp = f"{pattern}.{f.name}" if pattern else f.name
            _walk([getattr(o, f.name) for o in objs], sub, subp, allowed, name, sizes, out, what)
        return
    if isinstance(first, (tuple, list)):
        if any(len(o) != len(first) for o in objs):
            raise SymbolicError(f"{what}.{path} changes length with {name}")
        for i in range(len(first)):
            _walk([o[i] for o in objs], f"{path}.{i}", f"{pattern}.*", allowed, name, sizes, out, what)
        return
    if isinstance(first, dict):
        if any(set(o) != set(first) for o in objs):
            raise SymbolicError(f"{what}.{path} changes keys with {name}")
        for k in first:
            _walk([o[k] for o in objs], f"{path}.{k}", f"{pattern}.*", allowed, name, sizes, out, what)
        return
    if all(o == first for o in objs[1:]):
        return
    if isinstance(first, int) and not isinstance(first, bool) and pattern in allowed:
        out[path] = _fit(name, sizes, [int(o) for o in objs], f"{what}.{path}")
        return
    raise SymbolicError(f"{what}.{path} depends on {name} ({[o for o in objs]}), which a runtime int cannot express")


def _prefix_table(nid: str, sym_shape: tuple, values: list, name: str) -> int:
    """A constant whose shape follows the axis is a table computed from the positions when the module was traced (a
    rotary embedding's cos / sin rows).  One compilation can serve every size only if the table at a smaller size is
    the leading rows of the table at a larger one, laid out so that those rows are a prefix of the memory: exactly one
    dim follows the axis, every dim before it is 1, and the traced values agree on their common rows.  Returns that
    dim; the runtime then binds the leading rows of the largest table it has and re-traces for a larger one."""
    dims = [i for i, d in enumerate(sym_shape) if isinstance(d, Affine)]
    if len(dims) != 1 or any(d != 1 for d in sym_shape[: dims[0]]) or sym_shape[dims[0]].a < 1:
        raise SymbolicError(f"constant {nid!r} of shape {sym_shape} follows {name} in more than its leading dim")
    if any(v is None for v in values):
        raise SymbolicError(f"constant {nid!r} follows {name} and has no traced value to compare across sizes")
    d = dims[0]
    for v in values[1:]:
        small, large = (values[0], v) if values[0].shape[d] <= v.shape[d] else (v, values[0])
        if small.dtype != large.dtype or not bool((large.narrow(d, 0, small.shape[d]) == small).all()):
            raise SymbolicError(f"constant {nid!r} follows {name} and its rows at one size are not the leading rows at a larger size")
    return d


def symbolize(tiles: list[Graph], name: str, sizes: list[int]) -> Graph:
    """Annotate the tile graph of ``sizes[0]`` (the traced size): every ``TileOp`` body gets ``sym`` (a
    ``SymSpec``), every node ``hints['sym_shape']`` (its shape with ``Affine`` entries).  ``tiles`` are the fused,
    unscheduled tile graphs of the same module at ``sizes``."""
    base = tiles[0]
    for other in tiles[1:]:
        if list(other.nodes) != list(base.nodes) or other.inputs != base.inputs or other.outputs != base.outputs:
            raise SymbolicError(f"the kernel boundaries change with {name}")
    for nid, node in base.nodes.items():
        peers = [t.nodes[nid] for t in tiles]
        if any(type(p.op) is not type(node.op) or p.inputs != node.inputs or p.output.dtype != node.output.dtype for p in peers):
            raise SymbolicError(f"node {nid!r} changes with {name}")
        shapes = [tuple(int(d) for d in p.output.shape) for p in peers]
        if any(len(s) != len(shapes[0]) for s in shapes):
            raise SymbolicError(f"node {nid!r} changes rank with {name}")
        sym_shape = tuple(d[0] if len(set(d)) == 1 else _fit(name, sizes, list(d), f"{nid}.shape") for d in zip(*shapes))
        if any(isinstance(d, Affine) for d in sym_shape):
            node.hints["sym_shape"] = sym_shape
            if isinstance(node.op, ConstantOp):
                node.hints["prefix_table"] = _prefix_table(nid, sym_shape, [getattr(t, "constant_values", {}).get(nid) for t in tiles], name)
        # hints that carry views (logical shapes / strides over a buffer) must not depend on the axis either,
        # except through the shape entries the program resolves per launch
        if isinstance(node.op, TileOp):
            bodies = [p.op.body for p in peers]
            if any(type(b) is not type(bodies[0]) for b in bodies):
                raise SymbolicError(f"kernel {nid!r} changes kind with {name}")
            fields: dict = {}
            allowed = _ALLOWED.get(type(bodies[0]))
            if allowed is None:
                raise SymbolicError(f"kernel {nid!r}: {type(bodies[0]).__name__} has no symbolic form")
            _walk(bodies, "", "", allowed, name, sizes, fields, nid)
            node.op.body.sym = SymSpec(name, sizes[0], fields)
    return base


__all__ = ["SymbolicError", "symbolize"]
