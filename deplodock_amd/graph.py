"""Graph / Node / Tensor — the container every IR level shares.

A deliberately small equivalent of the reference's graph core
(emmy/compiler/graph.py:364-1000, tensor.py): nodes keyed by id, each with an
op, ordered input ids and one output ``Tensor``; ``inputs`` / ``outputs`` name
the boundary nodes.  Shapes are static ints here (a symbolic extent is a
``str`` name resolved at launch).
"""

from __future__ import annotations

from collections.abc import Iterator
from dataclasses import dataclass, field

from deplodock_amd.dtype import F32, DType, by_name
from deplodock_amd.ir.base import ConstantOp, InputOp, Op


@dataclass
class Tensor:
    """Symbolic descriptor of a buffer: name, shape, dtype (tensor.py:23-60)."""

    name: str
    shape: tuple
    dtype: DType = F32
    constant: bool = False
    value: float | None = None

    def __post_init__(self) -> None:
        if isinstance(self.dtype, str):
            self.dtype = by_name(self.dtype)
        self.shape = tuple(self.shape)

    @property
    def numel(self) -> int:
        n = 1
        for d in self.shape:
            n *= int(d)
        return n

    @property
    def nbytes(self) -> int:
        return self.numel * self.dtype.nbytes


@dataclass
class Node:
    id: str
    op: Op
    inputs: list[str]
    output: Tensor
    hints: dict = field(default_factory=dict)


class Graph:
    def __init__(self) -> None:
        self.nodes: dict[str, Node] = {}
        self.inputs: list[str] = []
        self.outputs: list[str] = []
        self._counter = 0

    # -- construction -----------------------------------------------------
    def _next_id(self, prefix: str = "n") -> str:
        while True:
            nid = f"{prefix}{self._counter}"
            self._counter += 1
            if nid not in self.nodes:
                return nid

    def add_node(self, op: Op, inputs: list[str], output: Tensor, node_id: str | None = None) -> str:
        nid = node_id or output.name or self._next_id()
        if nid in self.nodes:
            raise ValueError(f"duplicate node id {nid!r}")
        for i in inputs:
            if i not in self.nodes:
                raise KeyError(f"node {nid!r} references unknown input {i!r}")
        output.name = nid
        self.nodes[nid] = Node(nid, op, list(inputs), output)
        if isinstance(op, InputOp):
            self.inputs.append(nid)
        return nid

    def add_input(self, name: str, shape, dtype: DType = F32) -> str:
        return self.add_node(InputOp(), [], Tensor(name, shape, dtype), name)

    def add_constant(self, name: str, shape, dtype: DType = F32, value: float | None = None, source_path: str | None = None) -> str:
        t = Tensor(name, shape, dtype, constant=True, value=value)
        return self.add_node(ConstantOp(name=name, value=value, source_path=source_path), [], t, name)

    def remove_node(self, node_id: str) -> None:
        if self.consumers(node_id):
            raise ValueError(f"cannot remove {node_id!r}: it still has consumers")
        del self.nodes[node_id]
        if node_id in self.inputs:
            self.inputs.remove(node_id)
        if node_id in self.outputs:
            self.outputs.remove(node_id)

    # -- queries ------------------------------------------------------------
    def consumers(self, node_id: str) -> list[str]:
        return [n.id for n in self.nodes.values() if node_id in n.inputs]

    def constant_ops(self) -> Iterator[tuple[str, ConstantOp]]:
        for nid, n in self.nodes.items():
            if isinstance(n.op, ConstantOp):
                yield nid, n.op

    def node_role(self, node_id: str) -> str:
        """``input`` / ``constant`` / ``output`` / ``scratch`` (graph.py:673-684)."""
        n = self.nodes[node_id]
        if isinstance(n.op, InputOp):
            return "input"
        if isinstance(n.op, ConstantOp):
            return "constant"
        return "output" if node_id in self.outputs else "scratch"

    def topological_order(self) -> list[str]:
        order: list[str] = []
        state: dict[str, int] = {}

        def visit(nid: str) -> None:
            st = state.get(nid, 0)
            if st == 2:
                return
            if st == 1:
                raise ValueError(f"cycle through {nid!r}")
            state[nid] = 1
            for i in self.nodes[nid].inputs:
                visit(i)
            state[nid] = 2
            order.append(nid)

        for nid in self.nodes:
            visit(nid)
        return order

    def copy(self) -> Graph:
        g = Graph()
        for nid in self.topological_order():
            n = self.nodes[nid]
            g.nodes[nid] = Node(nid, n.op, list(n.inputs), Tensor(n.output.name, n.output.shape, n.output.dtype, n.output.constant, n.output.value), dict(n.hints))
        g.inputs = list(self.inputs)
        g.outputs = list(self.outputs)
        g._counter = self._counter
        return g

    def pretty_print(self) -> str:
        lines = []
        for nid in self.topological_order():
            n = self.nodes[nid]
            shape = "x".join(str(d) for d in n.output.shape)
            mark = " -> out" if nid in self.outputs else ""
            lines.append(f"{nid}: {type(n.op).__name__}({', '.join(n.inputs)}) [{shape} {n.output.dtype}]{mark}")
        return "\n".join(lines)
