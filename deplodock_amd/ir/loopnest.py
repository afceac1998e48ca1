"""The reference's Loop-IR statement vocabulary, read from its textual form.

A ``LoopOp`` of the reference serialises its body as a list of ``repr`` strings (emmy/compiler/graph.py:875-960,
one string per top-level statement), e.g. ``Loop(axis=Axis(name='a0', extent=128), body=(Load(...), Accum(...)))``.
The statement classes are emmy/compiler/ir/stmt/leaves.py (``Load`` :97, ``Assign`` :341, ``Accum`` :425,
``Write`` :708, ``Select`` / ``SelectBranch`` :886-894) and stmt/blocks.py:41 (``Loop``); index expressions are
emmy/compiler/ir/expr.py (``Var`` :184, ``Literal`` :219, ``BinaryExpr`` :265, ``TernaryExpr`` :490).

The reference reads that text back by evaluating it.  Here it is *parsed*: the text goes through ``ast.parse`` and
only calls of the names below, tuples and literals are accepted — nothing in the file is executed.

Semantics kept from the reference:

* ``Accum(name, value, op)`` folds ``value`` over the iterations of the loop that directly encloses it, starting
  from the operation's identity; the result is visible under ``name`` after that loop (leaves.py:425-447);
* ``Select`` binds the value of the first branch whose predicate holds (leaves.py:894-903);
* index arithmetic is integer arithmetic with *floor* division and modulo for ``/``, ``//`` and ``%``
  (expr.py:125-148) — a rotary embedding's ``a3 - 32`` makes negative intermediate values that wrap.
"""

from __future__ import annotations

import ast
from dataclasses import dataclass


class LoopNestError(ValueError):
    """The text is not a Loop-IR body this backend reads."""


@dataclass(frozen=True)
class Var:
    name: str


@dataclass(frozen=True)
class Lit:
    value: int | float


@dataclass(frozen=True)
class Bin:
    op: str
    left: object
    right: object


@dataclass(frozen=True)
class Ternary:
    cond: object
    if_true: object
    if_false: object


@dataclass(frozen=True)
class Load:
    name: str
    input: str
    index: tuple


@dataclass(frozen=True)
class Assign:
    name: str
    op: str
    args: tuple[str, ...]


@dataclass(frozen=True)
class Accum:
    name: str
    value: str
    op: str


@dataclass(frozen=True)
class Select:
    name: str
    branches: tuple[tuple[str, object], ...]  # (value, predicate)


@dataclass(frozen=True)
class Write:
    output: str
    index: tuple
    value: str


@dataclass(frozen=True)
class Loop:
    axis: str
    extent: int
    body: tuple


BIN_OPS = ("+", "-", "*", "/", "//", "%", "<", "<=", ">", ">=", "==", "&&", "||")
UNARY_OPS = ("negative", "reciprocal", "rsqrt", "sqrt", "exp", "log", "tanh", "sigmoid", "silu", "abs", "relu", "square")
BINARY_OPS = ("add", "subtract", "multiply", "divide", "maximum", "minimum")
ACCUM_IDENTITY = {"add": 0.0, "multiply": 1.0, "maximum": float("-inf"), "minimum": float("inf")}


def _kw(call: ast.Call, what: str, names: tuple[str, ...], optional: tuple[str, ...] = ()) -> dict:
    """Keyword (or positional, in declaration order) arguments of ``call`` as a dict of AST nodes."""
    got: dict[str, ast.AST] = {}
    order = names + optional
    if len(call.args) > len(order):
        raise LoopNestError(f"{what}: too many positional arguments")
    for key, arg in zip(order, call.args):
        got[key] = arg
    for k in call.keywords:
        if k.arg is None or k.arg in got:
            raise LoopNestError(f"{what}: bad keyword {k.arg!r}")
        got[k.arg] = k.value
    for key in names:
        if key not in got:
            raise LoopNestError(f"{what}: missing {key!r}")
    return got


def _const(node: ast.AST, what: str, types: tuple[type, ...]):
    if isinstance(node, ast.UnaryOp) and isinstance(node.op, ast.USub) and isinstance(node.operand, ast.Constant) and isinstance(node.operand.value, (int, float)):
        value = -node.operand.value
    elif isinstance(node, ast.Constant):
        value = node.value
    else:
        raise LoopNestError(f"{what}: expected a literal")
    if isinstance(value, bool) or not isinstance(value, types):
        raise LoopNestError(f"{what}: expected {' or '.join(t.__name__ for t in types)}, got {value!r}")
    return value


def _is_none(node: ast.AST) -> bool:
    return isinstance(node, ast.Constant) and node.value is None


def _tuple(node: ast.AST, what: str) -> list[ast.AST]:
    if not isinstance(node, (ast.Tuple, ast.List)):
        raise LoopNestError(f"{what}: expected a tuple")
    return list(node.elts)


def _callee(node: ast.AST, what: str) -> tuple[str, ast.Call]:
    if not (isinstance(node, ast.Call) and isinstance(node.func, ast.Name)):
        raise LoopNestError(f"{what}: expected a constructor call")
    return node.func.id, node


def _impl(node: ast.AST, what: str) -> str:
    name, call = _callee(node, what)
    if name != "ElementwiseImpl":
        raise LoopNestError(f"{what}: expected ElementwiseImpl(...), got {name}")
    return _const(_kw(call, what, ("name",))["name"], what, (str,))


def _expr(node: ast.AST):
    name, call = _callee(node, "index expression")
    if name == "Var":
        return Var(_const(_kw(call, name, ("name",))["name"], name, (str,)))
    if name == "Literal":
        kw = _kw(call, name, ("value",), ("dtype",))
        return Lit(_const(kw["value"], name, (int, float)))
    if name == "BinaryExpr":
        kw = _kw(call, name, ("op", "left", "right"))
        op = _const(kw["op"], name, (str,))
        if op not in BIN_OPS:
            raise LoopNestError(f"BinaryExpr: operator {op!r} is not read")
        return Bin(op, _expr(kw["left"]), _expr(kw["right"]))
    if name == "TernaryExpr":
        kw = _kw(call, name, ("cond", "if_true", "if_false"))
        return Ternary(_expr(kw["cond"]), _expr(kw["if_true"]), _expr(kw["if_false"]))
    raise LoopNestError(f"index expression: {name}(...) is not read")


def _stmt(node: ast.AST):
    name, call = _callee(node, "statement")
    if name == "Loop":
        kw = _kw(call, name, ("axis", "body"), ("unroll",))
        an, ac = _callee(kw["axis"], "Loop.axis")
        if an != "Axis":
            raise LoopNestError("Loop.axis: expected Axis(...)")
        akw = _kw(ac, "Axis", ("name", "extent"), ("source_axis", "role"))
        try:
            extent = _const(akw["extent"], "Axis.extent", (int,))
        except LoopNestError as exc:
            raise LoopNestError("Axis.extent: a symbolic extent is not read; write the kernel at concrete sizes") from exc
        if extent < 1:
            raise LoopNestError(f"Axis.extent: {extent}")
        return Loop(_const(akw["name"], "Axis.name", (str,)), extent, tuple(_stmt(s) for s in _tuple(kw["body"], "Loop.body")))
    if name == "Load":
        kw = _kw(call, name, (), ("name", "input", "index", "dtype", "names"))
        if "names" in kw and not _is_none(kw["names"]):
            names = [_const(n, "Load.names", (str,)) for n in _tuple(kw["names"], "Load.names")]
            if len(names) != 1:
                raise LoopNestError("Load: a vector load (the reference's vectorize pass) is a later stage than the Loop IR read here")
            lname = names[0]
        elif "name" in kw:
            lname = _const(kw["name"], "Load.name", (str,))
        else:
            raise LoopNestError("Load: missing name")
        if "input" not in kw or "index" not in kw:
            raise LoopNestError("Load: missing input / index")
        return Load(lname, _const(kw["input"], "Load.input", (str,)), tuple(_expr(e) for e in _tuple(kw["index"], "Load.index")))
    if name == "Assign":
        kw = _kw(call, name, ("name", "op", "args"), ("dtype",))
        op = _impl(kw["op"], "Assign.op")
        args = tuple(_const(a, "Assign.args", (str,)) for a in _tuple(kw["args"], "Assign.args"))
        if (op in UNARY_OPS and len(args) != 1) or (op in BINARY_OPS and len(args) != 2) or op not in UNARY_OPS + BINARY_OPS:
            raise LoopNestError(f"Assign: operation {op!r} with {len(args)} argument(s) is not read")
        return Assign(_const(kw["name"], "Assign.name", (str,)), op, args)
    if name == "Accum":
        kw = _kw(call, name, ("name", "value"), ("op", "dtype", "axes", "base"))
        if "base" in kw and not _is_none(kw["base"]):
            raise LoopNestError("Accum: a rescaled base (a streaming carrier) is a later stage than the Loop IR read here")
        op = _impl(kw["op"], "Accum.op") if "op" in kw else "add"
        if op not in ACCUM_IDENTITY:
            raise LoopNestError(f"Accum: operation {op!r} has no identity here")
        return Accum(_const(kw["name"], "Accum.name", (str,)), _const(kw["value"], "Accum.value", (str,)), op)
    if name == "Select":
        kw = _kw(call, name, ("name", "branches"))
        branches = []
        for b in _tuple(kw["branches"], "Select.branches"):
            bn, bc = _callee(b, "Select.branches")
            if bn != "SelectBranch":
                raise LoopNestError("Select.branches: expected SelectBranch(...)")
            bkw = _kw(bc, bn, ("value", "select"))
            branches.append((_const(bkw["value"], "SelectBranch.value", (str,)), _expr(bkw["select"])))
        if not branches:
            raise LoopNestError("Select: no branches")
        return Select(_const(kw["name"], "Select.name", (str,)), tuple(branches))
    if name == "Write":
        kw = _kw(call, name, ("output", "index", "value"), ("dtype",))
        return Write(_const(kw["output"], "Write.output", (str,)), tuple(_expr(e) for e in _tuple(kw["index"], "Write.index")), _const(kw["value"], "Write.value", (str,)))
    raise LoopNestError(f"statement {name}(...) is not read (tile- and kernel-stage statements belong to the reference's own lowering)")


def parse_body(texts: list[str] | tuple[str, ...]) -> tuple:
    """The statements of a ``LoopOp`` body from their textual form, one string per top-level statement."""
    out = []
    for text in texts:
        if not isinstance(text, str) or len(text) > 4_000_000:
            raise LoopNestError("LoopOp.body: expected a list of statement strings")
        try:
            tree = ast.parse(text, mode="eval")
        except (SyntaxError, RecursionError, MemoryError) as exc:
            raise LoopNestError(f"LoopOp.body: not a statement expression ({type(exc).__name__})") from exc
        try:
            out.append(_stmt(tree.body))
        except RecursionError as exc:
            raise LoopNestError("LoopOp.body: expression nested too deeply") from exc
    stmts = tuple(out)
    check_body(stmts)
    return stmts


def walk(stmts):
    for s in stmts:
        yield s
        if isinstance(s, Loop):
            yield from walk(s.body)


def expr_vars(e) -> set[str]:
    if isinstance(e, Var):
        return {e.name}
    if isinstance(e, Bin):
        return expr_vars(e.left) | expr_vars(e.right)
    if isinstance(e, Ternary):
        return expr_vars(e.cond) | expr_vars(e.if_true) | expr_vars(e.if_false)
    return set()


def check_body(stmts: tuple) -> None:
    """Scoping rules the emitters and the interpreter rely on: a name is bound once on its path, used after it is
    bound (an ``Accum`` after its loop), and index expressions name enclosing loop axes only."""

    def run(body: tuple, bound: set[str], axes: tuple[str, ...], in_loop: bool) -> set[str]:
        bound = set(bound)
        accum_ops: dict[str, str] = {}
        for s in body:
            if isinstance(s, Loop):
                if s.axis in axes:
                    raise LoopNestError(f"loop axis {s.axis!r} is nested inside itself")
                inner = run(s.body, bound, axes + (s.axis,), True)
                for t in s.body:
                    if isinstance(t, Accum):
                        if t.name not in inner:
                            raise LoopNestError(f"Accum {t.name!r} is not bound")
                        bound.add(t.name)
                continue
            exprs = s.index if isinstance(s, (Load, Write)) else tuple(p for _, p in s.branches) if isinstance(s, Select) else ()
            for e in exprs:
                free = expr_vars(e) - set(axes)
                if free:
                    raise LoopNestError(f"{type(s).__name__}: index names {sorted(free)} outside their loops")
            uses = s.args if isinstance(s, Assign) else (s.value,) if isinstance(s, (Accum, Write)) else tuple(v for v, _ in s.branches) if isinstance(s, Select) else ()
            for u in uses:
                if u not in bound:
                    raise LoopNestError(f"{type(s).__name__}: {u!r} is used before it is bound")
            if isinstance(s, Accum):
                if not in_loop:
                    raise LoopNestError(f"Accum {s.name!r} sits outside every loop")
                if s.name in bound and accum_ops.get(s.name) != s.op:  # several folds into one name must agree on the operation
                    raise LoopNestError(f"name {s.name!r} is bound twice")
                accum_ops[s.name] = s.op
                bound.add(s.name)  # visible to the enclosing scope once the loop ends (the caller binds it there)
            elif not isinstance(s, Write):
                if s.name in bound:
                    raise LoopNestError(f"name {s.name!r} is bound twice")
                bound.add(s.name)
        return bound

    run(stmts, set(), (), False)


__all__ = ["LoopNestError", "Var", "Lit", "Bin", "Ternary", "Load", "Assign", "Accum", "Select", "Write", "Loop", "parse_body", "walk", "expr_vars",
           "check_body", "BIN_OPS", "UNARY_OPS", "BINARY_OPS", "ACCUM_IDENTITY"]  # fmt: skip
