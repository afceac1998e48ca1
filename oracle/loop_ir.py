"""CPU restatement of the reference's Loop-IR semantics (test infrastructure: only tests/, smoke() and bench.py's
CPU leg may import this package; the product never does).

The reference evaluates a ``LoopOp`` by rendering its body to plain C++ loops over ``float32`` buffers
(emmy/compiler/ir/loop/ir.py:193-221) — sequential loops, ``Accum`` folding from the operation's identity over the
enclosing loop (emmy/compiler/ir/stmt/leaves.py:425-447), ``Select`` taking the first branch whose predicate holds
(:894-903), index arithmetic with floor division / modulo (emmy/compiler/ir/expr.py:125-148).  Two restatements
of exactly that:

* :func:`run_loops` — the statements executed one iteration at a time in Python: the definition, usable on tiny
  extents only;
* :func:`run_vectorised` — the same result with every loop axis turned into an array axis (numpy), outer loops run
  one iteration at a time where the iteration space would not fit in memory.  Checked against :func:`run_loops`
  on small nests and against PyTorch eager of the decoder layer the reference's kernel corpus was cut from
  (tests/test_loop_ir.py).
"""

from __future__ import annotations

import numpy as np

from deplodock_amd.ir import loopnest as L

_UNARY = {
    "negative": lambda x: -x,
    "reciprocal": lambda x: 1.0 / x,
    "rsqrt": lambda x: 1.0 / np.sqrt(x),
    "sqrt": np.sqrt,
    "exp": np.exp,
    "log": np.log,
    "tanh": np.tanh,
    "sigmoid": lambda x: 1.0 / (1.0 + np.exp(-x)),
    "silu": lambda x: x / (1.0 + np.exp(-x)),
    "abs": np.abs,
    "relu": lambda x: np.maximum(x, 0.0),
    "square": lambda x: x * x,
}
_BINARY = {"add": np.add, "subtract": np.subtract, "multiply": np.multiply, "divide": np.divide, "maximum": np.maximum, "minimum": np.minimum}
_REDUCE = {"add": np.sum, "multiply": np.prod, "maximum": np.max, "minimum": np.min}


def _index(e, env):
    """An index expression over ``env`` (axis name -> int or integer array); floor semantics for ``/`` and ``%``."""
    if isinstance(e, L.Var):
        return env[e.name]
    if isinstance(e, L.Lit):
        return e.value
    if isinstance(e, L.Ternary):
        return np.where(_index(e.cond, env), _index(e.if_true, env), _index(e.if_false, env))
    a, b = _index(e.left, env), _index(e.right, env)
    op = e.op
    if op == "+":
        return a + b
    if op == "-":
        return a - b
    if op == "*":
        return a * b
    if op in ("/", "//"):
        return a // b
    if op == "%":
        return a % b
    if op == "<":
        return a < b
    if op == "<=":
        return a <= b
    if op == ">":
        return a > b
    if op == ">=":
        return a >= b
    if op == "==":
        return a == b
    if op == "&&":
        return np.logical_and(a, b)
    if op == "||":
        return np.logical_or(a, b)
    raise ValueError(f"index operator {op!r}")


def run_loops(stmts: tuple, inputs: dict[str, np.ndarray], out_shape: tuple[int, ...], dtype=np.float64) -> np.ndarray:
    """The body executed literally: python loops, one scalar at a time."""
    out = np.zeros(out_shape, dtype=dtype)
    arrays = {k: np.asarray(v, dtype=dtype) for k, v in inputs.items()}

    def run(body, env, vals, acc):
        """One pass over ``body`` at the iteration ``env``; ``acc`` holds the accumulators of the enclosing loop."""
        for s in body:
            if isinstance(s, L.Loop):
                mine = {t.name: dtype(L.ACCUM_IDENTITY[t.op]) for t in s.body if isinstance(t, L.Accum)}
                for i in range(s.extent):
                    run(s.body, {**env, s.axis: i}, dict(vals), mine)  # what an iteration binds stays inside it
                vals.update(mine)
            elif isinstance(s, L.Load):
                vals[s.name] = arrays[s.input][tuple(int(_index(e, env)) for e in s.index)]
            elif isinstance(s, L.Assign):
                args = [vals[a] for a in s.args]
                vals[s.name] = dtype(_UNARY[s.op](args[0]) if s.op in _UNARY else _BINARY[s.op](*args))
            elif isinstance(s, L.Select):
                for v, pred in s.branches[:-1]:
                    if bool(_index(pred, env)):
                        vals[s.name] = vals[v]
                        break
                else:
                    vals[s.name] = vals[s.branches[-1][0]]  # the last branch is the catch-all
            elif isinstance(s, L.Accum):
                acc[s.name] = dtype(_BINARY[s.op](acc[s.name], vals[s.value]))
            elif isinstance(s, L.Write):
                out[tuple(int(_index(e, env)) for e in s.index)] = vals[s.value]

    run(stmts, {}, {}, {})
    return out


def _footprint(body: tuple) -> int:
    """Largest number of iteration points below ``body`` that the vectorised run would hold at once."""
    best = 1
    for s in body:
        if isinstance(s, L.Loop):
            best = max(best, s.extent * _footprint(s.body))
    return best


def run_vectorised(stmts: tuple, inputs: dict[str, np.ndarray], out_shape: tuple[int, ...], dtype=np.float64, budget: int = 1 << 24) -> np.ndarray:
    """Every loop axis an array axis; outer loops whose subtree would exceed ``budget`` points run one iteration
    at a time.  Invariant: at vector depth ``d`` every array value has ``d`` axes (extent or 1 each)."""
    out = np.zeros(out_shape, dtype=dtype)
    arrays = {k: np.asarray(v, dtype=dtype) for k, v in inputs.items()}

    def run(body, env, vals, depth, sequential_only):
        """Returns {accumulator name: (op, this body's contribution per point)} for the enclosing loop to fold."""
        accs: dict[str, tuple[str, object]] = {}
        for s in body:
            if isinstance(s, L.Loop):
                if sequential_only and s.extent * _footprint(s.body) > budget:
                    folded: dict[str, object] = {}
                    for i in range(s.extent):
                        inner = run(s.body, {**env, s.axis: i}, dict(vals), depth, True)
                        for name, (op, v) in inner.items():
                            folded[name] = v if i == 0 else _BINARY[op](folded[name], v)
                    vals.update(folded)
                else:
                    lift = lambda v: v[..., None] if isinstance(v, np.ndarray) and v.ndim == depth and depth > 0 else v  # noqa: E731
                    env2 = {k: lift(v) for k, v in env.items()}
                    env2[s.axis] = np.arange(s.extent).reshape((1,) * depth + (s.extent,))
                    inner = run(s.body, env2, {k: lift(v) for k, v in vals.items()}, depth + 1, False)
                    for name, (op, v) in inner.items():
                        full = np.broadcast_shapes(np.shape(v), (1,) * depth + (s.extent,))  # a value that does not vary along the loop is folded once per iteration all the same
                        vals[name] = _REDUCE[op](np.broadcast_to(v, full), axis=-1)
            elif isinstance(s, L.Load):
                idx = tuple(_index(e, env) for e in s.index)
                vals[s.name] = arrays[s.input][idx]
            elif isinstance(s, L.Assign):
                args = [vals[a] for a in s.args]
                vals[s.name] = np.asarray(_UNARY[s.op](args[0]) if s.op in _UNARY else _BINARY[s.op](*args), dtype=dtype)
            elif isinstance(s, L.Select):
                res = vals[s.branches[-1][0]]  # the last branch is the catch-all
                for v, pred in reversed(s.branches[:-1]):
                    res = np.where(_index(pred, env), vals[v], res)
                vals[s.name] = res
            elif isinstance(s, L.Accum):
                v = vals[s.value]
                accs[s.name] = (s.op, _BINARY[s.op](accs[s.name][1], v) if s.name in accs else v)
            elif isinstance(s, L.Write):
                idx = tuple(_index(e, env) for e in s.index)
                shape = np.broadcast_shapes(*(np.shape(i) for i in idx), np.shape(vals[s.value]))
                out[tuple(np.broadcast_to(i, shape) for i in idx)] = np.broadcast_to(vals[s.value], shape)
        return accs

    run(stmts, {}, {}, 0, True)
    return out


def infer_write_shape(stmts: tuple) -> tuple[int, ...]:
    """Output shape from the first ``Write``: per dimension, the largest index over the iteration space plus one
    (emmy/compiler/ir/loop/ir.py:223-252)."""
    extents: dict[str, int] = {}

    def find(body, axes):
        for s in body:
            if isinstance(s, L.Loop):
                r = find(s.body, {**axes, s.axis: s.extent})
                if r is not None:
                    return r
            elif isinstance(s, L.Write):
                extents.update(axes)
                return s
        return None

    w = find(stmts, {})
    if w is None:
        raise ValueError("no Write in the body")
    names = list(extents)
    env = {n: np.arange(extents[n]).reshape([extents[n] if m == n else 1 for m in names]) for n in names}
    return tuple(int(np.max(_index(e, env))) + 1 for e in w.index)


__all__ = ["run_loops", "run_vectorised", "infer_write_shape"]
