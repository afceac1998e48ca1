"""Scalar expression trees used inside kernel bodies (projections, epilogues).

A small counterpart of the reference's elementwise vocabulary
(emmy/compiler/ir/elementwise.py:36-78, intrinsic spellings
emmy/compiler/ir/kernel/render.py:374-384).  An expression renders to HIP C
(``render``) and evaluates on numpy arrays (``evaluate``) so kernel bodies can
be checked on the host without a GPU.

All arithmetic is fp32.  ``Round(bf16)`` marks a point where the value is
rounded to a storage type and widened again — this is how a fused kernel
reproduces the rounding points of an eager bf16 module.
"""

from __future__ import annotations

import math

from dataclasses import dataclass

import numpy as np

from deplodock_amd.dtype import bf16_bits_from_f32, f32_from_bf16_bits


class Expr:
    def __add__(self, o):
        return Bin("add", self, wrap(o))

    def __radd__(self, o):
        return Bin("add", wrap(o), self)

    def __sub__(self, o):
        return Bin("sub", self, wrap(o))

    def __rsub__(self, o):
        return Bin("sub", wrap(o), self)

    def __mul__(self, o):
        return Bin("mul", self, wrap(o))

    def __rmul__(self, o):
        return Bin("mul", wrap(o), self)

    def __truediv__(self, o):
        return Bin("div", self, wrap(o))

    def __neg__(self):
        return Un("neg", self)


@dataclass(frozen=True, eq=False)
class Var(Expr):
    name: str


@dataclass(frozen=True, eq=False)
class Const(Expr):
    value: float


@dataclass(frozen=True, eq=False)
class Un(Expr):
    op: str  # neg | exp | rsqrt | sqrt | rcp | sigmoid | silu | abs | tanh | relu | erf | gelu | gelu_tanh
    a: Expr


@dataclass(frozen=True, eq=False)
class Bin(Expr):
    op: str  # add | sub | mul | div | max | min | pow
    a: Expr
    b: Expr


@dataclass(frozen=True, eq=False)
class Round(Expr):
    """Round to ``dtype`` storage precision ("bf16" | "f16") and widen back to fp32."""

    dtype: str
    a: Expr


def wrap(v) -> Expr:
    if isinstance(v, Expr):
        return v
    return Const(float(v))


def float_literal(v: float) -> str:
    """An fp32 literal that round-trips exactly (hex float)."""
    f = float(np.float32(v))
    if f != f:
        return "__builtin_nanf(\"\")"
    if f in (float("inf"), float("-inf")):
        return "__builtin_inff()" if f > 0 else "(-__builtin_inff())"
    return f"{f.hex()}f"


# Unary / binary ops as (template over {a}, {b}) built from the render target's intrinsic spellings:
# this module decides the *shape* of an expression (what is a call, what an operator, where the
# reference's SiLU decomposition x * 1/(1+e^-x) sits — emmy/compiler/pipeline/passes/frontend/
# decomposition/020_silu.py), the target decides the names.
def _call(op: str, *args: str) -> str:
    from deplodock_amd.render_target import rt

    return f"{rt.intrinsic(op, 'f32')}({', '.join(args)})"


def _un_c(op: str, a: str, rounded: bool = False) -> str:
    """fp32 text of unary ``op`` on ``a``.  ``rounded``: the result goes to a 16-bit type straight away,
    so transcendentals take the hardware approximations (v_exp_f32 / v_rcp_f32, a couple of fp32 ulps):
    nothing of the difference survives the rounding, and the precise forms cost ~25 instructions each."""
    exp = (lambda x: _call("fast_exp", x)) if rounded else (lambda x: _call("exp", x))
    div = (lambda x, y: _call("fast_div", x, y)) if rounded else (lambda x, y: f"(({x}) / ({y}))")
    if op == "neg":
        return f"(-({a}))"
    if op == "exp":
        return exp(a)
    if op == "rcp":
        return f"(1.0f / ({a}))"
    if op == "sigmoid":
        return div("1.0f", f"1.0f + {exp(f'-({a})')}") if rounded else f"(1.0f / (1.0f + {exp(f'-({a})')}))"
    if op == "silu":
        return div(f"({a})", f"1.0f + {exp(f'-({a})')}") if rounded else f"(({a}) / (1.0f + {exp(f'-({a})')}))"
    if op in ("exp2", "fast_exp2", "rsqrt", "sqrt", "abs", "tanh", "erf"):
        return _call(op, a)
    if op == "relu":
        return _call("max", a, "0.0f")
    if op == "gelu":  # 0.5 x (1 + erf(x / sqrt 2)): emmy/compiler/pipeline/passes/frontend/decomposition/160_gelu.py
        return f"(0.5f * ({a}) * (1.0f + {_call('erf', f'({a}) * {float_literal(1.0 / math.sqrt(2.0))}')}))"
    if op == "gelu_tanh":  # 0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3))): decomposition/170_gelu_tanh.py
        inner = f"{float_literal(math.sqrt(2.0 / math.pi))} * (({a}) + {float_literal(0.044715)} * ({a}) * ({a}) * ({a}))"
        return f"(0.5f * ({a}) * (1.0f + {_call('tanh', inner)}))"
    raise KeyError(f"no rendering for unary op {op!r}")


_ROUNDED_UN = ("exp", "sigmoid", "silu")
_BIN_SYM = {"add": "+", "sub": "-", "mul": "*", "div": "/"}


def _bin_c(op: str, a: str, b: str) -> str:
    if op in _BIN_SYM:
        return f"(({a}) {_BIN_SYM[op]} ({b}))"
    if op in ("max", "min", "pow"):
        return _call(op, a, b)
    raise KeyError(f"no rendering for binary op {op!r}")


def _round_c(dtype: str, a: str) -> str:
    from deplodock_amd.render_target import rt

    return rt.convert(rt.convert(a, "f32", dtype), dtype, "f32")


def render(e: Expr, env: dict[str, str]) -> str:
    """HIP C text of ``e``; ``env`` maps variable names to C expressions."""
    if isinstance(e, Var):
        return env[e.name]
    if isinstance(e, Const):
        return float_literal(e.value)
    if isinstance(e, Un):
        return _un_c(e.op, render(e.a, env))
    if isinstance(e, Bin):
        return _bin_c(e.op, render(e.a, env), render(e.b, env))
    if isinstance(e, Round):
        if isinstance(e.a, Un) and e.a.op in _ROUNDED_UN:
            return _round_c(e.dtype, _un_c(e.a.op, render(e.a.a, env), rounded=True))
        return _round_c(e.dtype, render(e.a, env))
    raise TypeError(f"cannot render {type(e).__name__}")


def _erf(a: np.ndarray) -> np.ndarray:
    return np.vectorize(math.erf, otypes=[np.float32])(np.asarray(a, dtype=np.float64)).astype(np.float32).reshape(np.shape(a))


def evaluate(e: Expr, env: dict[str, np.ndarray]) -> np.ndarray:
    """Numpy fp32 evaluation with the same rounding points as the device code."""
    f32 = np.float32
    if isinstance(e, Var):
        return np.asarray(env[e.name], dtype=f32)
    if isinstance(e, Const):
        return f32(e.value)
    if isinstance(e, Round):
        a = np.asarray(evaluate(e.a, env), dtype=f32)
        if e.dtype == "bf16":
            return f32_from_bf16_bits(bf16_bits_from_f32(a)).reshape(a.shape)
        return a.astype(np.float16).astype(f32)
    if isinstance(e, Un):
        a = np.asarray(evaluate(e.a, env), dtype=f32)
        with np.errstate(over="ignore", divide="ignore", invalid="ignore"):
            return {
                "neg": lambda: -a,
                "exp": lambda: np.exp(a),
                "exp2": lambda: np.exp2(a),
                "fast_exp2": lambda: np.exp2(a),
                "rsqrt": lambda: (f32(1) / np.sqrt(a)).astype(f32),
                "sqrt": lambda: np.sqrt(a),
                "rcp": lambda: (f32(1) / a).astype(f32),
                "abs": lambda: np.abs(a),
                "tanh": lambda: np.tanh(a),
                "sigmoid": lambda: (f32(1) / (f32(1) + np.exp(-a))).astype(f32),
                "silu": lambda: (a / (f32(1) + np.exp(-a))).astype(f32),
                "relu": lambda: np.maximum(a, f32(0)),
                "erf": lambda: _erf(a),
                "gelu": lambda: (f32(0.5) * a * (f32(1) + _erf(a * f32(1.0 / math.sqrt(2.0))))).astype(f32),
                "gelu_tanh": lambda: (f32(0.5) * a * (f32(1) + np.tanh(f32(math.sqrt(2.0 / math.pi)) * (a + f32(0.044715) * a * a * a)))).astype(f32),
            }[e.op]().astype(f32)
    if isinstance(e, Bin):
        a = np.asarray(evaluate(e.a, env), dtype=f32)
        b = np.asarray(evaluate(e.b, env), dtype=f32)
        with np.errstate(over="ignore", divide="ignore", invalid="ignore"):
            return {
                "add": lambda: a + b,
                "sub": lambda: a - b,
                "mul": lambda: a * b,
                "div": lambda: a / b,
                "max": lambda: np.maximum(a, b),
                "min": lambda: np.minimum(a, b),
                "pow": lambda: np.power(a, b),
            }[e.op]().astype(f32)
    raise TypeError(f"cannot evaluate {type(e).__name__}")


def variables(e: Expr) -> set[str]:
    if isinstance(e, Var):
        return {e.name}
    if isinstance(e, Const):
        return set()
    if isinstance(e, (Un, Round)):
        return variables(e.a)
    if isinstance(e, Bin):
        return variables(e.a) | variables(e.b)
    raise TypeError(type(e).__name__)


def substitute(e: Expr, table: dict[str, Expr]) -> Expr:
    """``e`` with every variable named in ``table`` replaced by its entry (other variables stay)."""
    if isinstance(e, Var):
        return table.get(e.name, e)
    if isinstance(e, Const):
        return e
    if isinstance(e, Un):
        return Un(e.op, substitute(e.a, table))
    if isinstance(e, Round):
        return Round(e.dtype, substitute(e.a, table))
    if isinstance(e, Bin):
        return Bin(e.op, substitute(e.a, table), substitute(e.b, table))
    raise TypeError(type(e).__name__)


def pretty(e: Expr) -> str:
    if isinstance(e, Var):
        return e.name
    if isinstance(e, Const):
        return repr(float(np.float32(e.value)))
    if isinstance(e, Un):
        return f"{e.op}({pretty(e.a)})"
    if isinstance(e, Round):
        return f"{e.dtype}({pretty(e.a)})"
    if isinstance(e, Bin):
        sym = {"add": "+", "sub": "-", "mul": "*", "div": "/"}.get(e.op)
        if sym:
            return f"({pretty(e.a)} {sym} {pretty(e.b)})"
        return f"{e.op}({pretty(e.a)}, {pretty(e.b)})"
    raise TypeError(type(e).__name__)
