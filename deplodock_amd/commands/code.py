"""Inline ``--code`` expressions → a traceable module plus its example inputs.

Grammar (the one ``emmy compile --code`` / ``emmy run --code`` accept,
emmy/commands/trace.py:114-223): zero or more statements followed by one
expression.  ``torch``, ``nn`` and ``F`` are in scope.  When the expression is
a call of an ``nn.Module`` instance the module is traced as is, so its
parameters become graph constants; otherwise every tensor the expression names
(or builds inline with a ``torch.*`` constructor) becomes a graph input.
"""

from __future__ import annotations

import ast
import re
from dataclasses import dataclass, field

_TENSOR_MAKERS = frozenset({"randn", "rand", "zeros", "ones", "full", "arange", "empty", "randint", "tensor", "linspace", "randn_like", "rand_like", "zeros_like", "ones_like"})


class CodeError(ValueError):
    """The ``--code`` text is not a usable expression."""


@dataclass
class InlineProgram:
    module: object
    args: tuple
    kwargs: dict = field(default_factory=dict)
    slug: str = "code"
    input_names: tuple[str, ...] = ()


def slugify(text: str, limit: int = 48) -> str:
    s = re.sub(r"[^0-9a-zA-Z]+", "-", text).strip("-").lower()
    return (s[:limit].rstrip("-")) or "code"


def _eval(node: ast.expr, scope: dict):
    return eval(compile(ast.Expression(node), "<--code>", "eval"), scope)  # noqa: S307 - local CLI, user's own text


class _LiftTensors(ast.NodeTransformer):
    """Replace inline ``torch.<maker>(...)`` calls and bare tensor names with
    parameters of a generated ``forward``."""

    def __init__(self, scope: dict):
        import torch

        self.scope = scope
        self.torch = torch
        self.params: dict[str, object] = {}
        self._anon = 0

    def visit_Call(self, node: ast.Call):
        f = node.func
        if isinstance(f, ast.Attribute) and isinstance(f.value, ast.Name) and f.value.id == "torch" and f.attr in _TENSOR_MAKERS:
            value = _eval(node, self.scope)
            if isinstance(value, self.torch.Tensor):
                name = f"_x{self._anon}"
                self._anon += 1
                self.params[name] = value
                return ast.copy_location(ast.Name(id=name, ctx=ast.Load()), node)
        return self.generic_visit(node)

    def visit_Name(self, node: ast.Name):
        if isinstance(node.ctx, ast.Load) and isinstance(self.scope.get(node.id), self.torch.Tensor):
            self.params.setdefault(node.id, self.scope[node.id])
        return node


def parse_inline(code: str) -> InlineProgram:
    import torch
    import torch.nn.functional as F

    try:
        tree = ast.parse(code, mode="exec")
    except SyntaxError as e:
        raise CodeError(f"--code failed to parse: {e}") from e
    if not tree.body or not isinstance(tree.body[-1], ast.Expr):
        raise CodeError('--code must end with an expression (e.g. "torch.exp(torch.neg(x))")')
    final = tree.body[-1].value
    scope: dict = {"torch": torch, "nn": torch.nn, "F": F}
    exec(compile(ast.Module(body=tree.body[:-1], type_ignores=[]), "<--code>", "exec"), scope)  # noqa: S102 - local CLI

    if isinstance(final, ast.Call):
        try:
            callee = _eval(final.func, scope)
        except Exception:  # noqa: BLE001 - anything here just means "not a module call"
            callee = None
        if isinstance(callee, torch.nn.Module):
            args = tuple(_eval(a, scope) for a in final.args)
            kwargs = {k.arg: _eval(k.value, scope) for k in final.keywords if k.arg}
            return InlineProgram(callee, args, kwargs, slugify(ast.unparse(final.func)), tuple(f"arg{i}" for i in range(len(args))))

    lift = _LiftTensors(scope)
    body = ast.fix_missing_locations(lift.visit(final))
    if not lift.params:
        raise CodeError("--code expression has no tensor inputs to trace")
    anon = [k for k in lift.params if k.startswith("_x")]
    rename = {anon[0]: "x"} if len(anon) == 1 and "x" not in lift.params else {old: f"x{i}" for i, old in enumerate(anon)}
    params = {rename.get(k, k): v for k, v in lift.params.items()}
    for n in ast.walk(body):
        if isinstance(n, ast.Name) and n.id in rename:
            n.id = rename[n.id]
    src = f"class _Inline(torch.nn.Module):\n    def forward(self, {', '.join(params)}):\n        return {ast.unparse(body)}\n"
    exec(src, scope)  # noqa: S102 - local CLI
    return InlineProgram(scope["_Inline"](), tuple(params.values()), {}, slugify(ast.unparse(final)), tuple(params))
