"""Tracer coverage of the ops the reference's tracer accepts (emmy/compiler/trace/torch.py:489-503, 526-800): which
frontend op each ATen call becomes, which kernels follow, and the host evaluation of the added element-wise functions
against PyTorch on the CPU."""

import numpy as np
import pytest
import torch
import torch.nn.functional as Fn
from torch import nn

from deplodock_amd import HipBackend, trace_module
from deplodock_amd.ir import expr as E
from deplodock_amd.ir import frontend as F
from deplodock_amd.ir.hip import HipOp
from deplodock_amd.trace.torch import TraceError


class _Fn(nn.Module):
    def __init__(self, fn):
        super().__init__()
        self.fn = fn

    def forward(self, *args):
        return self.fn(*args)


def _ops(mod, *args):
    g = trace_module(mod.eval(), args)
    return g, [type(n.op).__name__ + (f":{n.op.fn}" if isinstance(n.op, F.ElementwiseOp) else "") for n in g.nodes.values() if not type(n.op).__name__.startswith(("Input", "Constant"))]


def _kernels(g):
    return [n.op.kernel_name.rsplit("_", 1)[0] for n in HipBackend().compile(g).nodes.values() if isinstance(n.op, HipOp)]


X = torch.randn(4, 32, 64)


@pytest.mark.parametrize(
    "fn, args, ops, kernels",
    [
        (Fn.gelu, (X,), ["ElementwiseOp:gelu"], ["k_pointwise_elementwise"]),
        (lambda t: Fn.gelu(t, approximate="tanh"), (X,), ["ElementwiseOp:gelu_tanh"], ["k_pointwise_elementwise"]),
        (Fn.relu, (X,), ["ElementwiseOp:relu"], ["k_pointwise_elementwise"]),
        (torch.erf, (X,), ["ElementwiseOp:erf"], ["k_pointwise_elementwise"]),
        (lambda t: t.amax(-1), (X,), ["AmaxOp"], ["k_amax_reduce"]),
        (lambda t: t.sum(1), (X,), ["SumOp"], ["k_gather", "k_sum_reduce"]),  # the reduced axis is moved last by a copy
        (lambda t: torch.softmax(t, 1), (X,), ["SoftmaxOp"], ["k_gather", "k_softmax_reduce", "k_gather"]),  # ... and the result copied back into the traced order
        (lambda b, a, w: torch.addmm(b, a, w), (torch.randn(16), torch.randn(8, 32), torch.randn(32, 16)), ["MatmulOp", "ElementwiseOp:add"], ["k_gather", "k_matmul", "k_pointwise_elementwise"]),
        (lambda a, w: a @ w.t(), (torch.randn(8, 32), torch.randn(16, 32)), ["TransposeOp", "MatmulOp"], ["k_matmul"]),
        (lambda a, b: torch.cat([a, b], 1), (X, X), ["CatOp"], ["k_cat"]),
        (lambda t, i: t.index_select(2, i), (X, torch.tensor([3, 1])), ["GatherOp"], ["k_index_rows"]),
    ],
)
def test_aten_calls_become_frontend_ops_and_kernels(launcher_lib, fn, args, ops, kernels):
    g, got = _ops(_Fn(fn), *args)
    assert got == ops
    assert _kernels(g) == kernels


def test_modules():
    g, got = _ops(nn.LayerNorm(64), X)
    assert got == ["LayerNormOp"] and [n.op for n in g.nodes.values() if isinstance(n.op, F.LayerNormOp)][0] == F.LayerNormOp(eps=1e-5, has_weight=True, has_bias=True)
    assert _kernels(g) == ["k_layer_norm_reduce"]
    g, got = _ops(nn.LayerNorm(64, elementwise_affine=False), X)
    assert [n.op for n in g.nodes.values() if isinstance(n.op, F.LayerNormOp)][0] == F.LayerNormOp(eps=1e-5)
    g, got = _ops(nn.Embedding(50, 16), torch.randint(0, 50, (3, 7)))
    assert got == ["GatherOp"] and _kernels(g) == ["k_index_rows"]


def test_what_stays_refused():
    with pytest.raises(TraceError, match="last axis"):
        trace_module(nn.LayerNorm((32, 64)).eval(), (X,))
    with pytest.raises(TraceError, match="multi-axis"):
        trace_module(_Fn(lambda t: t.amax((1, 2))).eval(), (X,))
    with pytest.raises(TraceError, match="unsupported ATen op"):
        trace_module(_Fn(lambda t, i: torch.gather(t, 1, i)).eval(), (X, torch.zeros(4, 2, 64, dtype=torch.int64)))


@pytest.mark.parametrize("op, ref", [("relu", torch.relu), ("erf", torch.erf), ("gelu", Fn.gelu), ("gelu_tanh", lambda t: Fn.gelu(t, approximate="tanh"))])
def test_host_evaluation_of_the_added_functions(op, ref):
    x = np.linspace(-6, 6, 4001, dtype=np.float32)
    got = E.evaluate(E.Un(op, E.Var("x")), {"x": x})
    np.testing.assert_allclose(got, ref(torch.from_numpy(x)).numpy(), rtol=2e-6, atol=2e-6)  # (1 + erf cancels for x << 0: absolute, not relative, agreement there)
    text = E.render(E.Un(op, E.Var("x")), {"x": "v"})
    assert "v" in text and text.count("(") == text.count(")")


def test_pow_forms():
    x = np.linspace(0.1, 3, 50, dtype=np.float32)
    np.testing.assert_allclose(E.evaluate(E.Bin("pow", E.Var("x"), E.Const(2.5)), {"x": x}), x**2.5, rtol=1e-6)
    assert "powf" in E.render(E.Bin("pow", E.Var("x"), E.Const(2.5)), {"x": "v"})
    g, _ = _ops(_Fn(lambda t: t.pow(3)), X)
    (k,) = [n.op for n in HipBackend().compile(g).nodes.values() if isinstance(n.op, HipOp)]
    assert "powf" not in k.kernel_source  # a small whole power is a product
