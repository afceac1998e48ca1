"""The prescribed oracle: PyTorch eager on the same module and seeded inputs.

TEST INFRASTRUCTURE ONLY (see ``oracle/__init__.py``).  Runs a workload
(``deplodock_amd.workloads``: module + seeded inputs, re-exported here) through
PyTorch eager, compares within the stated tolerance, and times eager on the host
cores for the CPU baseline.
"""

from __future__ import annotations

import math
from dataclasses import dataclass

import torch
from torch import nn

from deplodock_amd.workloads import (  # noqa: F401  (the shapes are the product's; the checker re-exports them)
    BF16_RTOL,
    FP32_RTOL,
    Case,
    NormedRopeAttention,
    Qwen3Block,
    Sdpa,
    linear_case,
    normed_rope_attention_case,
    qwen3_block_case,
    rms_norm_case,
    sdpa_case,
    softmax_case,
)


def block_weights(case: Case) -> dict:
    """Parameter arrays of a :func:`qwen3_block_case` keyed the way ``emmy_ops.qwen3_block`` wants."""
    sd = {k: v.float().numpy() for k, v in case.module.state_dict().items()}
    pick = lambda frag: next(v for k, v in sd.items() if frag in k)  # noqa: E731
    return {
        "input_layernorm": pick("input_layernorm"), "post_attention_layernorm": pick("post_attention_layernorm"),
        "q_proj": pick("q_proj"), "k_proj": pick("k_proj"), "v_proj": pick("v_proj"), "o_proj": pick("o_proj"),
        "q_norm": pick("q_norm"), "k_norm": pick("k_norm"), "gate_proj": pick("gate_proj"), "up_proj": pick("up_proj"), "down_proj": pick("down_proj"),
    }  # fmt: skip


def run_eager(case: Case, device: str = "cpu") -> torch.Tensor:
    m = case.module.to(device)
    with torch.no_grad():
        out = m(*(t.to(device) for t in case.inputs))
    return out


def assert_close(actual: torch.Tensor, expected: torch.Tensor, rtol: float, atol: float, what: str = "") -> None:
    a, e = actual.detach().float().cpu(), expected.detach().float().cpu()
    if a.shape != e.shape:
        raise AssertionError(f"{what}: shape {tuple(a.shape)} != {tuple(e.shape)}")
    err = (a - e).abs()
    bound = atol + rtol * e.abs()
    bad = err > bound
    if bool(bad.any()) or not bool(torch.isfinite(a).all()):
        idx = int(torch.argmax(err - bound))
        raise AssertionError(
            f"{what}: {int(bad.sum())}/{a.numel()} elements outside atol={atol} rtol={rtol}; "
            f"worst |diff|={float(err.flatten()[idx]):.3e} at flat index {idx} (expected {float(e.flatten()[idx]):.6e}, got {float(a.flatten()[idx]):.6e})"
        )


def time_eager_cpu(case: Case, *, threads: int, warmup: int = 1, iters: int = 3) -> float:
    """Median seconds per forward of ``case`` on ``threads`` host cores."""
    import statistics
    import time

    old = torch.get_num_threads()
    torch.set_num_threads(threads)
    try:
        m = case.module.cpu()
        with torch.no_grad():
            for _ in range(warmup):
                m(*case.inputs)
            samples = []
            for _ in range(iters):
                t0 = time.perf_counter()
                m(*case.inputs)
                samples.append(time.perf_counter() - t0)
    finally:
        torch.set_num_threads(old)
    return statistics.median(samples)


__all__ = ["Case", "rms_norm_case", "softmax_case", "linear_case", "sdpa_case", "qwen3_block_case", "run_eager", "assert_close", "time_eager_cpu", "block_weights", "math"]
