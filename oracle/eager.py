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
    MaskedQwen3Block,
    MaskedSdpa,
    causal_bias,
    masked_qwen3_block_case,
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


def run_eager_fp32(case: Case, device: str = "cpu") -> torch.Tensor:
    """Eager on an fp32 copy of the module (its parameters upcast as they are) and upcast inputs:
    the value the 16-bit runs approximate."""
    import copy

    m = copy.deepcopy(case.module).float().to(device)
    with torch.no_grad():
        return m(*(t.to(device).float() if t.is_floating_point() else t.to(device) for t in case.inputs))


def row_rel_l2(actual: torch.Tensor, exact: torch.Tensor) -> torch.Tensor:
    """Per row (last axis) ``|actual - exact|_2 / |exact|_2`` in float64: an error measure that scales
    with the row it is taken on, unlike an absolute floor."""
    a, e = actual.detach().double().cpu(), exact.detach().double().cpu()
    if a.shape != e.shape:
        raise AssertionError(f"shape {tuple(a.shape)} != {tuple(e.shape)}")
    return (a - e).norm(dim=-1) / e.norm(dim=-1).clamp_min(1e-30)


def assert_rows_within_baseline(actual: torch.Tensor, baseline: torch.Tensor, exact: torch.Tensor, factor: float = 1.5, what: str = "") -> None:
    """Scale-aware parity: every row of ``actual`` must be as close to ``exact`` (an fp32 run), in
    relative L2, as ``factor`` times the worst row of ``baseline`` (16-bit eager on the same
    inputs), and the rows' mean error within ``factor`` times the baseline's mean.  A result that
    drops or misplaces part of a row's terms moves that row by far more than rounding does."""
    ra, rb = row_rel_l2(actual, exact), row_rel_l2(baseline, exact)
    if not bool(torch.isfinite(actual.detach().float()).all()):
        raise AssertionError(f"{what}: non-finite values")
    worst, mean = float(ra.max()), float(ra.mean())
    lim_worst, lim_mean = factor * float(rb.max()), factor * float(rb.mean())
    if worst > lim_worst or mean > lim_mean:
        idx = int(torch.argmax(ra))
        raise AssertionError(
            f"{what}: row-relative L2 error vs the fp32 run: worst row {worst:.3e} (flat row {idx}; allowed {lim_worst:.3e} = {factor} x the 16-bit eager run's worst), "
            f"mean {mean:.3e} (allowed {lim_mean:.3e}); {int((ra > lim_worst).sum())}/{ra.numel()} rows over"
        )


def assert_mean_error_within_baseline(actual: torch.Tensor, baseline: torch.Tensor, exact: torch.Tensor, factor: float = 1.5, what: str = "") -> None:
    """``mean|actual - exact| <= factor * mean|baseline - exact|``: the result may not be further
    from the fp32 run, on average, than ``factor`` times what 16-bit eager is."""
    a, b, e = (t.detach().double().cpu() for t in (actual, baseline, exact))
    ours, theirs = float((a - e).abs().mean()), float((b - e).abs().mean())
    if not ours <= factor * theirs:
        raise AssertionError(f"{what}: mean |ours - fp32| = {ours:.3e} exceeds {factor} x mean |16-bit eager - fp32| = {theirs:.3e}")


def position_coded_values(like: torch.Tensor) -> torch.Tensor:
    """``V[..., j, :] = j / S``: attention over it returns each query's weighted mean key position,
    so a key block that is skipped, taken twice or taken from the wrong place shifts the row."""
    s = like.shape[-2]
    pos = (torch.arange(s, dtype=torch.float32) / s).to(like.dtype)
    return pos[:, None].expand(like.shape).contiguous()


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


__all__ = ["Case", "rms_norm_case", "softmax_case", "linear_case", "sdpa_case", "qwen3_block_case", "run_eager", "run_eager_fp32", "assert_close", "row_rel_l2", "assert_rows_within_baseline",
           "assert_mean_error_within_baseline", "position_coded_values", "time_eager_cpu", "block_weights", "math"]  # fmt: skip
