"""Weight prefetch across launches (``passes/prefetch.py``): which kernels get the extra lanes, what the change to a
kernel's source and launch is, and that the results do not change."""

from __future__ import annotations

import re

import pytest
import torch

from deplodock_amd import HipBackend, trace_module
from deplodock_amd import workloads as wl
from deplodock_amd.context import Context
from deplodock_amd.ir.hip import HipOp
from deplodock_amd.passes import prefetch


def kernels(compiled):
    return [compiled.nodes[n].op for n in compiled.topological_order() if isinstance(compiled.nodes[n].op, HipOp)]


def test_only_programs_beyond_the_last_level_cache_prefetch_by_default(launcher_lib, monkeypatch):
    """A two-layer model's weights fit the memory-side cache: nothing changes.  Forced on, every kernel whose successor
    streams a large constant gets the lanes, and off is off."""
    monkeypatch.delenv("EMMY_PREFETCH", raising=False)
    case = wl.qwen3_model_case(seq=32, layers=2)
    plain = kernels(HipBackend().compile(trace_module(case.module, case.inputs)))
    assert not any("PREFETCH" in k.knobs for k in plain)
    monkeypatch.setenv("EMMY_PREFETCH", "1")
    forced = kernels(HipBackend().compile(trace_module(case.module, case.inputs)))
    assert len(forced) == len(plain)
    forms = [k.knobs.get("PREFETCH") for k in forced]
    # embedding -> q/k/v weights; q/k/v projection -> head norms + rotary embedding -> attention (no weights); attention
    # -> o_proj; o_proj -> gate/up; gate/up -> down; down -> the next layer's q/k/v (the last one: the final norm, no
    # large constant)
    assert forms == ["workgroups", None, None, "workgroups", "workgroups", "wave", "workgroups", None, None, "workgroups", "workgroups", "wave", None, None]
    for before, after in zip(plain, forced):
        if "PREFETCH" not in after.knobs:
            assert after.kernel_name == before.kernel_name
            continue
        assert after.kernel_name.startswith(before.kernel_name + "_pf") and after.arg_order[:-1] == before.arg_order
        assert after.lds_bytes == before.lds_bytes
        if after.knobs["PREFETCH"] == "wave":
            assert after.grid == before.grid and after.block[0][0] == before.block[0][0] + 64
            assert f"if (threadIdx.x >= {before.block[0][0]}u) {{" in after.kernel_source
        else:
            assert after.block == before.block and after.grid[0][0] == before.grid[0][0] + Context().compute_units
            assert f"if (blockIdx.x >= {before.grid[0][0]}u) {{" in after.kernel_source
    monkeypatch.setenv("EMMY_PREFETCH", "0")
    assert not any("PREFETCH" in k.knobs for k in kernels(HipBackend().compile(trace_module(case.module, case.inputs))))


def test_prefetch_loads_share_one_register_that_is_waited_for(launcher_lib, monkeypatch):
    """The compiler knows nothing of when an ``asm`` load's data arrives and would hand its destination register to
    the next value computed (an address of the following iteration, overwritten in mid-use): every load of a
    prefetching wave therefore names one variable as input and output, and the wave waits on it before it ends."""
    monkeypatch.setenv("EMMY_PREFETCH", "1")
    case = wl.qwen3_model_case(seq=32, layers=1)
    for k in kernels(HipBackend().compile(trace_module(case.module, case.inputs))):
        if "PREFETCH" not in k.knobs:
            continue
        guard = k.kernel_source[k.kernel_source.index("emh_pf) {") :].split("    return;\n  }\n")[0]
        loads = re.findall(r'asm volatile\("global_load_dword %0, %1, off" : "([^"]+)"\(v_\)', guard)
        assert loads and set(loads) == {"+v"}, guard
        assert "unsigned v_ = 0u;" in guard and guard.rstrip().endswith('asm volatile("s_waitcnt vmcnt(0)" : "+v"(v_));')
        assert "gridDim" not in k.kernel_source and "blockDim" not in k.kernel_source


def test_a_consumer_whose_rows_to_workgroups_mapping_is_known_is_prefetched_per_xcd(launcher_lib, monkeypatch):
    """The few-row contraction says which rows of its weight workgroup j streams (``weight_slices``): the kernel before
    it deals the slices of each XCD's workgroups to its own lanes on that XCD, so the lines land in the L2 that will
    be asked for them."""
    monkeypatch.setenv("EMMY_PREFETCH", "1")
    case = wl.qwen3_model_case(seq=32, layers=1)
    ks = kernels(HipBackend().compile(trace_module(case.module, case.inputs)))
    gate_up = next(k for k in ks if "silu_mul" in k.kernel_name)
    assert gate_up.knobs["STAGE"].startswith("d4/ks") and gate_up.weight_slices[1] * gate_up.weight_slices[2] == 2 * 3072 * 1024 * 2
    before = ks[ks.index(gate_up) - 1]
    assert before.arg_order[-1] == gate_up.weight_slices[0]
    assert "const unsigned xcd_ = blockIdx.x % 8u" in before.kernel_source and "slices xcd_, xcd_ + 8" in before.kernel_source


def test_what_does_not_take_the_change_is_left_alone():
    ctx = Context()
    src = 'extern "C" __global__ __launch_bounds__(256) void k_x(const float* __restrict__ a, float* __restrict__ o) {\n  o[blockIdx.x * 256 + threadIdx.x] = a[0];\n}\n'
    base = dict(kernel_source=src, kernel_name="k_x", arg_order=("a", "o"), grid=((64,), (1,), (1,)), block=((256,), (1,), (1,)), lds_bytes=0)
    ok = prefetch.with_prefetch(HipOp(**base), "w", 1 << 20, None, ctx)
    assert ok is not None and ok.arg_order == ("a", "o", "w") and ok.grid[0] == (64 + ctx.compute_units,) and "k_x_pf" in ok.kernel_source
    assert prefetch.with_prefetch(HipOp(**{**base, "runtime_args": ("n",)}), "w", 1 << 20, None, ctx) is None  # launch sized at run time
    assert prefetch.with_prefetch(HipOp(**{**base, "grid": ((64,), (2,), (1,))}), "w", 1 << 20, None, ctx) is None  # not a 1-D launch
    assert prefetch.with_prefetch(HipOp(**{**base, "kernel_source": src.replace("blockIdx.x * 256", "blockIdx.x * blockDim.x")}), "w", 1 << 20, None, ctx) is None
    # many workgroups, or much LDS: one more wave per workgroup instead of more workgroups
    wave = prefetch.with_prefetch(HipOp(**{**base, "grid": ((256,), (1,), (1,))}), "w", 1 << 20, None, ctx)
    assert wave.knobs["PREFETCH"] == "wave" and wave.block[0] == (320,) and "__launch_bounds__(256 + 64)" in wave.kernel_source
    assert prefetch.with_prefetch(HipOp(**{**base, "grid": ((256,), (1,), (1,)), "block": ((1024,), (1,), (1,))}), "w", 1 << 20, None, ctx) is None


@pytest.mark.gpu
@pytest.mark.parametrize("seq", [32, 1])
def test_prefetching_kernels_compute_what_the_plain_ones_do(device, seq, monkeypatch):
    """Bit for bit: the extra lanes only read."""
    case = wl.qwen3_model_case(seq=seq, layers=3)
    outs = []
    for pin in ("0", "1"):
        monkeypatch.setenv("EMMY_PREFETCH", pin)
        be = HipBackend()
        compiled = be.compile(trace_module(case.module, case.inputs))
        assert any("PREFETCH" in k.knobs for k in kernels(compiled)) == (pin == "1")
        prog = be.program(compiled, {compiled.inputs[0]: case.inputs[0].to(device)})
        try:
            for _ in range(3):
                prog.run()
            torch.cuda.synchronize()
            outs.append(prog.output_tensors()[compiled.outputs[0]].clone())
        finally:
            prog.close()
    assert torch.equal(outs[0], outs[1])
