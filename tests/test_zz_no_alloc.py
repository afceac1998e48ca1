"""``emh_launch_scratch``: the launch entry point that allocates nothing, against ``emh_launch``.

A split contraction (``REDUCE=g<n>k`` / ``g<n>a``) needs device memory beyond its inputs and outputs: the
fp32 partial planes the partial kernel writes and the combine kernel folds.  Through ``emh_launch`` that
workspace is a tensor of the caller's; through ``emh_launch_scratch`` it is the library's own device array.
Both must give the same output — bit for bit for the fixed-order ``k`` arm, within the bf16 tolerance for the
atomic arm — on two calls in a row, the second with a smaller input (the array keeps the first call's contents)."""

from __future__ import annotations

import pytest
import torch

from deplodock_amd import HipBackend, trace_module
from deplodock_amd.backend.hip import launcher
from deplodock_amd.backend.hip.program import _LibraryScratch
from deplodock_amd.ir.hip import HipOp
from oracle import eager

pytestmark = pytest.mark.gpu


def _both_ways(case, device, reduce, monkeypatch):
    monkeypatch.setenv("EMMY_REDUCE", reduce)
    monkeypatch.setenv("EMMY_TILE", "a:mfma_16x16x32_bf16/w2x2/f1x2/k2")
    be = HipBackend()
    compiled = be.compile(trace_module(case.module, case.inputs))
    assert sum(isinstance(n.op, HipOp) for n in compiled.nodes.values()) == 2
    data = {compiled.inputs[0]: case.inputs[0].to(device)}
    outs = []
    for library_scratch in (False, True):
        prog = be.program(compiled, data, library_scratch=library_scratch)
        try:
            assert any(isinstance(t, _LibraryScratch) for t in prog.arrays.values()) == library_scratch
            prog.run()
            torch.cuda.synchronize()
            outs.append(prog.output_tensors()[compiled.outputs[0]].clone())
        finally:
            prog.close()
    return outs, eager.run_eager(case, device)


@pytest.mark.parametrize("reduce", ["g2k", "g4a"])
def test_library_scratch_launches_match_caller_workspace_launches(device, reduce, monkeypatch):
    big = eager.linear_case(m=128, k=1024, n=3072, seed=31)
    small = eager.linear_case(m=40, k=512, n=1000, seed=32)
    for case in (big, small):  # two calls in a row on the same array, the second smaller
        (plain, lent), want = _both_ways(case, device, reduce, monkeypatch)
        eager.assert_close(lent.reshape(want.shape), want, case.rtol, case.atol, f"{case.name} {reduce} through emh_launch_scratch vs eager")
        if reduce.endswith("k"):
            assert torch.equal(lent, plain), f"{case.name} {reduce}: library scratch and caller workspace differ"
        else:
            eager.assert_close(lent, plain.float(), 2 ** -7, 1e-3, f"{case.name} {reduce}: library scratch vs caller workspace")


def test_library_scratch_rejects_what_does_not_fit(device, launcher_lib, monkeypatch):
    """More workspace than the array holds is refused with a clear error, on the host and by the library."""
    monkeypatch.setenv("EMMY_REDUCE", "g4k")
    monkeypatch.setenv("EMMY_TILE", "a:mfma_16x16x32_bf16/w2x2/f1x2/k2")
    case = eager.linear_case(m=512, k=1024, n=3072, seed=33)  # 4 planes x 512 x 3072 x 4 B = 24 MiB
    be = HipBackend()
    compiled = be.compile(trace_module(case.module, case.inputs))
    with pytest.raises(ValueError, match="scratch array holds"):
        be.program(compiled, {compiled.inputs[0]: case.inputs[0].to(device)}, library_scratch=True)
    from deplodock_amd.backend.hip import hiprtc
    from deplodock_amd.backend.hip.launcher import PackedArgs

    k = hiprtc.load_function('extern "C" __global__ void k_fill_one(float* x) { x[threadIdx.x] = 1.0f; }', "k_fill_one")
    args = PackedArgs([0])
    with pytest.raises(launcher.LauncherError, match="does not fit"):
        launcher_lib.launch_scratch(k.fn, (1, 1, 1), (64, 1, 1), 0, None, args, 0, 0, launcher.EMH_SCRATCH_MAX_BYTES + 4, False)
    with pytest.raises(launcher.LauncherError, match="multiple of 256"):
        launcher_lib.launch_scratch(k.fn, (1, 1, 1), (64, 1, 1), 0, None, args, 0, 128, 256, False)
    with pytest.raises(launcher.LauncherError, match="not a parameter"):
        launcher_lib.launch_scratch(k.fn, (1, 1, 1), (64, 1, 1), 0, None, args, 1, 0, 256, False)
    launcher_lib.launch_scratch(k.fn, (1, 1, 1), (64, 1, 1), 0, None, args, 0, 0, 256, True)  # a good call still works after the refusals
    torch.cuda.synchronize()
    assert args.slots[0].value in (0, None)  # the caller's parameter storage is left alone
