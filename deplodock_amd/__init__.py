"""deplodock_amd — an MI355X (gfx950 / CDNA4) kernel backend for the emmy compiler's hot path.

The package turns scheduled kernels (row reductions, tiled contractions, fused
flash attention, pointwise maps) into HIP source written for wave64, MFMA and
LDS, compiles it with hipRTC and launches it through ``libemmy_hip.so`` (a
C-ABI library bound with ``ctypes``) on PyTorch-ROCm tensors.

Public surface (mirrors the reference's compiler API):

    from deplodock_amd import trace_module, HipBackend
    graph    = trace_module(module, example_inputs)
    backend  = HipBackend()
    compiled = backend.compile(graph)
    result, _ = backend.run(compiled, input_data={...})
"""

from deplodock_amd.backend import Backend, BenchmarkResult, LaunchTime, RunResult  # noqa: F401


def __getattr__(name):
    # Lazy: importing the package must not import torch or load the native library.
    if name == "HipBackend":
        from deplodock_amd.backend.hip.backend import HipBackend

        return HipBackend
    if name == "trace_module":
        from deplodock_amd.trace.torch import trace_module

        return trace_module
    raise AttributeError(name)


__version__ = "0.1.0"
