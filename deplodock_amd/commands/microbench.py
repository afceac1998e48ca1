"""``microbench``: the two hardware figures the schedules are argued from.

* sustained MFMA rate (back-to-back ``mfma_f32_32x32x16_bf16``, one wave per SIMD);
* MFMA / VALU co-issue: cycles for one MFMA followed by K independent vector
  instructions (``v_fma_f32`` or ``v_exp_f32``), for one and two waves per SIMD —
  how much softmax arithmetic hides behind the matrix pipe.

No counterpart in the reference (its constants are NVIDIA's); the kernels are
emitted, compiled and launched through the same hipRTC / launcher path as
everything else.
"""

from __future__ import annotations

import sys


def _kernel_source(name: str, k: int, kind: str, threads: int, mfma: bool) -> str:
    from deplodock_amd.emit import prelude

    valu = "\n".join(
        f"      x{i % 8} = __builtin_fmaf(x{i % 8}, 1.0001f, 0.5f);" if kind == "fma" else f"      x{i % 8} = __builtin_amdgcn_exp2f(x{i % 8});" for i in range(k)
    )
    m0 = "acc0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc0, 0, 0, 0);" if mfma else ""
    m1 = "acc1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc1, 0, 0, 0);" if mfma else ""
    return (
        prelude.header()
        + f"""
extern "C" __global__ __launch_bounds__({threads}) void {name}(float* out, int iters) {{
  f32x16 acc0, acc1;
  for (int r = 0; r < 16; ++r) {{ acc0[r] = 0.f; acc1[r] = 0.f; }}
  bf16x8 a, b;
  for (int r = 0; r < 8; ++r) {{ a[r] = (__bf16)(threadIdx.x * 0.001f); b[r] = (__bf16)1.0f; }}
  float x0 = threadIdx.x * 1e-3f, x1 = x0 + 1, x2 = x0 + 2, x3 = x0 + 3, x4 = x0 + 4, x5 = x0 + 5, x6 = x0 + 6, x7 = x0 + 7;
  for (int it = 0; it < iters; ++it) {{
    #pragma unroll
    for (int u = 0; u < 4; ++u) {{
      {m0}
{valu}
      {m1}
{valu}
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); __builtin_amdgcn_sched_group_barrier(0x402, {k}, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); __builtin_amdgcn_sched_group_barrier(0x402, {k}, 0);
    }}
  }}
  float s = x0 + x1 + x2 + x3 + x4 + x5 + x6 + x7;
  for (int r = 0; r < 16; ++r) s += acc0[r] + acc1[r];
  out[blockIdx.x * blockDim.x + threadIdx.x] = s;
}}
"""
    )


def coissue_seconds(k: int, kind: str, waves_per_simd: int, mfma: bool = True, iters: int = 2000) -> float:
    """Seconds per (MFMA + ``k`` vector instructions) group per wave slot."""
    import torch

    from deplodock_amd.backend.hip import hiprtc, launcher
    from deplodock_amd.backend.hip.launcher import PackedArgs

    lib = launcher.load()
    threads = 256 * waves_per_simd
    name = f"k_coissue_{k}_{kind}_{waves_per_simd}_{int(mfma)}"
    fn = hiprtc.load_function(_kernel_source(name, k, kind, threads, mfma), name)
    cus = lib.device_props(0)["compute_units"]
    out = torch.zeros(cus * threads, device="cuda")
    args = PackedArgs([out.data_ptr()], [iters])
    e0, e1 = lib.event_create(), lib.event_create()
    lib.launch(fn.fn, (cus, 1, 1), (threads, 1, 1), 0, None, args)
    torch.cuda.synchronize()
    lib.event_record(e0, None)
    lib.launch(fn.fn, (cus, 1, 1), (threads, 1, 1), 0, None, args)
    lib.event_record(e1, None)
    torch.cuda.synchronize()
    ms = lib.event_elapsed_ms(e0, e1)
    lib.event_destroy(e0)
    lib.event_destroy(e1)
    return ms * 1e-3 / (iters * 8) / waves_per_simd


def register_microbench_command(subparsers) -> None:
    p = subparsers.add_parser("microbench", help="Measure the MFMA rate and MFMA/VALU co-issue of the GPU")
    p.set_defaults(func=handle_microbench)


def handle_microbench(args) -> None:
    import torch

    if not torch.cuda.is_available():
        print("error: no HIP device visible", file=sys.stderr)
        sys.exit(1)
    from deplodock_amd.backend.hip import launcher
    from deplodock_amd.commands.table import render_table

    cus = launcher.load().device_props(0)["compute_units"]
    base = coissue_seconds(0, "fma", 1)
    tflops = cus * 4 * 32 * 32 * 16 * 2 / base / 1e12
    clk = 32.0 / base  # a 32x32x16 bf16 MFMA occupies its SIMD's matrix pipe for 8 passes of 4 cycles
    print(f"MFMA 32x32x16 bf16, one wave per SIMD on {cus} CUs: {tflops:.0f} TFLOP/s sustained ({base * 1e9:.2f} ns per MFMA; {clk / 1e9:.2f} GHz if that is 32 cycles)")
    rows = []
    for wps in (1, 2):
        for kind in ("fma", "exp"):
            for k in (2, 4, 8, 12, 16):
                both = coissue_seconds(k, kind, wps) * clk
                alone = coissue_seconds(k, kind, wps, mfma=False) * clk
                rows.append([str(wps), f"v_{kind}_f32", str(k), f"{both:.1f}", f"{alone:.1f}", f"{32.0 / both:.2f}"])
    print()
    for line in render_table(["waves/SIMD", "VALU op", "K per MFMA", "cycles MFMA+K", "cycles K alone", "MFMA pipe busy"], rows, "llrrrr"):
        print(line)
