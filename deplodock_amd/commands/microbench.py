"""``microbench``: the hardware figures the schedules are argued from.

* sustained MFMA rate (back-to-back ``mfma_f32_32x32x16_bf16``, one wave per SIMD);
* MFMA / VALU co-issue: cycles for one MFMA followed by K independent vector
  instructions (``v_fma_f32`` or ``v_exp_f32``), for one and two waves per SIMD —
  how much softmax arithmetic hides behind the matrix pipe;
* ``--l1fill``: the rate at which a compute unit can pull operand bytes in through
  its vector L1 with nothing else going on — load-only kernels (plain
  ``global_load_dwordx4`` into registers, and ``global_load_lds_dwordx4`` straight
  into LDS) swept over waves per CU, loads in flight per wave, the address pattern
  (contiguous 1 KiB per wave, or eight 128-byte pieces of rows a fixed stride apart,
  which is what a GEMM slab fetch looks like) and L2-resident against streamed
  operands.  That figure, not the MFMA peak, bounds a contraction whose tile needs
  more bytes per MFMA cycle than it delivers.

* ``--flash``: where the software-pipelined attention kernels (``FLASH=.../ws``, ``.../sp``) spend their clocks on the
  benchmark shape: per-iteration and per-pass phase stamps of wave 0 of workgroup 0 (``-DEMH_STAMP=1|2``, read with
  the shader clock), and timings with one part of the kernel taken out (``-DEMH_ABLATE``: no requests inside the loop,
  no consumer arithmetic, no exponentials, no fragment reads), next to the default kernel's time in the same process.

* ``--lds``: the rate at which the waves of a CU read 16-byte MFMA operand fragments out of
  LDS (``ds_read_b128``), for the lane-to-address patterns the emitters use — 16- and 32-row
  fragment layouts over XOR-swizzled slabs of 64, 128 and 256 bytes a row — against a
  conflict-free linear pattern, in bytes per clock per CU measured with the shader clock.

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


_L1FILL_SRC = r"""
#define UNIT 1024  /* bytes one wave-level 16-byte-per-lane load moves */
// Offsets stay 32-bit and every divisor is a power of two: the address arithmetic must not be
// what the kernel measures.
EMH_DEV unsigned emh_unit_offset(unsigned u, int lane) {
  if (STRIDE == 0) return u * UNIT + lane * 16;  // contiguous: one wave reads 1 KiB in a run
  // rows: a unit is the 128-byte piece kt of 8 consecutive rows; as in a GEMM slab fetch a
  // workgroup walks all its ROWBLOCKS row blocks at one kt before it moves to the next piece
  const unsigned rb = u % ROWBLOCKS, kt = (u / ROWBLOCKS) % KT, lap = u / (ROWBLOCKS * KT);
  return ((lap * ROWBLOCKS + rb) * 8 + lane / 8) * (unsigned)STRIDE + kt * 128 + (lane % 8) * 16;
}
extern "C" __global__ __launch_bounds__(NT) void KNAME(const unsigned char* __restrict__ src, unsigned* __restrict__ out,
                                                      int units_per_wave, int wg_units, int wg_kib, int share) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  // Workgroup ids rotate over the XCDs.  `share` workgroups of one XCD walk the same bytes
  // (an L2-resident operand block shared by the tiles of a row, as in a GEMM); with share = 0
  // every workgroup has bytes of its own.
  const int xcd = blockIdx.x % XCDS, slot = blockIdx.x / XCDS;
  const long base = (share ? (long)(xcd * share + slot % share) : (long)blockIdx.x) * wg_kib * 1024L;
  const unsigned char* p = src + base;
  u32x4 acc = {0u, 0u, 0u, 0u};
  // wave w takes units w, w + waves, ...; workgroups sharing bytes start at different units
  #define EMH_UNIT(i) emh_unit_offset(((unsigned)(i) * (NT / 64) + wave + slot * 7) & (unsigned)(wg_units - 1), lane)  /* wg_units is a power of two */
#if TO_LDS
  unsigned char* dst = lds + wave * (INFLIGHT * UNIT);
  #pragma unroll
  for (int i = 0; i < INFLIGHT; ++i) emh_dma16(p + EMH_UNIT(i), dst + i * UNIT);
  for (int it = INFLIGHT; it < units_per_wave; it += INFLIGHT) {
    #pragma unroll
    for (int i = 0; i < INFLIGHT; ++i) {
      __builtin_amdgcn_s_waitcnt(EMH_WAIT_VM(INFLIGHT - 1));  // the oldest load has landed: its slot is free again
      emh_dma16(p + EMH_UNIT(it + i), dst + i * UNIT);
    }
  }
  __builtin_amdgcn_s_waitcnt(EMH_WAIT_VM(0));
  emh_lds_publish(lds + tid * 4);
  acc[0] = *(const unsigned*)(dst + lane * 4);
#else
  u32x4 r[INFLIGHT];
  #pragma unroll
  for (int i = 0; i < INFLIGHT; ++i) r[i] = EMH_LD((const u32x4*)(p + EMH_UNIT(i)));
  for (int it = INFLIGHT; it < units_per_wave; it += INFLIGHT) {
    #pragma unroll
    for (int i = 0; i < INFLIGHT; ++i) {
      acc ^= r[i];
      r[i] = EMH_LD((const u32x4*)(p + EMH_UNIT(it + i)));
    }
  }
  #pragma unroll
  for (int i = 0; i < INFLIGHT; ++i) acc ^= r[i];
#endif
  if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x9e3779b9u) { out[blockIdx.x * NT + tid] = acc[0]; lds[tid] = 1; }  // keeps the loads (and the LDS that bounds occupancy) alive
}
"""

_WAIT_VM = "#define EMH_WAIT_VM(n) ((((n) & 0xF) | ((((n) >> 4) & 0x3) << 14)) | 0x3F70)  /* vmcnt <= n, other counters left alone */\n"


def l1fill_source(name: str, *, waves: int, inflight: int, stride: int, to_lds: bool, nontemporal: bool, row_blocks: int = 32, kt: int = 16, xcds: int = 8) -> str:
    """Source of one load-only kernel.  ``stride`` = 0 reads contiguous 1 KiB runs; otherwise a wave
    reads 128-byte pieces of 8 rows ``stride`` bytes apart."""
    from deplodock_amd.emit import prelude

    defs = {"KNAME": name, "NT": waves * 64, "INFLIGHT": inflight, "STRIDE": stride, "TO_LDS": int(to_lds), "ROWBLOCKS": row_blocks, "KT": kt, "XCDS": xcds,
            "EMH_LD(p)": "__builtin_nontemporal_load(p)" if nontemporal else "(*(p))"}  # fmt: skip
    return prelude.header(prelude.DMA) + _WAIT_VM + "".join(f"#define {k} {v}\n" for k, v in defs.items()) + _L1FILL_SRC


def l1fill_bytes_per_second(*, waves: int, inflight: int, stride: int, to_lds: bool, resident: bool, wg_per_cu: int = 1, mib_per_wg: int = 16, lds_per_cu: int = 160 * 1024) -> float:
    """Bytes per second the whole GPU pulls in with one load-only kernel (median of 5 launches).

    ``resident``: the workgroups of an XCD loop over bytes that stay in its L2 (eight operand
    blocks of 256 KiB, each walked by a quarter of the XCD's workgroups); otherwise every workgroup
    streams 4 MiB of its own once, from a buffer larger than the last-level cache."""
    import torch

    from deplodock_amd.backend.hip import hiprtc, launcher
    from deplodock_amd.backend.hip.launcher import PackedArgs

    lib = launcher.load()
    cus = lib.device_props(0)["compute_units"]
    nt = waves * 64
    name = f"k_l1fill_w{waves}_u{inflight}_s{stride}_{'lds' if to_lds else 'reg'}_{'l2' if resident else 'hbm'}"
    fn = hiprtc.load_function(l1fill_source(name, waves=waves, inflight=inflight, stride=stride, to_lds=to_lds, nontemporal=not resident), name, cached=False)
    lds_bytes = max(lds_per_cu // wg_per_cu - 4096, waves * inflight * 1024 if to_lds else 0)  # also pins the number of workgroups a CU holds
    if lds_bytes > 64 * 1024:
        try:
            lib.func_set_dynamic_lds(fn.fn, lds_bytes)
        except launcher.LauncherError as exc:
            print(f"# {name}: {exc}; attributes {lib.func_attributes(fn.fn)}", flush=True)
            if waves * inflight * 1024 > 64 * 1024:
                raise
            lds_bytes = 64 * 1024
    grid = cus * wg_per_cu
    wg_bytes = 256 * 1024 if resident else 4 * 1024 * 1024 * max(1, stride // 2048)  # streamed: 4 MiB actually read per workgroup
    if stride:  # whole laps of (32 row blocks x 8 rows), of which 16 pieces of 128 bytes per row are read
        laps = max(1, wg_bytes // (256 * stride))
        laps = 1 << (laps.bit_length() - 1)  # the kernel wraps a workgroup's unit index with a mask
        wg_bytes, wg_units = laps * 256 * stride, laps * 512
    else:
        wg_units = wg_bytes // 1024
    share = 8 if resident else 0
    region = (8 * share * wg_bytes) if resident else grid * wg_bytes
    buf = torch.empty(region + 4096, dtype=torch.uint8, device="cuda").random_(0, 255)
    out = torch.zeros(grid * nt, dtype=torch.int32, device="cuda")
    per_wave = (mib_per_wg * 1024 if resident else wg_units) // waves
    units_per_wave = max(inflight, per_wave // inflight * inflight)
    if wg_units & (wg_units - 1) or wg_bytes >= 2**31:
        raise ValueError("l1fill: a workgroup's unit count must be a power of two and its bytes fit 31 bits")
    args = PackedArgs([buf.data_ptr(), out.data_ptr()], [units_per_wave, wg_units, wg_bytes // 1024, share])
    e0, e1 = lib.event_create(), lib.event_create()
    times = []
    for _ in range(6):
        lib.event_record(e0, None)
        lib.launch(fn.fn, (grid, 1, 1), (nt, 1, 1), lds_bytes, None, args)
        lib.event_record(e1, None)
        torch.cuda.synchronize()
        times.append(lib.event_elapsed_ms(e0, e1) * 1e-3)
    lib.event_destroy(e0)
    lib.event_destroy(e1)
    lib.module_unload(fn.module)
    moved = grid * waves * units_per_wave * 1024
    return moved / sorted(times[1:])[len(times[1:]) // 2]


def handle_l1fill(args) -> None:
    from deplodock_amd.backend.hip import launcher
    from deplodock_amd.commands.table import render_table

    props = launcher.load().device_props(0)
    cus, clk = props["compute_units"], props["clock_khz"] * 1e3
    print(f"load-only kernels on {cus} CUs; B/clk/CU at the {clk / 1e9:.2f} GHz engine clock the driver reports")
    rows = []
    quick = getattr(args, "quick", False)
    for resident in (True, False):
        for stride in (0, 2048, 2048 + 128, 8192) if not quick else (0, 2048):
            for to_lds in (False, True):
                for waves in (4, 8, 16) if not quick else (8,):
                    for inflight in (2, 4, 8, 16) if not quick else (4,):
                        if to_lds and waves * inflight > 128:
                            continue
                        bps = l1fill_bytes_per_second(waves=waves, inflight=inflight, stride=stride, to_lds=to_lds, resident=resident)
                        rows.append(["L2" if resident else "HBM", "1 KiB runs" if stride == 0 else f"8 rows x 128 B, stride {stride}", "global_load_lds_dwordx4" if to_lds else "global_load_dwordx4",
                                     str(waves), str(inflight), f"{waves * inflight}", f"{bps / 1e12:.2f}", f"{bps / clk / cus:.1f}"])  # fmt: skip
                        print("  ".join(rows[-1]), flush=True)
    print()
    for line in render_table(["operands in", "pattern", "load", "waves/CU", "loads in flight/wave", "KiB in flight/CU", "TB/s", "B/clk/CU"], rows, "lllrrrrr"):
        print(line)


_LDS_SRC = r"""
// Wave w reads fragments of rows (w * READS + r) * AM + lr, k chunk kk * KG + lk: the EMH_READ of a contraction.
extern "C" __global__ __launch_bounds__(NT) void KNAME(unsigned long long* __restrict__ ticks, unsigned* __restrict__ out, int iters) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  for (int i = tid; i < LDS_BYTES / 4; i += NT) ((unsigned*)lds)[i] = i * 2654435761u;
  __syncthreads();
  const int lr = lane % AM, lk = lane / AM;
  unsigned addr[KS][READS];
  #pragma unroll
  for (int kk = 0; kk < KS; ++kk)
  #pragma unroll
  for (int r = 0; r < READS; ++r) {
    const int row = ((wave * READS + r) * AM + lr) % ROWS, c = kk * KG + lk;
    addr[kk][r] = LINEAR ? (unsigned)((((wave * KS + kk) * READS + r) * 64 + lane) * 16) % LDS_BYTES
                         : (unsigned)(row * ROWB + ((c ^ ((row / RPL) % CPR)) % CPR) * 16);
  }
  u32x4 acc = {0u, 0u, 0u, 0u};
  const unsigned base = (unsigned)(unsigned long long)(__attribute__((address_space(3))) unsigned char*)lds;
  const unsigned long long t0 = __builtin_amdgcn_s_memtime();
  for (int it = 0; it < iters; ++it) {
    #pragma unroll
    for (int kk = 0; kk < KS; ++kk) {
      u32x4 v[READS];
      #pragma unroll
      for (int r = 0; r < READS; ++r) asm volatile("ds_read_b128 %0, %1" : "=v"(v[r]) : "v"(base + addr[kk][r]));
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      #pragma unroll
      for (int r = 0; r < READS; ++r) acc ^= v[r];
    }
  }
  const unsigned long long t1 = __builtin_amdgcn_s_memtime();
  if (lane == 0) ticks[blockIdx.x * (NT / 64) + wave] = t1 - t0;
  if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x9e3779b9u) out[tid] = acc[0];
}
"""


def lds_read_bytes_per_clock(*, atom_rows: int, row_bytes: int, waves: int, reads: int = 8, linear: bool = False, iters: int = 2000) -> float:
    """Bytes per shader clock one CU's waves read from LDS with the contraction emitter's fragment addressing:
    ``atom_rows`` rows a fragment (16 or 32, the lane groups beyond them take neighbouring 16-byte k chunks),
    ``row_bytes`` a slab row, chunks XOR-swizzled by ``(row / rows_per_256B) % chunks_per_row``."""
    import torch

    from deplodock_amd.backend.hip import hiprtc, launcher
    from deplodock_amd.backend.hip.launcher import PackedArgs
    from deplodock_amd.emit import prelude

    lib = launcher.load()
    cpr = row_bytes // 16
    kg = 64 // atom_rows
    ks = max(1, cpr // kg)
    rows = 256
    nt = waves * 64
    name = f"k_ldsread_a{atom_rows}_r{row_bytes}_w{waves}_n{reads}_{int(linear)}"
    defs = dict(NT=nt, AM=atom_rows, KG=kg, KS=ks, READS=reads, ROWS=rows, ROWB=row_bytes, CPR=cpr, RPL=max(1, 16 // cpr), LINEAR=int(linear), LDS_BYTES=rows * row_bytes)
    src = prelude.header() + "".join(f"#define {k} {v}\n" for k, v in defs.items()) + _LDS_SRC.replace("KNAME", name)
    fn = hiprtc.load_function(src, name, cached=False)
    cus = lib.device_props(0)["compute_units"]
    ticks = torch.zeros(cus * waves, dtype=torch.int64, device="cuda")
    out = torch.zeros(nt, dtype=torch.int32, device="cuda")
    args = PackedArgs([ticks.data_ptr(), out.data_ptr()], [iters])
    for _ in range(2):
        lib.launch(fn.fn, (cus, 1, 1), (nt, 1, 1), rows * row_bytes, None, args)
    torch.cuda.synchronize()
    lib.module_unload(fn.module)
    per_cu = ticks.view(cus, waves).max(dim=1).values.double().median().item()  # a CU is done when its slowest wave is
    return waves * iters * ks * reads * 1024 / per_cu


def handle_lds(args) -> None:
    from deplodock_amd.commands.table import render_table

    rows = []
    for waves in (4, 8, 16):
        rows.append(["linear (lane * 16)", "-", str(waves), f"{lds_read_bytes_per_clock(atom_rows=16, row_bytes=128, waves=waves, linear=True):.1f}"])
        for atom_rows in (16, 32):
            for row_bytes in (64, 128, 256):
                rows.append([f"{atom_rows}-row fragments", str(row_bytes), str(waves), f"{lds_read_bytes_per_clock(atom_rows=atom_rows, row_bytes=row_bytes, waves=waves):.1f}"])
        print("  ".join(rows[-1]), flush=True)
    for line in render_table(["ds_read_b128 pattern", "slab row bytes", "waves/CU", "B/clk/CU"], rows, "llrr"):
        print(line)


def handle_flash(args) -> None:
    """Stamps and ablations of the software-pipelined attention forms (the switches are compile-time defines of
    ``emit/flash_ws.py``; an ablated kernel's output is not attention, a stamped kernel's first output words hold the
    stamps)."""
    import os

    import torch

    from deplodock_amd import HipBackend, trace_module, workloads
    from deplodock_amd.commands.table import render_table

    dev = torch.device("cuda:0")
    case = workloads.sdpa_case(s=int(args.seq))
    pins = [p for p in (args.pins or "w2/kv32/s2/p/ws,w2/kv32/s4/p/sp").split(",") if p]
    saved = {k: os.environ.get(k) for k in ("EMMY_FLASH", "EMMY_HIPRTC_FLAGS")}

    def build(pin, flags):
        for key, val in (("EMMY_FLASH", pin), ("EMMY_HIPRTC_FLAGS", flags)):
            if val:
                os.environ[key] = val
            else:
                os.environ.pop(key, None)
        be = HipBackend()
        compiled = be.compile(trace_module(case.module, case.inputs))
        return be, compiled, {n: t.to(dev) for n, t in zip(compiled.inputs, case.inputs)}

    def time_us(pin, flags):
        be, compiled, data = build(pin, flags)
        res = be.benchmark(compiled, warmup=3, num_iters=30, input_data=data)
        return res.time_ms * 1e3

    def stamps(pin, mode):
        be, compiled, data = build(pin, f"-DEMH_STAMP={mode}")
        prog = be.program(compiled, data)
        try:
            for _ in range(2):
                prog.run()
                torch.cuda.synchronize()
            w = prog.output_tensors()[compiled.outputs[0]].reshape(-1)[:8].view(torch.float32)
            return [w[i].item() for i in range(4)]
        finally:
            prog.close()

    try:
        rows = [["default", "-", f"{time_us(None, None):.2f}", "", "", "", ""]]
        for pin in pins:
            rows.append([pin, "-", f"{time_us(pin, None):.2f}", "", "", "", ""])
            for what, flag in (("no requests in the loop", 1), ("no consumer arithmetic", 2), ("no exponentials", 3), ("no fragment reads", 4)):
                rows.append([pin, what, f"{time_us(pin, f'-DEMH_ABLATE={flag}'):.2f}", "", "", "", ""])
            it = stamps(pin, 1)
            rows.append([pin, "clocks per iteration (wave 0): barrier / lead / first half / second half", "", f"{it[3]:.0f}", f"{it[0]:.0f}", f"{it[1]:.0f}", f"{it[2]:.0f}"])
            ph = stamps(pin, 2)
            rows.append([pin, "clocks per workgroup (wave 0): prologue / loops / tail / close + store", "", f"{ph[0]:.0f}", f"{ph[1]:.0f}", f"{ph[2]:.0f}", f"{ph[3]:.0f}"])
            print("  ".join(rows[-1]), flush=True)
    finally:
        for key, val in saved.items():
            if val is None:
                os.environ.pop(key, None)
            else:
                os.environ[key] = val
    for line in render_table(["FLASH", "variant", "us", "a", "b", "c", "d"], rows, "llrrrrr"):
        print(line)


def handle_fp32_attention(args) -> None:
    """fp32 causal attention with grouped heads (the reference's ``sdpa`` perf shape, tests/perf/cases.py:174-190, and
    longer sequences): the streaming kernel's forms against the decomposed route and eager."""
    import os

    import torch

    from deplodock_amd import HipBackend, trace_module, workloads
    from deplodock_amd.commands.table import render_table
    from deplodock_amd.ir.hip import HipOp

    dev = torch.device("cuda:0")
    saved = os.environ.get("EMMY_FLASH")
    rows = []
    try:
        for seq in (int(x) for x in args.seq.split(",")):
            case = workloads.sdpa_case(s=seq)
            inputs = tuple(t.float() for t in case.inputs)
            on_dev = [t.to(dev) for t in inputs]
            for _ in range(3):
                case.module(*on_dev)
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(10):
                case.module(*on_dev)
            e1.record()
            torch.cuda.synchronize()
            row = [str(seq), f"{case.algo_flops / 1e9:.2f}"]
            best = None
            for pin in (None, "f32/w4", "f32/s2", "f32/s2/sp", "f32/s4", "f32/s4/sp", "f32/s4/o", "f32/s8/o", "decompose"):
                if pin == "decompose" and seq > 2048:
                    row.append("")
                    continue
                if pin:
                    os.environ["EMMY_FLASH"] = pin
                else:
                    os.environ.pop("EMMY_FLASH", None)
                be = HipBackend()
                compiled = be.compile(trace_module(case.module, inputs))
                res = be.benchmark(compiled, warmup=3, num_iters=10 if seq >= 2048 else 30, input_data=dict(zip(compiled.inputs, on_dev)))
                us = sum(p.time_ms for p in res.per_launch) * 1e3
                if pin is None:
                    (op,) = [n.op for n in compiled.nodes.values() if isinstance(n.op, HipOp)]
                    row.append(f"{op.knobs['FLASH']} {us:.1f}")
                    best = us
                else:
                    row.append(f"{us:.1f}")
            row += [f"{e0.elapsed_time(e1) * 100:.1f}", f"{case.algo_flops / best / 1e6:.1f}", f"{case.algo_flops / best / 1e6 / 157.3:.2f}"]
            rows.append(row)
    finally:
        if saved is None:
            os.environ.pop("EMMY_FLASH", None)
        else:
            os.environ["EMMY_FLASH"] = saved
    print("fp32 causal attention, 16 query / 8 key-value heads of 128, us per call (the decomposed route: sum of its kernels)")
    for line in render_table(["S", "GFLOP", "default", "w4", "s2", "s2/sp", "s4", "s4/sp", "s4/o", "s8/o", "decomposed", "eager fp32", "TFLOP/s", "of fp32 MFMA peak"], rows, "rrlrrrrrrrrrrr"):
        print(line)


def handle_stamps(args) -> None:
    """Phase stamps of the default attention kernel and of the ring contractions (``-DEMH_STAMP=1`` / ``2`` builds of
    ``emit/flash.py`` and ``emit/contraction.py``): the first thread of workgroup 0 leaves four floats over the first
    16 bytes it stored — clocks per key step / slab by phase, and clocks per part of the kernel."""
    import os

    import torch

    from deplodock_amd import HipBackend, trace_module, workloads
    from deplodock_amd.commands.table import render_table
    from deplodock_amd.ir.hip import HipOp

    dev = torch.device("cuda:0")
    saved = os.environ.get("EMMY_HIPRTC_FLAGS")

    def run(case, mode, where):
        if mode:
            os.environ["EMMY_HIPRTC_FLAGS"] = f"-DEMH_STAMP={mode}"
        else:
            os.environ.pop("EMMY_HIPRTC_FLAGS", None)
        be = HipBackend()
        compiled = be.compile(trace_module(case.module, case.inputs))
        (op,) = [n.op for n in compiled.nodes.values() if isinstance(n.op, HipOp)]
        data = {n: t.to(dev) for n, t in zip(compiled.inputs, case.inputs)}
        if not mode:
            res = be.benchmark(compiled, warmup=3, num_iters=30, input_data=data)
            return op, res.time_ms * 1e3
        prog = be.program(compiled, data)
        try:
            for _ in range(3):
                prog.run()
                torch.cuda.synchronize()
            flat = prog.output_tensors()[compiled.outputs[0]].reshape(-1)
            w = flat[where(op) : where(op) + 8].view(torch.float32)
            return op, [w[i].item() for i in range(4)]
        finally:
            prog.close()

    rows = []
    try:
        for seq in (2048, 512):
            case = workloads.sdpa_case(s=seq)

            def first_row(op, seq=seq):  # the first row workgroup 0 stores in its last pass: row 0 of a mirrored pair, else the last query block's
                rows_wg = 32 * int(op.knobs["FLASH"].split("/")[0][1:])
                return 0 if "/p" in op.knobs["FLASH"] else (seq - rows_wg) * 128

            op, us = run(case, 0, first_row)
            _, st = run(case, 1, first_row)
            _, ph = run(case, 2, first_row)
            rows.append([f"attention S={seq} {op.knobs['FLASH']}", f"{us:.2f}", "step: scores / softmax / output MFMAs / hand-over", *(f"{v:.0f}" for v in st)])
            rows.append(["", "", "pass: prologue / key loop / close / store", *(f"{v:.0f}" for v in ph)])
        for m, k, n in ((4096, 4096, 4096), (2048, 1024, 3072), (512, 1024, 3072)):
            case = workloads.linear_case(m=m, k=k, n=n)
            op, us = run(case, 0, lambda op: 0)
            _, st = run(case, 1, lambda op: 0)
            _, ph = run(case, 2, lambda op: 0)
            what = "period: MFMAs / fragment reads / barrier / -" if op.knobs["STAGE"].endswith("/pp") else "slab: steps before / hand-over / last step / -"
            rows.append([f"linear {m}x{k}x{n} {op.knobs['TILE'].split('/', 1)[1]} {op.knobs['STAGE']}", f"{us:.2f}", what, *(f"{v:.0f}" for v in st)])
            rows.append(["", "", "kernel: prologue / k loop / epilogue arithmetic / stores", *(f"{v:.0f}" for v in ph)])
    finally:
        if saved is None:
            os.environ.pop("EMMY_HIPRTC_FLAGS", None)
        else:
            os.environ["EMMY_HIPRTC_FLAGS"] = saved
    for line in render_table(["kernel", "us", "clocks of workgroup 0's first wave", "a", "b", "c", "d"], rows, "lrlrrrr"):
        print(line)


def register_microbench_command(subparsers) -> None:
    p = subparsers.add_parser("microbench", help="Measure the MFMA rate, MFMA/VALU co-issue and the L1 fill rate of the GPU")
    p.add_argument("--l1fill", action="store_true", help="sweep load-only kernels: bytes per clock a CU pulls through its vector L1")
    p.add_argument("--quick", action="store_true", help="with --l1fill: a four-line sweep")
    p.add_argument("--lds", action="store_true", help="fragment-read rate out of LDS for the emitters' swizzled layouts")
    p.add_argument("--flash", action="store_true", help="phase stamps and ablations of the software-pipelined attention kernels on the benchmark shape")
    p.add_argument("--stamps", action="store_true", help="phase stamps (shader clocks) of the default attention kernel and of the ring contractions on the benchmark shapes")
    p.add_argument("--fp32-attention", action="store_true", help="fp32 attention: the streaming kernel's forms against the decomposed route and eager (--seq: comma-separated lengths)")
    p.add_argument("--pins", default=None, help="with --flash: comma-separated EMMY_FLASH pins (default: the ws and sp forms of the benchmark shape)")
    p.add_argument("--seq", default="2048", help="with --flash: sequence length; with --fp32-attention: comma-separated lengths")
    p.set_defaults(func=handle_microbench)


def handle_microbench(args) -> None:
    import torch

    if not torch.cuda.is_available():
        print("error: no HIP device visible", file=sys.stderr)
        sys.exit(1)
    if getattr(args, "l1fill", False):
        handle_l1fill(args)
        return
    if getattr(args, "lds", False):
        handle_lds(args)
        return
    if getattr(args, "flash", False):
        handle_flash(args)
        return
    if getattr(args, "stamps", False):
        handle_stamps(args)
        return
    if getattr(args, "fp32_attention", False):
        handle_fp32_attention(args)
        return
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
