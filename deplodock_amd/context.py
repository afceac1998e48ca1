"""Per-compilation hardware facts for gfx950 (MI355X).

The reference's ``Context`` (emmy/compiler/context.py:69-260) carries NVIDIA
facts (warp 32, 48 KB static smem, SM count 170).  This one carries what the
gfx950 schedule heuristics and emitters read instead.
"""

from __future__ import annotations

from dataclasses import dataclass

HBM_PEAK_BYTES_PER_S = 8.0e12  # MI355X HBM3E
MFMA_BF16_PEAK_FLOPS = 2.5e15  # dense bf16/fp16 MFMA
MFMA_FP32_PEAK_FLOPS = 157.3e12


@dataclass(frozen=True)
class Context:
    arch: str = "gfx950"
    wave_size: int = 64
    compute_units: int = 256
    xcds: int = 8  # accelerator complex dies; each has its own L2
    simds_per_cu: int = 4
    max_threads_per_block: int = 1024
    lds_bytes_per_cu: int = 160 * 1024
    static_lds_cap: int = 64 * 1024  # per-workgroup LDS without opting into more
    lds_banks: int = 64
    vgprs_per_lane: int = 512  # unified VGPR+AGPR file at one wave per SIMD
    l2_bytes_per_xcd: int = 4 * 1024 * 1024
    backend_name: str = "hip"
    compile_flags: str = ""
    tune_db: object = None  # a ``deplodock_amd.tune.TuneDB`` the schedule consults for pins, or None

    @property
    def cus_per_xcd(self) -> int:
        return self.compute_units // self.xcds

    @classmethod
    def from_target(cls, target: str = "gfx950", **kw) -> Context:
        """Build a context for ``--target gfx950`` (emmy/compiler/target.py:28-83
        parses ``sm_NN``; only gfx950 exists here)."""
        t = target.split(":")[0].strip().lower()
        if t != "gfx950":
            raise ValueError(f"unsupported target {target!r}: this backend emits gfx950 code only")
        return cls(arch=t, **kw)

    @classmethod
    def probe(cls) -> Context:
        """Context for the live device, falling back to the nominal MI355X
        figures when no GPU is visible (compile-only hosts)."""
        from deplodock_amd.backend.hip import launcher

        try:
            lib = launcher.load()
            if lib.device_count() > 0:
                p = lib.device_props(0)
                return cls(arch=p["arch"].split(":")[0], compute_units=p["compute_units"], wave_size=p["wavefront_size"])
        except launcher.LauncherError:
            pass
        return cls()


DEFAULT = Context()
