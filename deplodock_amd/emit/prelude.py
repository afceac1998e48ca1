"""Source fragments shared by every emitted kernel.

Replaces the reference's CUDA preludes (emmy/compiler/ir/kernel/render.py:36-372:
TMA helpers, ldmatrix / mma.sync PTX wrappers) with what CDNA4 offers instead:
wave64 DPP / swizzle / permlane butterflies, native bf16 conversion and MFMA
fragment types.  hipRTC predefines the HIP device runtime, so no #include.
"""

from __future__ import annotations

TYPES = r"""
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned short u16x4 __attribute__((ext_vector_type(4)));
#define EMH_DEV __device__ __forceinline__
"""

# Direct-to-LDS loads and their publication; only the emitters that stage through LDS include it.
DMA = r"""
// Direct-to-LDS load of 16 bytes per lane: lane l's bytes land at lds_base + 16*l
// (lds_base: the wave-uniform LDS byte address, carried in M0).  Issued as inline
// assembly on purpose: for the builtin the compiler assumes any later LDS read may
// alias the load's LDS write and drains every outstanding load (vmcnt(0)) before
// it, which turns a ring of slabs into one slab in flight.  The caller orders
// reads after loads itself (vmcnt wait, LDS fence read, barrier).  M0 is named as
// clobbered so the compiler never keeps a value of its own in it across the load.
EMH_DEV unsigned emh_lds_addr(const void* p) { return (unsigned)(unsigned long)(__attribute__((address_space(3))) const void*)p; }
// Publishing direct-to-LDS data to the other waves: the counter that tracks the
// loads can reach its target before the LDS writes are visible.  A flat load from
// LDS travels the same path as those writes and so queues behind them; waiting for
// it (on the LDS counter alone: the vector-memory counter would also drain the
// younger loads of the ring) orders them before the barrier that follows.
EMH_DEV void emh_lds_publish(const void* lds_generic) {
  unsigned d_;
  asm volatile("flat_load_dword %0, %1 sc0 sc1\n\ts_waitcnt lgkmcnt(0)" : "=v"(d_) : "v"(lds_generic) : "memory");
}
EMH_DEV void emh_dma16(const void* g, const void* lds_wave_base) {
  const unsigned m0_ = __builtin_amdgcn_readfirstlane(emh_lds_addr(lds_wave_base));
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" :: "v"(g), "s"(m0_) : "memory", "m0");
}
// The same load with its address split into a wave-uniform 64-bit base (scalar registers) and a 32-bit
// per-lane byte offset: a loop that walks the base needs no vector arithmetic per request.
EMH_DEV void emh_dma16s(const void* sbase, unsigned voff, unsigned lds_wave_base) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" :: "v"(voff), "s"(sbase), "s"(lds_wave_base) : "memory", "m0");
}
// Values that are wave-uniform by construction but that the compiler may keep in vector registers (they went
// through a branch on the wave's role): these move them to scalar registers, once, where they are computed.
EMH_DEV unsigned emh_uniform(unsigned x) { return (unsigned)__builtin_amdgcn_readfirstlane(x); }
EMH_DEV const unsigned char* emh_uniform(const void* p) {
  // the builtin returns a signed int: each half goes through unsigned, or a low half with bit 31 set would
  // sign-extend over the high half
  const unsigned long b_ = (unsigned long)p;
  const unsigned lo_ = (unsigned)__builtin_amdgcn_readfirstlane((unsigned)b_), hi_ = (unsigned)__builtin_amdgcn_readfirstlane((unsigned)(b_ >> 32));
  return (const unsigned char*)(((unsigned long)hi_ << 32) | (unsigned long)lo_);
}
"""

# Wave64 butterflies.  Each step combines a lane with its partner at XOR
# distance 1, 2 (quad_perm), then mirrored halves of 8 and 16 lanes (after the
# earlier steps a mirrored partner holds the same value as the XOR partner),
# then XOR 16 through the LDS crossbar (ds_swizzle, no memory touched); the two
# 32-lane halves, uniform by then, meet through v_readlane.  Every lane of each W-lane group ends with the
# group result, and the combination order is fixed (bit-reproducible).
# The reference's counterpart is the __shfl_xor_sync butterfly plus a
# shared-memory tree (emmy/compiler/ir/kernel/ir.py:608-702).
WAVE_REDUCE = r"""
template <int CTRL> EMH_DEV float emh_dpp(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
EMH_DEV float emh_xor16(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x401F));
}
struct EmhSum { static EMH_DEV float op(float a, float b) { return a + b; } static EMH_DEV float identity() { return 0.0f; } };
struct EmhMax { static EMH_DEV float op(float a, float b) { return fmaxf(a, b); } static EMH_DEV float identity() { return -__builtin_inff(); } };
struct EmhMin { static EMH_DEV float op(float a, float b) { return fminf(a, b); } static EMH_DEV float identity() { return __builtin_inff(); } };
template <class M, int W> EMH_DEV float emh_wave_reduce(float v) {
  if (W >= 2) v = M::op(v, emh_dpp<0xB1>(v));   // quad_perm [1,0,3,2]
  if (W >= 4) v = M::op(v, emh_dpp<0x4E>(v));   // quad_perm [2,3,0,1]
  if (W >= 8) v = M::op(v, emh_dpp<0x141>(v));  // row_half_mirror
  if (W >= 16) v = M::op(v, emh_dpp<0x140>(v)); // row_mirror
  if (W >= 32) v = M::op(v, emh_xor16(v));
  if (W >= 64) {  // both 32-lane halves are uniform by now: combine them through scalar registers
    float lo = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 0));
    float hi = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 32));
    v = M::op(lo, hi);
  }
  return v;
}
"""

MONOID_STRUCT = {"sum": "EmhSum", "max": "EmhMax", "min": "EmhMin"}


def header(*parts: str) -> str:
    return "\n".join(p.strip("\n") for p in (TYPES, *parts)) + "\n"
