"""Fused attention for short sequences on 16-bit operands: one row group per workgroup, its waves split the keys.

The streaming kernel of ``emit/flash.py`` shares every staged K / V block between the waves of a workgroup and pays a
workgroup barrier per key step; where a sequence is a handful of key steps long (the decoder block at 512 tokens: four)
those hand-overs, not the matrix pipe, are the kernel's time.  This form keeps the same algebra and fragment layouts —
``S^T = K Q^T`` so a lane owns one query, ``P`` from the accumulator registers straight into the B operand of
``O^T = V^T P^T``, V fragments from the transposing LDS read, the online ``(m, l, O)`` carrier of
emmy/compiler/pipeline/passes/lowering/kernel/_twist.py:229-363 — but gives every wave its own key blocks:

* a workgroup is 32 query rows and ``kv_split`` waves (2, 4 or 8); wave g takes key blocks g, g + kv_split, ... and
  stages them itself with direct-to-LDS loads into its own region (one 32-key K block, one V block): **no barrier in the
  loop**.  The next K block is requested when the score MFMAs are done and lands under the softmax and the output
  MFMAs; the next V block is requested after the output MFMAs and lands under the next scores (waits by count of
  outstanding requests).
* K lies in LDS as [pair of 16-byte chunks][row][32 bytes]: a wave's fragment reads at one k position are 1 KiB in a
  row (conflict-free), and request u of a block is one loop-invariant lane offset plus 32 bytes x u.  V keeps the
  ``[key][d]`` rows with the chunk swizzle the transposing reads want; the rows of one request share their swizzle, so
  a V request is one lane offset plus a row step as well.
* the waves' ``(m, l, O)`` meet once, through LDS, with the exp-family combine, and the output leaves in whole rows.

Every wave fetches its own blocks, so the K / V traffic per CU is that of the shared form's 64-row workgroups at twice
the workgroups: the form is for sequences short enough that the launch is latency-bound (the scheduler's rule).
"""

from __future__ import annotations

import math

from deplodock_amd.context import Context
from deplodock_amd.emit import prelude
from deplodock_amd.emit.errors import LoweringError
from deplodock_amd.ir.expr import float_literal
from deplodock_amd.ir.hip import HipOp
from deplodock_amd.ir.sym import Affine, CeilDiv, c_value, param_name
from deplodock_amd.ir.tile import Flash
from deplodock_amd.render_target import rt

HEAD_DIMS = (64, 128)


def lds_bytes(head_dim: int, kvs: int) -> int:
    """The waves' K / V regions during the loop; at the close the same memory holds their fp32 partial outputs
    (rows padded by four floats) and ``(m, l)`` pairs."""
    return max(kvs * 2 * 32 * head_dim * 2, kvs * (32 * (head_dim + 4) + 64) * 4)


def max_key_split(head_dim: int, lds_limit: int) -> int:
    return next((k for k in (8, 4, 2) if lds_bytes(head_dim, k) <= lds_limit), 1)


_SRC = r"""
#define CPR (D / 8)                    /* 16-byte chunks per row */
#define RPR (64 / CPR)                 /* V rows per direct-to-LDS request */
#define NIK (D / 16)                   /* requests of a wave per K block: 32 rows x two chunks each */
#define NIV (32 / RPR)                 /* requests of a wave per V block: whole rows */
#define NDB (D / 32)                   /* 32-column blocks of the output */
#define TG (D / 32 < 4 ? D / 32 : 4)
#define REGION (2 * 32 * D * 2)        /* bytes of LDS per wave in the loop: its K block, then its V block */
#define PS (D + 4)                     /* floats per row of a wave's partial output at the close */
#define PART (32 * PS + 64)            /* floats per wave at the close: 32 rows, then (m, l) per row */
// V keeps [key][d] order; its 16-byte chunks are XOR-swizzled in groups of four so the four consecutive key rows one
// transposing read touches sit in four different bank quarters.
#define EMH_VROT(row) (D >= 128 ? ((row) % 4) : (((row) >> 1) & 1))  /* 128-byte rows: two rows share a bank line */
EMH_DEV int emh_vswz(int row, int c) { return c ^ (EMH_VROT(row) << 2); }
typedef short emh_s16x4 __attribute__((ext_vector_type(4)));

extern "C" __global__ __launch_bounds__(NT) void KNAME(const ELT* __restrict__ Q, const ELT* __restrict__ Kp,
                                                      const ELT* __restrict__ Vp MASK_PARAM, ELT* __restrict__ Op SYM_PARAM) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];  // [KVS waves][K: D / 16 x 32 x 32 B | V: 32 x D]
  const int tid = threadIdx.x, lane = tid % 64, grp = __builtin_amdgcn_readfirstlane(tid / 64);
  const int lq = lane % 32, lh = lane / 32;
  // Workgroup ids go round-robin over the XCDs, each with its own L2: consecutive logical ids (the query blocks of one
  // head, then the next head of the same KV group) are dealt to one XCD, so a KV head's keys and values come out of one L2.
  const int grid = (int)gridDim.x;
  const int bid = grid % XCDS == 0 ? (int)(blockIdx.x % XCDS) * (grid / XCDS) + (int)(blockIdx.x / XCDS) : (int)blockIdx.x;
  const int qblocks = (SQ + 31) / 32;
  const int qb = (qblocks - 1) - bid % qblocks;  // under a causal mask the heaviest blocks start first
  const int head = (bid / qblocks) % HQ;
  const int batch = bid / (qblocks * HQ);
  const int kvh = head / GROUP;
  const int q0 = qb * 32;
  const int qrow = q0 + lq;
  const int qrow_c = qrow < SQ ? qrow : SQ - 1;

  const ELT* kbase = Kp + K_OFF + (long)batch * K_SB + (long)kvh * K_SH;
  const ELT* vbase = Vp + V_OFF + (long)batch * V_SB + (long)kvh * V_SH;
#if HAS_MASK
  const MELT* mrow = Mp + M_OFF + (long)batch * M_SB + (long)head * M_SH + (long)qrow_c * M_SS;
#endif
  int kend = SKV;
  if (CAUSAL) { const int last = (q0 + 32 < SQ ? q0 + 32 : SQ); kend = last < kend ? last : kend; }
  const int nblocks = (kend + 31) / 32;

  unsigned char* kl = lds + grp * REGION;
  unsigned char* vl = kl + 32 * D * 2;
  const unsigned kl_s = emh_uniform(emh_lds_addr(kl)), vl_s = emh_uniform(emh_lds_addr(vl));
  // Lane offsets (bytes) of the requests of a block that lies wholly inside the sequence: K request u is rows lane / 2,
  // chunk 2 u + lane % 2; V request i is rows i RPR + lane / CPR, chunk position lane % CPR, which holds the chunk that
  // the row's swizzle maps there (the rows of a request are whole groups of four, so they share it).
  const unsigned koff = (unsigned)(lane / 2) * (unsigned)(K_SS * 2) + (unsigned)(lane % 2) * 16u;
  const unsigned voff = (unsigned)(lane / CPR) * (unsigned)(V_SS * 2) + (unsigned)emh_vswz(lane / CPR, lane % CPR) * 16u;
  // A block that hangs over the sequence's end repeats the last key in the rows past it (masked below, finite here): per-lane addresses.
  #define EMH_REQUEST_K(j_) { \
    if ((j_) * 32 + 32 <= SKV) { \
      const unsigned char* b_ = emh_uniform(kbase + (long)(j_) * 32 * K_SS); \
      _Pragma("unroll") for (int i = 0; i < NIK; ++i) emh_dma16s(b_ + i * 32, koff, kl_s + i * 1024); \
    } else { \
      _Pragma("unroll") for (int i = 0; i < NIK; ++i) { \
        int key_ = (j_) * 32 + lane / 2; key_ = key_ < SKV ? key_ : SKV - 1; \
        emh_dma16(kbase + (long)key_ * K_SS + i * 16 + (lane % 2) * 8, kl + i * 1024); \
      } \
    } }
  #define EMH_REQUEST_V(j_) { \
    if ((j_) * 32 + 32 <= SKV) { \
      const unsigned char* b_ = emh_uniform(vbase + (long)(j_) * 32 * V_SS); \
      _Pragma("unroll") for (int i = 0; i < NIV; ++i) emh_dma16s(b_ + (long)i * RPR * V_SS * 2, voff, vl_s + i * 1024); \
    } else { \
      _Pragma("unroll") for (int i = 0; i < NIV; ++i) { \
        const int row_ = i * RPR + lane / CPR; \
        int key_ = (j_) * 32 + row_; key_ = key_ < SKV ? key_ : SKV - 1; \
        emh_dma16(vbase + (long)key_ * V_SS + emh_vswz(row_, lane % CPR) * 8, vl + i * 1024); \
      } \
    } }

  f32x16 oacc[NDB];
  #pragma unroll
  for (int b = 0; b < NDB; ++b)
    #pragma unroll
    for (int r = 0; r < 16; ++r) oacc[b][r] = 0.0f;
  float m_run = -__builtin_inff(), l_run = 0.0f;  // l_run: this lane's 16 keys of every block; the halves meet at the close

  if (grp < nblocks) {
    EMH_REQUEST_K(grp)
    EMH_REQUEST_V(grp)
  }
  // The query's fragments, requested behind the first blocks and waited for here, before the loop: a load of the
  // compiler's own still outstanding at the loop's head would make it wait inside the loop, by a count that knows
  // nothing of the requests above and so drains them.
  FRAG qf[D / 16];
  {
    const ELT* qp = Q + Q_OFF + (long)batch * Q_SB + (long)head * Q_SH + (long)qrow_c * Q_SS;
    #pragma unroll
    for (int kk = 0; kk < D / 16; ++kk) qf[kk] = *(const FRAG*)(qp + 16 * kk + 8 * lh);
    #pragma unroll
    for (int kk = 0; kk < D / 16; ++kk) {
      u32x4 t_ = __builtin_bit_cast(u32x4, qf[kk]);
      asm volatile("" : "+v"(t_));
      qf[kk] = __builtin_bit_cast(FRAG, t_);
    }
  }
  // ds_read_b64_tr_b16: within 16 lanes, lane i receives element (i % 4) of the 8-byte chunks addressed by lanes i/4,
  // i/4 + 4, i/4 + 8, i/4 + 12.  Lane i therefore points at key row (i / 4) and d-chunk 4*(i % 4) of its half tile, and
  // receives four consecutive keys of its own d = 32*T + (l % 32): the V operand fragment of an MFMA step is two such
  // reads and no shuffling.
  const int i16 = lane % 16, q4 = i16 / 4;
  const int v_lane = (4 * lh + q4) * (D * 2) + ((lane % 32) / 16) * 32 + (i16 % 4) * 8;
  int v_tile[TG];
  #pragma unroll
  for (int T = 0; T < TG; ++T) v_tile[T] = v_lane + ((T ^ EMH_VROT(q4)) * 64);

  #pragma unroll 1
  for (int j = grp; j < nblocks; j += KVS) {
    const bool more = j + KVS < nblocks;
    const int k0 = j * 32;
    asm volatile("s_waitcnt vmcnt(%0)" :: "n"(NIV) : "memory");  // this block's K has landed (its V may still be on its way)
    emh_lds_publish(kl);
    f32x16 s;
    #pragma unroll
    for (int r = 0; r < 16; ++r) s[r] = 0.0f;
    {
      const unsigned char* kfrag = kl + lq * 32 + lh * 16;
      FRAG kf[D / 16];
      #pragma unroll
      for (int kk = 0; kk < D / 16; ++kk) kf[kk] = *(const FRAG*)(kfrag + kk * 1024);
      #pragma unroll
      for (int kk = 0; kk < D / 16; ++kk) s = MFMA(kf[kk], qf[kk], s, 0, 0, 0);
    }
    // the K fragments are in registers (the MFMAs above consumed them): the region takes the next block
    asm volatile("" :: "v"(s[0]) : "memory");
    if (more) EMH_REQUEST_K(j + KVS)
    // register r: key k0 + 8 (r / 4) + 4 lh + r % 4 of query qrow, in log2 units from here on
    float mx = -__builtin_inff();
    #pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int key = k0 + 8 * (r / 4) + 4 * lh + (r % 4);
      float v = s[r] * SCALE_LOG2;
#if HAS_MASK
      v += (float)mrow[key < SKV ? key : SKV - 1] * 1.4426950408889634f;
#endif
      if (key >= SKV || (CAUSAL && key > qrow)) v = -__builtin_inff();
      s[r] = v;
      mx = fmaxf(mx, v);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    // The reference maximum is raised only when a row outgrows it by 2^8 (probabilities stay below 2^8, far inside the
    // operands' range), so the rescale of the accumulators is rare.
    const bool raise = mx > m_run + 8.0f;  // (from -inf any finite maximum raises; a block of masked keys never does)
    if (__any(raise)) {
      const float alpha = raise ? EXP2(m_run - mx) : 1.0f;
      m_run = raise ? mx : m_run;
      l_run *= alpha;
      #pragma unroll
      for (int b = 0; b < NDB; ++b)
        #pragma unroll
        for (int r = 0; r < 16; ++r) oacc[b][r] *= alpha;
    }
    const float m_use = m_run == -__builtin_inff() ? 0.0f : m_run;  // nothing but masked keys so far: every term is 0
    float lsum = 0.0f;
    #pragma unroll
    for (int r = 0; r < 16; ++r) { s[r] = EXP2(s[r] - m_use); lsum += s[r]; }
    l_run += lsum;
    if (more) asm volatile("s_waitcnt vmcnt(%0)" :: "n"(NIK) : "memory");  // V of this block (the next K block may be on its way)
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    emh_lds_publish(vl);
    // all V fragments of the block are fetched before its output MFMAs: the LDS latency is paid once per block
    u32x4 vfr[2 * NDB];
    #pragma unroll
    for (int h2 = 0; h2 < 2; ++h2)
      #pragma unroll
      for (int dt = 0; dt < NDB; ++dt) {
        const unsigned char* vp = vl + (16 * h2) * (D * 2) + (dt / TG) * 256 + v_tile[dt % TG];
        const emh_s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) emh_s16x4*)(vp));
        const emh_s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) emh_s16x4*)(vp + 8 * (D * 2)));
        const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2_ = __builtin_bit_cast(u32x2, hi);
        u32x4 av;
        av[0] = l2[0]; av[1] = l2[1]; av[2] = h2_[0]; av[3] = h2_[1];
        vfr[h2 * NDB + dt] = av;
      }
    __builtin_amdgcn_sched_barrier(0);
    #pragma unroll
    for (int h2 = 0; h2 < 2; ++h2) {
      FRAG pf;
      #pragma unroll
      for (int t = 0; t < 8; ++t) pf[t] = (ELT)s[8 * h2 + t];
      #pragma unroll
      for (int dt = 0; dt < NDB; ++dt) oacc[dt] = MFMA(__builtin_bit_cast(FRAG, vfr[h2 * NDB + dt]), pf, oacc[dt], 0, 0, 0);
    }
    #pragma unroll
    for (int b = 0; b < NDB; ++b) asm volatile("" :: "v"(oacc[b][0]) : "memory");  // every V fragment has been consumed
    if (more) EMH_REQUEST_V(j + KVS)
  }

  // Close: when every wave is done with its blocks the same memory takes the waves' unnormalised output rows, maxima and
  // sums; after the second barrier the threads of the workgroup each finish 16-byte pieces of the output rows
  // (consecutive threads, consecutive pieces).
  __syncthreads();
  {
    const float l = l_run + __shfl_xor(l_run, 32, 64);
    float* part = (float*)lds + grp * PART;
    #pragma unroll
    for (int b = 0; b < NDB; ++b)
      #pragma unroll
      for (int g = 0; g < 4; ++g) {
        f32x4 y; y[0] = oacc[b][4 * g]; y[1] = oacc[b][4 * g + 1]; y[2] = oacc[b][4 * g + 2]; y[3] = oacc[b][4 * g + 3];
        *(f32x4*)(part + lq * PS + 32 * b + 8 * g + 4 * lh) = y;
      }
    if (lh == 0) { part[32 * PS + 2 * lq] = m_run; part[32 * PS + 2 * lq + 1] = l; }
  }
  __syncthreads();
  for (int idx = tid; idx < 32 * (D / 8); idx += NT) {
    const int row = idx / (D / 8), c8 = (idx % (D / 8)) * 8;
    if (q0 + row >= SQ) continue;
    float m = -__builtin_inff();
    #pragma unroll
    for (int g = 0; g < KVS; ++g) m = fmaxf(m, ((const float*)lds)[g * PART + 32 * PS + 2 * row]);
    const float m_use = m == -__builtin_inff() ? 0.0f : m;
    float l = 0.0f;
    float acc[8];
    #pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = 0.0f;
    #pragma unroll
    for (int g = 0; g < KVS; ++g) {
      const float* part = (const float*)lds + g * PART;
      const float w = EXP2(part[32 * PS + 2 * row] - m_use);
      l += part[32 * PS + 2 * row + 1] * w;
      const f32x4 t0 = *(const f32x4*)(part + row * PS + c8), t1 = *(const f32x4*)(part + row * PS + c8 + 4);
      #pragma unroll
      for (int e = 0; e < 4; ++e) { acc[e] += t0[e] * w; acc[4 + e] += t1[e] * w; }
    }
    const float inv = 1.0f / l;
    FRAG y;
    #pragma unroll
    for (int e = 0; e < 8; ++e) y[e] = (ELT)(acc[e] * inv);
    *(FRAG*)(Op + O_OFF + (long)batch * O_SB + (long)head * O_SH + (long)(q0 + row) * O_SS + c8) = y;
  }
}
"""


def pv_supported(body: Flash) -> str | None:
    """Why ``body`` cannot take this form (``None``: it can): 16-bit operands, head_dim 64 or 128 with nothing padded,
    every row on a 16-byte boundary at every size a symbolic stride can take."""
    if body.dtype.name not in ("bf16", "f16"):
        return "16-bit operands"
    if body.head_dim not in HEAD_DIMS or body.head_dim_real not in (None, body.head_dim):
        return f"head_dim {' or '.join(map(str, HEAD_DIMS))} with whole rows"
    if body.kv_ctas > 1 or body.partials is not None:
        return "no key split across workgroups"
    sym = getattr(body, "sym", None)
    symf = sym.fields if sym is not None else {}
    for field, offset, heads in (("q_strides", body.q_offset, body.q_heads), ("k_strides", body.k_offset, body.kv_heads), ("v_strides", body.v_offset, body.kv_heads), ("o_strides", body.o_offset, body.q_heads)):
        vals = [symf.get(f"{field}.2", getattr(body, field)[2]), offset]
        vals += [symf.get(f"{field}.1", getattr(body, field)[1])] if heads > 1 else []
        vals += [symf.get(f"{field}.0", getattr(body, field)[0])] if body.batch > 1 else []
        if not all((v.a % 8 == 0 and v.b % 8 == 0) if isinstance(v, Affine) else (isinstance(v, int) and v % 8 == 0) for v in vals):
            return "rows on 16-byte boundaries"
    return None


def emit_flash_pv(body: Flash, name: str, ctx: Context = Context()) -> HipOp:
    why = pv_supported(body)
    if why is not None:
        raise LoweringError(f"flash (key-split waves): needs {why}")
    if body.q_heads % body.kv_heads:
        raise LoweringError("flash: q heads must be a multiple of kv heads")
    kvs = body.kv_split
    if body.waves != 1 or kvs not in (2, 4, 8) or body.pair or body.ws or body.sp or body.mfma_sum or body.deep:
        raise LoweringError(f"flash (key-split waves): w{body.waves}/s{kvs} is not one row group of 2, 4 or 8 waves, or carries a flag of the shared forms")
    D = body.head_dim
    lds = lds_bytes(D, kvs)
    if lds > ctx.lds_bytes_per_cu:
        raise LoweringError(f"flash (key-split waves): {lds} B of LDS exceeds {ctx.lds_bytes_per_cu} B per CU")
    sym = getattr(body, "sym", None)
    symf = sym.fields if sym is not None else {}
    for key in symf:
        if key not in ("q_len", "kv_len") and not (key.split(".")[0] in ("q_strides", "k_strides", "v_strides", "o_strides", "mask_strides") and key.split(".")[1] in ("0", "1", "2")):
            raise LoweringError(f"flash: {key} cannot follow a symbolic axis")

    def stride(field: str, i: int):
        return symf.get(f"{field}.{i}", getattr(body, field)[i])

    has_mask = body.mask is not None
    if has_mask and body.mask_dtype.name not in ("bf16", "f16", "f32"):
        raise LoweringError("flash: the mask must be a floating-point tensor")
    bf16 = body.dtype.name == "bf16"
    NT = 64 * kvs
    defs = {
        "KNAME": name, "NT": NT, "KVS": kvs, "D": D,
        "ELT": rt.type_name(body.dtype.name), "FRAG": rt.vector_type(body.dtype.name, 8)[0],
        "MFMA": "__builtin_amdgcn_mfma_f32_32x32x16_bf16" if bf16 else "__builtin_amdgcn_mfma_f32_32x32x16_f16",
        "EXP2": rt.intrinsic("fast_exp2", "f32"),
        "SQ": c_value(symf.get("q_len", body.q_len)), "SKV": c_value(symf.get("kv_len", body.kv_len)),
        "HQ": body.q_heads, "GROUP": body.q_heads // body.kv_heads, "CAUSAL": int(bool(body.causal)), "XCDS": ctx.xcds,
        "SCALE_LOG2": float_literal(body.scale * math.log2(math.e)),
        "SYM_PARAM": f", int {param_name(sym.name)}" if symf else "",
        "HAS_MASK": int(has_mask),
        "MASK_PARAM": f", const {rt.type_name(body.mask_dtype.name)}* __restrict__ Mp" if has_mask else "",
        **({"MELT": rt.type_name(body.mask_dtype.name), "M_SB": c_value(stride("mask_strides", 0)), "M_SH": c_value(stride("mask_strides", 1)),
            "M_SS": c_value(stride("mask_strides", 2)), "M_OFF": body.mask_offset} if has_mask else {}),
        "Q_SB": c_value(stride("q_strides", 0)), "Q_SH": c_value(stride("q_strides", 1)), "Q_SS": c_value(stride("q_strides", 2)), "Q_OFF": body.q_offset,
        "K_SB": c_value(stride("k_strides", 0)), "K_SH": c_value(stride("k_strides", 1)), "K_SS": c_value(stride("k_strides", 2)), "K_OFF": body.k_offset,
        "V_SB": c_value(stride("v_strides", 0)), "V_SH": c_value(stride("v_strides", 1)), "V_SS": c_value(stride("v_strides", 2)), "V_OFF": body.v_offset,
        "O_SB": c_value(stride("o_strides", 0)), "O_SH": c_value(stride("o_strides", 1)), "O_SS": c_value(stride("o_strides", 2)), "O_OFF": body.o_offset,
    }  # fmt: skip
    head = f"// {name}: key-split waves B={body.batch} Hq={body.q_heads} Hkv={body.kv_heads} Sq={body.q_len} Skv={body.kv_len} D={D} causal={body.causal}\n"
    head += "".join(f"#define {k} {v}\n" for k, v in defs.items())
    qblocks = -(-body.q_len // 32)
    return HipOp(
        kernel_source=prelude.header(prelude.DMA) + head + _SRC,
        kernel_name=name,
        arg_order=(body.q, body.k, body.v, *((body.mask,) if has_mask else ()), body.out),
        grid=((CeilDiv(symf["q_len"], 32), body.q_heads * body.batch) if "q_len" in symf else (qblocks * body.q_heads * body.batch,), (1,), (1,)),
        block=((NT,), (1,), (1,)),
        lds_bytes=lds,
        runtime_args=(sym.name,) if symf else (),
        comment=f"flash key-split waves Sq={body.q_len} Skv={body.kv_len} D={D} causal={body.causal} split={kvs}",
        algo_bytes=body.algo_bytes(),
        algo_flops=body.algo_flops(),
        knobs={"FLASH": f"w1/kv32/s{kvs}/pv"},
    )


__all__ = ["emit_flash_pv", "pv_supported", "lds_bytes", "max_key_split", "HEAD_DIMS"]
