"""Fused attention emitter: ``softmax(q k^T * scale + causal) v`` on MFMA.

Stands where the reference's warp-flash realisation stands
(``realize_warp_twist``, emmy/compiler/pipeline/passes/lowering/kernel/_twist.py:229-363;
fragment softmax ``FragmentApply/RowReduce/Mask``, emmy/compiler/ir/kernel/ir.py:791-984;
GQA ``head // group`` and causal ``Select(kv <= m)``, passes/lowering/tile/_flash.py:116-125)
and keeps its streaming algebra — statistics start at ``m = -1e30, l = 0``;
per key block ``mn = max(m, rowmax)``, ``alpha = exp(m - mn)``, ``p = exp(s - mn)``,
``l = l*alpha + sum p``, ``O = O*alpha + p v``; the close is ``O / l`` — but the
kernel is laid out for CDNA4:

* Scores are computed **transposed**, ``S^T = K Q^T``.  In the 32x32 MFMA
  accumulator layout a lane then owns *one query* (its column) and 16 of the
  32 keys (its rows), so row max / row sum are in-lane loops plus a single
  exchange with lane ``l ^ 32``, and the rescale factor ``alpha`` is one scalar per
  lane for all of its ``O`` registers.  (The reference needs 4-lane butterflies
  per row on ``m16n8`` fragments, ir.py:733-787.)
* ``P`` never leaves registers: the accumulator registers of ``S^T`` *are* the B
  operand of ``O^T = V^T P^T`` after a bf16 convert, under a fixed permutation of
  the 16 keys of an MFMA step that is applied identically to the ``V`` operand
  (a contraction does not care in which order its terms are summed).  The
  reference round-trips ``P`` through shared memory (``flash_pv_smem``, _twist.py:324-330).
* ``V`` stays ``[key][d]`` in LDS; the A operand is gathered with 8-byte reads of
  four consecutive ``d`` and a register transpose, which assigns output rows
  ``d = 4*m + T`` to MFMA tile ``T`` — again a fixed permutation, undone when
  storing.
* One workgroup = ``waves`` waves x 32 query rows; K/V blocks of 64 keys are
  staged in LDS (K XOR-swizzled for conflict-free 16-byte fragment reads) and
  prefetched through registers one block ahead.  Causal workgroups stop at the
  diagonal and are launched heaviest-first.
"""

from __future__ import annotations

import math

from deplodock_amd.context import Context
from deplodock_amd.emit import prelude
from deplodock_amd.emit.errors import LoweringError
from deplodock_amd.ir.expr import float_literal
from deplodock_amd.ir.hip import HipOp
from deplodock_amd.ir.tile import Flash

_SRC = r"""
EMH_DEV int emh_kswz(int row, int c) { return c ^ (row % CPR); }
EMH_DEV float emh_xor32(float v) { return __shfl_xor(v, 32, 64); }

extern "C" __global__ __launch_bounds__(NT) void KNAME(const ELT* __restrict__ Q, const ELT* __restrict__ Kp,
                                                      const ELT* __restrict__ Vp, ELT* __restrict__ Op) {
  __shared__ __attribute__((aligned(16))) unsigned char lds[2 * 2 * BKV * D * 2];  // [buf][K|V][key][d]
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  const int lq = lane % 32, lh = lane / 32;
  // Heaviest (latest) query blocks first: causal work grows with the block index.
  const int qb = (QBLOCKS - 1) - (int)(blockIdx.x % QBLOCKS);
  const int head = (blockIdx.x / QBLOCKS) % HQ;
  const int batch = blockIdx.x / (QBLOCKS * HQ);
  const int kvh = head / GROUP;
  const int q0 = qb * BQ;            // first query row of the workgroup
  const int qw0 = q0 + wave * 32;    // first query row of this wave
  const int qrow = qw0 + lq;         // this lane's query row
  const ELT* qbase = Q + Q_OFF + (long)batch * Q_SB + (long)head * Q_SH;
  const ELT* kbase = Kp + K_OFF + (long)batch * K_SB + (long)kvh * K_SH;
  const ELT* vbase = Vp + V_OFF + (long)batch * V_SB + (long)kvh * V_SH;

  // Q fragments (B operand of S^T = K Q^T): lane (q = l%32, h = l/32) holds
  // q[qrow][16*kk + 8*h .. +8] for every k-step kk.
  FRAG qf[D / 16];
  {
    const int qr = qrow < SQ ? qrow : SQ - 1;
    const ELT* qp = qbase + (long)qr * Q_SS + 8 * lh;
    #pragma unroll
    for (int kk = 0; kk < D / 16; ++kk) qf[kk] = *(const FRAG*)(qp + 16 * kk);
  }

  // Number of key blocks this workgroup visits.
  int ntiles = (SKV + BKV - 1) / BKV;
  if (CAUSAL) {
    const int lim = (q0 + BQ - 1 < SQ - 1 ? q0 + BQ - 1 : SQ - 1) / BKV + 1;  // last block touching the diagonal
    if (lim < ntiles) ntiles = lim;
  }

  // Staging: K and V blocks are BKV x D elements = BKV*D/8 16-byte chunks each.
  constexpr int CHUNKS = BKV * D / 8;
  constexpr int PER_T = CHUNKS / NT;
  u32x4 rk[PER_T], rv[PER_T];
  #define EMH_GLOAD(jt) { \
    _Pragma("unroll") for (int i = 0; i < PER_T; ++i) { \
      const int q_ = tid + i * NT; const int row_ = q_ / CPR, c_ = q_ % CPR; \
      int kr_ = (jt) * BKV + row_; if (kr_ > SKV - 1) kr_ = SKV - 1; \
      rk[i] = *(const u32x4*)(kbase + (long)kr_ * K_SS + c_ * 8); \
      rv[i] = *(const u32x4*)(vbase + (long)kr_ * V_SS + c_ * 8); } }
  #define EMH_LSTORE(buf) { \
    unsigned char* sk_ = lds + (buf) * (2 * BKV * D * 2); unsigned char* sv_ = sk_ + BKV * D * 2; \
    _Pragma("unroll") for (int i = 0; i < PER_T; ++i) { \
      const int q_ = tid + i * NT; const int row_ = q_ / CPR, c_ = q_ % CPR; \
      *(u32x4*)(sk_ + row_ * (D * 2) + emh_kswz(row_, c_) * 16) = rk[i]; \
      *(u32x4*)(sv_ + row_ * (D * 2) + c_ * 16) = rv[i]; } }

  f32x16 oacc[D / 32];
  #pragma unroll
  for (int t = 0; t < D / 32; ++t)
  #pragma unroll
  for (int r = 0; r < 16; ++r) oacc[t][r] = 0.0f;
  float m_run = -1.0e30f, l_run = 0.0f;

  EMH_GLOAD(0);
  EMH_LSTORE(0);
  __syncthreads();

  for (int jt = 0; jt < ntiles; ++jt) {
    const int cur = jt & 1;
    if (jt + 1 < ntiles) EMH_GLOAD(jt + 1);
    const int k0 = jt * BKV;
    // A wave whose rows all lie above this key block has nothing to add (causal).
    const bool active = !CAUSAL || (k0 <= qw0 + 31);
    if (active) {
      const unsigned char* sK = lds + cur * (2 * BKV * D * 2);
      const unsigned char* sV = sK + BKV * D * 2;
      // ---- S^T = K Q^T for BKV/32 sub-blocks of 32 keys ----
      f32x16 sacc[BKV / 32];
      #pragma unroll
      for (int u = 0; u < BKV / 32; ++u) {
        #pragma unroll
        for (int r = 0; r < 16; ++r) sacc[u][r] = 0.0f;
        const int krow = u * 32 + lq;
        #pragma unroll
        for (int kk = 0; kk < D / 16; ++kk) {
          const FRAG kf = *(const FRAG*)(sK + krow * (D * 2) + emh_kswz(krow, kk * 2 + lh) * 16);
          sacc[u] = MFMA(kf, qf[kk], sacc[u], 0, 0, 0);
        }
      }
      // ---- scale (log2 domain), mask, running max ----
      // Register r of sub-block u is key k0 + 32u + 8*(r/4) + 4*lh + r%4 for query qrow.
      const bool need_mask = (CAUSAL && (k0 + BKV - 1 > qw0)) || (k0 + BKV > SKV);
      float mx = -1.0e30f;
      #pragma unroll
      for (int u = 0; u < BKV / 32; ++u)
      #pragma unroll
      for (int r = 0; r < 16; ++r) {
        float s = sacc[u][r] * SCALE_LOG2;
        if (need_mask) {
          const int key = k0 + 32 * u + 8 * (r / 4) + 4 * lh + (r % 4);
          if ((CAUSAL && key > qrow) || key >= SKV) s = -1.0e30f;
        }
        sacc[u][r] = s;
        mx = fmaxf(mx, s);
      }
      mx = fmaxf(mx, emh_xor32(mx));  // the other half of this query's keys lives in lane l^32
      const float m_new = fmaxf(m_run, mx);
      const float alpha = EXP2(m_run - m_new);
      m_run = m_new;
      float psum = 0.0f;
      #pragma unroll
      for (int u = 0; u < BKV / 32; ++u)
      #pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float p = EXP2(sacc[u][r] - m_new);
        sacc[u][r] = p;
        psum += p;
      }
      l_run = l_run * alpha + psum;  // per-lane partial over this lane's keys; halves meet at the end
      #pragma unroll
      for (int t = 0; t < D / 32; ++t)
      #pragma unroll
      for (int r = 0; r < 16; ++r) oacc[t][r] *= alpha;
      // ---- O^T += V^T P^T ----
      // MFMA step (u, s) contracts 16 keys.  Operand slot (h, t) of that step is
      // key 32u + 16s + 4h + t (t < 4) or 32u + 16s + 8 + 4h + (t - 4): exactly the
      // keys whose probabilities this lane already holds in sacc[u][8s .. 8s+7].
      #pragma unroll
      for (int u = 0; u < BKV / 32; ++u)
      #pragma unroll
      for (int s = 0; s < 2; ++s) {
        FRAG pf;
        #pragma unroll
        for (int t = 0; t < 8; ++t) pf[t] = (ELT)sacc[u][8 * s + t];
        // Gather V: for each of the 8 keys, 4 consecutive d (= 4*lq .. 4*lq+3) per 32-wide tile group.
        #pragma unroll
        for (int dg = 0; dg < D / 128 + (D % 128 ? 1 : 0); ++dg) {
          u32x2 vr[8];
          #pragma unroll
          for (int t = 0; t < 8; ++t) {
            const int key = 32 * u + 16 * s + 4 * lh + (t < 4 ? t : t + 4);
            vr[t] = *(const u32x2*)(sV + key * (D * 2) + dg * 256 + lq * 8);
          }
          // Register transpose 8 keys x 4 d -> 4 fragments of 8 keys.
          #pragma unroll
          for (int T = 0; T < 4; ++T) {
            if (dg * 4 + T >= D / 32) continue;
            u32x4 av;
            #pragma unroll
            for (int w = 0; w < 4; ++w) {
              const unsigned lo = vr[2 * w][T / 2], hi = vr[2 * w + 1][T / 2];
              av[w] = (T % 2 == 0) ? __builtin_amdgcn_perm(hi, lo, 0x05040100u) : __builtin_amdgcn_perm(hi, lo, 0x07060302u);
            }
            oacc[dg * 4 + T] = MFMA(__builtin_bit_cast(FRAG, av), pf, oacc[dg * 4 + T], 0, 0, 0);
          }
        }
      }
    }
    if (jt + 1 < ntiles) EMH_LSTORE((jt + 1) & 1);
    __syncthreads();
  }

  // ---- close: O / l, undo the d permutation, store ----
  const float l_tot = l_run + emh_xor32(l_run);
  const float inv = 1.0f / l_tot;
  if (qrow < SQ) {
    ELT* op = Op + O_OFF + (long)batch * O_SB + (long)head * O_SH + (long)qrow * O_SS;
    // Tile T = 4*dg + Tl, register r = 4*i + j holds d = 128*dg + 4*(8*i + 4*lh + j) + Tl.
    #pragma unroll
    for (int dg = 0; dg < D / 128 + (D % 128 ? 1 : 0); ++dg)
    #pragma unroll
    for (int i = 0; i < 4; ++i)
    #pragma unroll
    for (int j = 0; j < 4; ++j) {
      PACK4 y;
      #pragma unroll
      for (int Tl = 0; Tl < 4; ++Tl) {
        const int T = dg * 4 + Tl;
        y[Tl] = (T < D / 32) ? (ELT)(oacc[T < D / 32 ? T : 0][4 * i + j] * inv) : (ELT)0.0f;
      }
      const int d = 128 * dg + 4 * (8 * i + 4 * lh + j);
      if (d < D) *(PACK4*)(op + d) = y;
    }
  }
}
"""


def emit_flash(body: Flash, name: str, ctx: Context = Context()) -> HipOp:
    D = body.head_dim
    if body.dtype.name not in ("bf16", "f16"):
        raise LoweringError("flash: MFMA tier needs 16-bit operands")
    if D % 128 or D > 256:
        raise LoweringError(f"flash: head_dim {D} must be 128 or 256 on this tier")
    if body.q_heads % body.kv_heads:
        raise LoweringError("flash: q heads must be a multiple of kv heads")
    waves = body.waves
    BQ = 32 * waves
    BKV = body.block_kv
    if BKV % 32 or BKV < 32:
        raise LoweringError("flash: key block must be a multiple of 32")
    NT = waves * 64
    if (BKV * D // 8) % NT:
        raise LoweringError("flash: key block does not divide over the workgroup's threads")
    lds = 2 * 2 * BKV * D * 2
    if lds > ctx.static_lds_cap:
        raise LoweringError(f"flash: {lds} B of LDS exceeds the static cap {ctx.static_lds_cap}")
    for st in (body.q_strides, body.k_strides, body.v_strides):
        if st[2] % 8:
            raise LoweringError("flash: sequence strides must keep 16-byte row alignment")
    if body.o_strides[2] % 4 or any(o % 8 for o in (body.q_offset, body.k_offset, body.v_offset)) or body.o_offset % 4:
        raise LoweringError("flash: offsets / output stride break vector alignment")
    qblocks = -(-body.q_len // BQ)
    bf16 = body.dtype.name == "bf16"
    defs = {
        "KNAME": name,
        "NT": NT,
        "D": D,
        "BQ": BQ,
        "BKV": BKV,
        "CPR": D // 8,
        "SQ": body.q_len,
        "SKV": body.kv_len,
        "HQ": body.q_heads,
        "GROUP": body.q_heads // body.kv_heads,
        "QBLOCKS": qblocks,
        "CAUSAL": 1 if body.causal else 0,
        "SCALE_LOG2": float_literal(body.scale * math.log2(math.e)),
        "Q_SB": body.q_strides[0], "Q_SH": body.q_strides[1], "Q_SS": body.q_strides[2], "Q_OFF": body.q_offset,
        "K_SB": body.k_strides[0], "K_SH": body.k_strides[1], "K_SS": body.k_strides[2], "K_OFF": body.k_offset,
        "V_SB": body.v_strides[0], "V_SH": body.v_strides[1], "V_SS": body.v_strides[2], "V_OFF": body.v_offset,
        "O_SB": body.o_strides[0], "O_SH": body.o_strides[1], "O_SS": body.o_strides[2], "O_OFF": body.o_offset,
        "ELT": "__bf16" if bf16 else "_Float16",
        "FRAG": "bf16x8" if bf16 else "f16x8",
        "PACK4": "bf16x4" if bf16 else "f16x4",
        "MFMA": "__builtin_amdgcn_mfma_f32_32x32x16_bf16" if bf16 else "__builtin_amdgcn_mfma_f32_32x32x16_f16",
        # 2^x straight on the transcendental unit; inputs are <= 0 and the result
        # feeds a 16-bit operand, so the fast form loses nothing that survives.
        "EXP2": "__builtin_amdgcn_exp2f",
    }  # fmt: skip
    head = f"// {name}: B={body.batch} Hq={body.q_heads} Hkv={body.kv_heads} Sq={body.q_len} Skv={body.kv_len} D={D} causal={body.causal}\n"
    head += "".join(f"#define {k} {v}\n" for k, v in defs.items())
    source = prelude.header() + head + _SRC
    grid = qblocks * body.q_heads * body.batch
    return HipOp(
        kernel_source=source,
        kernel_name=name,
        arg_order=(body.q, body.k, body.v, body.out),
        grid=((grid,), (1,), (1,)),
        block=((NT,), (1,), (1,)),
        lds_bytes=0,
        comment=f"flash Sq={body.q_len} Skv={body.kv_len} D={D} causal={body.causal} waves={waves} bkv={BKV}",
        algo_bytes=body.algo_bytes(),
        algo_flops=body.algo_flops(),
        knobs={"FLASH": f"w{waves}/kv{BKV}"},
    )
