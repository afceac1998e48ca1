"""Streaming attention on fp32 MFMA atoms: ``softmax(q k^T * scale + mask) v`` for fp32 operands, and for 16-bit
operands whose rows are not whole 16-byte chunks (converted to fp32 as they are staged).

fp32 is the precision the reference compiles (tests/perf/cases.py:20-23, its ``sdpa`` cases ``:174-190``); it reaches a
streaming kernel by decomposing the fused op and finding the online ``(m, l, O)`` carrier again
(emmy/compiler/pipeline/passes/frontend/decomposition/010_sdpa.py:53-138, passes/lowering/tile/_flash.py:116-125,
passes/lowering/kernel/_twist.py:229-363).  This emitter keeps that algebra — per key block ``mn = max(m, rowmax)``,
``alpha = exp(m - mn)``, ``p = exp(s - mn)``, ``l = l*alpha + sum p``, ``O = O*alpha + p v``, close ``O / l`` — so the scores
never reach device memory, and lays it out the way the 16-bit kernel is:

* ``S^T = K Q^T`` on ``v_mfma_f32_32x32x2_f32`` (full fp32 products and sums): a lane owns one query (its accumulator
  column) and 16 of a block's 32 keys, so row maximum and row sum are in-lane loops plus one exchange with lane
  ``l ^ 32``, and ``alpha`` is one scalar per lane.
* ``P`` stays in registers: accumulator register ``r`` of a lane in half ``h`` is key ``8 (r / 4) + r % 4 + 4 h`` of its
  query, which is exactly the B operand of the atom ``O^T += V^T[.., {key, key + 4}] P^T`` — sixteen atoms per 32 output
  columns walk the block's keys in that order, and the V operand is read from LDS in the same order.
* The contraction over ``d`` in the scores is order-free as well: a lane reads 16 bytes of its key's row per four atoms
  (``d = 8 u + 4 h + 0..3``) and holds its query's values in the same order.
* Two forms.  *Key-split* (``kv_split`` = 2, 4 or 8; rows of whole aligned pairs of 16-byte chunks, up to 128 columns):
  a workgroup is one group of 32 query rows whose waves each take every k-th 32-key block and stage it themselves with
  direct-to-LDS loads — no barrier in the loop, one merge of the waves' ``(m, l, O)`` through LDS at the close.  By
  default a wave's K block and V block take turns in one LDS region (``one_region``: they are never needed at the same
  time), which halves a wave's LDS so that a SIMD holds two waves and one's atoms fill the other's waits.  *Shared*
  (everything else): 256 threads per workgroup, ``waves`` of them (1, 2 or 4) own 32 query rows each, all of them stage
  the 32-key K / V blocks (global -> registers -> LDS, two buffers, one barrier a step; up to 128 columns the loads are
  issued a step ahead of the arithmetic); K rows are padded by 4 floats and V rows by 8, which makes the 16-byte K
  reads and the 4-byte V reads of a wave conflict-free.
* Rows of any length up to 256 values: the tiles are ``DP`` = the next multiple of 32 wide, columns past the row's end are
  staged as zeros and not stored; rows that are not whole aligned 16-byte chunks are read value by value.
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

MAX_HEAD_DIM = 256
THREADS = 256
BLOCK_KV = 32


def padded_head_dim(d: int) -> int:
    return -(-d // 32) * 32


def lds_bytes(head_dim: int) -> int:
    dp = padded_head_dim(head_dim)
    return 2 * BLOCK_KV * ((dp + 4) + (dp + 8)) * 4


_SOFTMAX = r"""      // register r: key k0 + 8 (r / 4) + 4 h + r % 4 of query qrow, in log2 units from here on
      float mx = -__builtin_inff();
      #pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int key = k0 + 8 * (r / 4) + 4 * h + (r % 4);
        float v = s[r] * SCALE_LOG2;
#if HAS_MASK
        v += (float)mrow[key < SKV ? key : SKV - 1] * 1.4426950408889634f;
#endif
        if (key >= SKV || (CAUSAL && key > qrow)) v = -__builtin_inff();
        s[r] = v;
        mx = fmaxf(mx, v);
      }
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      // The reference maximum is raised only when a row outgrows it by 2^8 (probabilities stay below 2^8, far inside
      // fp32 range), so the rescale of the accumulators is rare.
      const bool raise = mx > m_run + 8.0f;  // (from -inf any finite maximum raises; a block of masked keys never does)
      if (__any(raise)) {
        const float alpha = raise ? exp2f(m_run - mx) : 1.0f;
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
      for (int r = 0; r < 16; ++r) { s[r] = exp2f(s[r] - m_use); lsum += s[r]; }
      l_run += lsum;
"""

_SRC = r"""
#define KS (DP + 4)                    /* floats per K row in LDS */
#define VS (DP + 8)                    /* floats per V row in LDS */
#define BUF (BKV * KS + BKV * VS)      /* floats per buffer */
#define CPR (DP / 4)                   /* 16-byte chunks per staged row */
#define NCH (BKV * CPR / NT)           /* chunks of a K (or V) block per thread */
#define NDB (DP / 32)                  /* 32-column blocks of the output */

// Four values of a row starting at column c (a multiple of 4): one 16-byte load where rows are whole aligned chunks,
// else value by value; columns at or past the row's end read as zero.
EMH_DEV f32x4 emh_row4(const ELT* __restrict__ row, int c) {
  f32x4 r = {0.0f, 0.0f, 0.0f, 0.0f};
#if VEC4
  if (c < DR) r = *(const f32x4*)(row + c);
#else
  #pragma unroll
  for (int i = 0; i < 4; ++i) if (c + i < DR) r[i] = (float)row[c + i];
#endif
  return r;
}

extern "C" __global__ __launch_bounds__(NT) void KNAME(const ELT* __restrict__ Q, const ELT* __restrict__ Kp,
                                                      const ELT* __restrict__ Vp MASK_PARAM, ELT* __restrict__ Op SYM_PARAM) {
  extern __shared__ __attribute__((aligned(16))) float lds[];  // [2 buffers][K: BKV x KS | V: BKV x VS]
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  const int n = lane % 32, h = lane / 32;
  // Workgroup ids go round-robin over the XCDs, each with its own L2: consecutive logical ids (the query blocks of one
  // head, then the next head of the same KV group) are dealt to one XCD, so a KV head's keys and values come out of one L2.
  const int grid = (int)gridDim.x;
  const int bid = grid % XCDS == 0 ? (int)(blockIdx.x % XCDS) * (grid / XCDS) + (int)(blockIdx.x / XCDS) : (int)blockIdx.x;
  const int qblocks = (SQ + BQ - 1) / BQ;
  const int qb = (qblocks - 1) - bid % qblocks;  // under a causal mask the heaviest blocks start first
  const int head = (bid / qblocks) % HQ;
  const int batch = bid / (qblocks * HQ);
  const int kvh = head / GROUP;
  const int q0 = qb * BQ, qw0 = q0 + wave * 32;
  const int qrow = qw0 + n;
  const int qrow_c = qrow < SQ ? qrow : SQ - 1;
  const bool owns_rows = wave < WAVES && qw0 < SQ;  // the other waves of the workgroup only stage

  // A lane's query, in the order the score atoms walk d: atoms 4u .. 4u+3 contract d = 8u + 4h + 0..3.
  float qf[DP / 8][4];
  if (owns_rows) {
    const ELT* qp = Q + Q_OFF + (long)batch * Q_SB + (long)head * Q_SH + (long)qrow_c * Q_SS;
    #pragma unroll
    for (int u = 0; u < DP / 8; ++u) {
      const f32x4 t = emh_row4(qp, 8 * u + 4 * h);
      #pragma unroll
      for (int i = 0; i < 4; ++i) qf[u][i] = t[i];
    }
  }
  const ELT* kbase = Kp + K_OFF + (long)batch * K_SB + (long)kvh * K_SH;
  const ELT* vbase = Vp + V_OFF + (long)batch * V_SB + (long)kvh * V_SH;
#if HAS_MASK
  const MELT* mrow = Mp + M_OFF + (long)batch * M_SB + (long)head * M_SH + (long)qrow_c * M_SS;
#endif

  // keys this workgroup streams: all of them, or up to its last query's diagonal
  int kend = SKV;
  if (CAUSAL) { const int last = (q0 + BQ < SQ ? q0 + BQ : SQ); kend = last < kend ? last : kend; }
  const int steps = (kend + BKV - 1) / BKV;

  f32x16 oacc[NDB];
  #pragma unroll
  for (int b = 0; b < NDB; ++b)
    #pragma unroll
    for (int r = 0; r < 16; ++r) oacc[b][r] = 0.0f;
  float m_run = -__builtin_inff(), l_run = 0.0f;  // l_run: this lane's 16 keys of every block; the halves meet at the close

  f32x4 kreg[NCH], vreg[NCH];
  #define EMH_FETCH(t_) { \
    _Pragma("unroll") for (int c = 0; c < NCH; ++c) { \
      const int idx_ = tid + c * NT, row_ = idx_ / CPR, col_ = (idx_ % CPR) * 4; \
      int key_ = (t_) * BKV + row_; key_ = key_ < SKV ? key_ : SKV - 1;  /* rows past the end repeat the last key: masked below, finite here */ \
      kreg[c] = emh_row4(kbase + (long)key_ * K_SS, col_); \
      vreg[c] = emh_row4(vbase + (long)key_ * V_SS, col_); \
    } }
  #define EMH_PLACE(buf_) { \
    float* kl_ = lds + (buf_) * BUF; float* vl_ = kl_ + BKV * KS; \
    _Pragma("unroll") for (int c = 0; c < NCH; ++c) { \
      const int idx_ = tid + c * NT, row_ = idx_ / CPR, col_ = (idx_ % CPR) * 4; \
      *(f32x4*)(kl_ + row_ * KS + col_) = kreg[c]; \
      *(f32x4*)(vl_ + row_ * VS + col_) = vreg[c]; \
    } }

  EMH_FETCH(0)
  EMH_PLACE(0)
  __syncthreads();
  #pragma unroll 1
  for (int t = 0; t < steps; ++t) {
    const bool more = t + 1 < steps;
    if (PRE && more) EMH_FETCH(t + 1)
    const int k0 = t * BKV;
    // a wave whose rows all lie above this block's first key under the causal mask has nothing in it
    if (owns_rows && !(CAUSAL && k0 > qw0 + 31)) {
      const float* kl = lds + (t & 1) * BUF;
      const float* vl = kl + BKV * KS;
      f32x16 s;
      #pragma unroll
      for (int r = 0; r < 16; ++r) s[r] = 0.0f;
      #pragma unroll
      for (int u = 0; u < DP / 8; ++u) {
        const f32x4 kf = *(const f32x4*)(kl + n * KS + 8 * u + 4 * h);
        #pragma unroll
        for (int i = 0; i < 4; ++i) s = __builtin_amdgcn_mfma_f32_32x32x2f32(kf[i], qf[u][i], s, 0, 0, 0);
      }
@SOFTMAX@      #pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float* vr = vl + (8 * (r / 4) + 4 * h + (r % 4)) * VS + n;
        #pragma unroll
        for (int b = 0; b < NDB; ++b) oacc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(vr[32 * b], s[r], oacc[b], 0, 0, 0);
      }
    }
    if (more) {
      if (!PRE) EMH_FETCH(t + 1)  // wide rows: the staging registers are not held across the step's arithmetic
      EMH_PLACE((t + 1) & 1)
    }
    __syncthreads();
  }

  if (owns_rows && qrow < SQ) {  // lanes n and n + 32 hold the same query: both halves of an exchange are in or out together
    const float l = l_run + __shfl_xor(l_run, 32, 64);
    const float inv = 1.0f / l;
    ELT* op = Op + O_OFF + (long)batch * O_SB + (long)head * O_SH + (long)qrow * O_SS;
    #pragma unroll
    for (int b = 0; b < NDB; ++b)
      #pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int d = 32 * b + 8 * g + 4 * h;  // registers 4g .. 4g+3: output columns d .. d+3 of this lane's query
#if OVEC4
        if (d < DR) { f32x4 y; y[0] = oacc[b][4 * g] * inv; y[1] = oacc[b][4 * g + 1] * inv; y[2] = oacc[b][4 * g + 2] * inv; y[3] = oacc[b][4 * g + 3] * inv; *(f32x4*)(op + d) = y; }
#else
        #pragma unroll
        for (int i = 0; i < 4; ++i) if (d + i < DR) op[d + i] = (ELT)(oacc[b][4 * g + i] * inv);
#endif
      }
  }
}
"""

# The form for short sequences: a workgroup is one group of 32 query rows and KVS waves that split its key blocks
# (wave g takes blocks g, g + KVS, ...), so a launch has KVS times the waves of the shared form.  Nothing is shared
# between the waves until the close: each stages its own K / V blocks with direct-to-LDS loads into its own region (one
# K block, one V block) and needs no barrier — the next K block is requested when the scores are done and lands under
# the softmax and the output atoms, the next V block is requested after the output atoms and lands under the next
# scores.  The (m, l, O) of the waves are merged through LDS with the exp-family combine.
_SRC_PRIVATE = r"""
#define CPRL (DPL / 4)                 /* 16-byte chunks per V row in LDS (DPL: the padded row length, a power of two) */
#define RPR (64 / CPRL)                /* V rows per direct-to-LDS request */
#define NIK (DP / 8)                   /* requests of a wave per K block: 32 rows x two chunks each */
#define NIV (32 / RPR)                 /* requests of a wave per V block: whole rows */
#define NDB (DP / 32)                  /* 32-column blocks of the output */
#if ONE_REGION
#define REGION (32 * DPL)             /* floats of LDS per wave in the loop: its K block and its V block take turns */
#else
#define REGION (32 * DP + 32 * DPL)    /* floats of LDS per wave: its K block, then its V block */
#endif
#define PS (DPL + 4)                   /* floats per row of a wave's partial output at the close */
#define PART (ONE_REGION ? 32 * PS + 64 : REGION)  /* floats between the waves' partials at the close */
// K lies in LDS as [pair of chunks u][row][8 floats]: the 16-byte fragment reads of a wave at one u (row n, half h) are
// 1 KiB in a row, conflict-free, and request u of a block is one lane offset plus 32 bytes x u.  V keeps [row][d] with its
// 128-byte halves swapped between rows r and r + 4, the two rows a 4-byte read touches; the rows of one request share
// that swap, so a request is one of two lane offsets plus a row step.
EMH_DEV int emh_vswz(int row) { return CPRL >= 16 ? ((row >> 2) & 1) << 3 : 0; }
// chunks past the row's end (a head_dim below the tile's width) are fetched from the row's first chunk: finite values
// that never count — q's columns there are zero, and v's only reach output columns that are not stored
EMH_DEV int emh_gchunk(int c) { return c < DR / 4 ? c : 0; }

// (one region a wave: two waves a SIMD is the point, so the register budget is half the file)
#if ONE_REGION
#define EMH_OCCUPANCY __attribute__((amdgpu_waves_per_eu(2)))
#else
#define EMH_OCCUPANCY
#endif
extern "C" __global__ __launch_bounds__(NT) EMH_OCCUPANCY void KNAME(const float* __restrict__ Q, const float* __restrict__ Kp,
                                                      const float* __restrict__ Vp MASK_PARAM, float* __restrict__ Op SYM_PARAM) {
  extern __shared__ __attribute__((aligned(16))) float lds[];  // [KVS waves][K: DP / 8 x 32 x 8 | V: 32 x DPL]
  const int tid = threadIdx.x, lane = tid % 64, grp = __builtin_amdgcn_readfirstlane(tid / 64);
  const int n = lane % 32, h = lane / 32;
  const int grid = (int)gridDim.x;
  const int bid = grid % XCDS == 0 ? (int)(blockIdx.x % XCDS) * (grid / XCDS) + (int)(blockIdx.x / XCDS) : (int)blockIdx.x;
  const int qblocks = (SQ + 31) / 32;
  const int qb = (qblocks - 1) - bid % qblocks;  // under a causal mask the heaviest blocks start first
  const int head = (bid / qblocks) % HQ;
  const int batch = bid / (qblocks * HQ);
  const int kvh = head / GROUP;
  const int q0 = qb * 32;
  const int qrow = q0 + n;
  const int qrow_c = qrow < SQ ? qrow : SQ - 1;

#if KV_CTAS > 1
  // Key split across workgroups: slice blockIdx.y of the keys, [kv0, kv0 + SKV), is this workgroup's whole key range (no
  // mask of either kind in this form, so key indices below are simply relative to the slice); the close leaves the
  // slice's unnormalised output rows, maximum and sum in the workspace for the combine kernel.
  const int kv0 = (int)blockIdx.y * KV_CHUNK;
  const int skv_slice = SKV_ALL - kv0 < KV_CHUNK ? SKV_ALL - kv0 : KV_CHUNK;
  #define SKV skv_slice
#else
  const int kv0 = 0;
#endif
  const float* kbase = Kp + K_OFF + (long)batch * K_SB + (long)kvh * K_SH + (long)kv0 * K_SS;
  const float* vbase = Vp + V_OFF + (long)batch * V_SB + (long)kvh * V_SH + (long)kv0 * V_SS;
#if HAS_MASK
  const MELT* mrow = Mp + M_OFF + (long)batch * M_SB + (long)head * M_SH + (long)qrow_c * M_SS;
#endif
  int kend = SKV;
  if (CAUSAL) { const int last = (q0 + 32 < SQ ? q0 + 32 : SQ); kend = last < kend ? last : kend; }
  const int nblocks = (kend + 31) / 32;

  float* kl = lds + grp * REGION;
  float* vl = ONE_REGION ? kl : kl + 32 * DP;
  const unsigned kl_s = emh_uniform(emh_lds_addr(kl)), vl_s = emh_uniform(emh_lds_addr(vl));
  // Lane offsets of the requests of a block that lies wholly inside the sequence: K request u is rows lane / 2, chunk
  // 2 u + lane % 2; V request i is rows i RPR + lane / CPRL, chunk position lane % CPRL, which holds chunk position ^ swap.
  const unsigned koff = (unsigned)(lane / 2) * (unsigned)(K_SS * 4) + (unsigned)(lane % 2) * 16u;
  const unsigned voff0 = (unsigned)(lane / CPRL) * (unsigned)(V_SS * 4) + (unsigned)emh_gchunk(lane % CPRL) * 16u;
  const unsigned voff1 = (unsigned)(lane / CPRL) * (unsigned)(V_SS * 4) + (unsigned)emh_gchunk((lane % CPRL) ^ 8) * 16u;
  // A block that hangs over the sequence's end repeats the last key in the rows past it (masked below, finite here): per-lane addresses.
  #define EMH_REQUEST_K(j_) { \
    if ((j_) * 32 + 32 <= SKV) { \
      const unsigned char* b_ = emh_uniform(kbase + (long)(j_) * 32 * K_SS); \
      _Pragma("unroll") for (int i = 0; i < NIK; ++i) emh_dma16s(b_ + (2 * i < DR / 4 ? i * 32 : 0), koff, kl_s + i * 1024); \
    } else { \
      _Pragma("unroll") for (int i = 0; i < NIK; ++i) { \
        int key_ = (j_) * 32 + lane / 2; key_ = key_ < SKV ? key_ : SKV - 1; \
        emh_dma16(kbase + (long)key_ * K_SS + (2 * i < DR / 4 ? i * 8 : 0) + (lane % 2) * 4, kl + i * 256); \
      } \
    } }
  #define EMH_REQUEST_V(j_) { \
    if ((j_) * 32 + 32 <= SKV) { \
      const unsigned char* b_ = emh_uniform(vbase + (long)(j_) * 32 * V_SS); \
      _Pragma("unroll") for (int i = 0; i < NIV; ++i) emh_dma16s(b_ + (long)i * RPR * V_SS * 4, emh_vswz(i * RPR) ? voff1 : voff0, vl_s + i * 1024); \
    } else { \
      _Pragma("unroll") for (int i = 0; i < NIV; ++i) { \
        const int row_ = i * RPR + lane / CPRL; \
        int key_ = (j_) * 32 + row_; key_ = key_ < SKV ? key_ : SKV - 1; \
        emh_dma16(vbase + (long)key_ * V_SS + emh_gchunk((lane % CPRL) ^ emh_vswz(row_)) * 4, vl + i * 256); \
      } \
    } }

  f32x16 oacc[NDB];
  #pragma unroll
  for (int b = 0; b < NDB; ++b)
    #pragma unroll
    for (int r = 0; r < 16; ++r) oacc[b][r] = 0.0f;
  float m_run = -__builtin_inff(), l_run = 0.0f;

  if (grp < nblocks) {
    EMH_REQUEST_K(grp)
    if (!ONE_REGION) EMH_REQUEST_V(grp)
  }
  // The query's values, requested behind the first blocks and waited for here, before the loop: a load of the
  // compiler's own still outstanding at the loop's head would make it wait inside the loop, by a count that knows
  // nothing of the requests above and so drains them.
  float qf[DP / 8][4];
  {
    const float* qp = Q + Q_OFF + (long)batch * Q_SB + (long)head * Q_SH + (long)qrow_c * Q_SS;
    #pragma unroll
    for (int u = 0; u < DP / 8; ++u) {
      f32x4 t = {0.0f, 0.0f, 0.0f, 0.0f};
      if (8 * u + 4 * h < DR) t = *(const f32x4*)(qp + 8 * u + 4 * h);
      #pragma unroll
      for (int i = 0; i < 4; ++i) qf[u][i] = t[i];
    }
    #pragma unroll
    for (int u = 0; u < DP / 8; ++u)
      #pragma unroll
      for (int i = 0; i < 4; ++i) asm volatile("" : "+v"(qf[u][i]));
  }
@LOOP@
  // Close: every wave leaves its unnormalised output rows, maximum and sum in LDS; after the barrier the threads of
  // the workgroup each finish 16-byte pieces of the output rows (consecutive threads, consecutive pieces).  Where the
  // partials are wider than the loop's regions they overlap a neighbour's blocks: every wave is done with those first.
  if (ONE_REGION) __syncthreads();
  {
    const float l = l_run + __shfl_xor(l_run, 32, 64);
    float* part = lds + grp * PART;
    #pragma unroll
    for (int b = 0; b < NDB; ++b)
      #pragma unroll
      for (int g = 0; g < 4; ++g) {
        f32x4 y; y[0] = oacc[b][4 * g]; y[1] = oacc[b][4 * g + 1]; y[2] = oacc[b][4 * g + 2]; y[3] = oacc[b][4 * g + 3];
        *(f32x4*)(part + n * PS + 32 * b + 8 * g + 4 * h) = y;
      }
    if (h == 0) { part[32 * PS + 2 * n] = m_run; part[32 * PS + 2 * n + 1] = l; }
  }
  __syncthreads();
  for (int idx = tid; idx < 32 * (DR / 4); idx += NT) {
    const int row = idx / (DR / 4), c4 = (idx % (DR / 4)) * 4;
    if (q0 + row >= SQ) continue;
    float m = -__builtin_inff();
    #pragma unroll
    for (int g = 0; g < KVS; ++g) m = fmaxf(m, lds[g * PART + 32 * PS + 2 * row]);
    const float m_use = m == -__builtin_inff() ? 0.0f : m;
    float l = 0.0f;
    f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
    #pragma unroll
    for (int g = 0; g < KVS; ++g) {
      const float* part = lds + g * PART;
      const float w = exp2f(part[32 * PS + 2 * row] - m_use);
      l += part[32 * PS + 2 * row + 1] * w;
      const f32x4 t = *(const f32x4*)(part + row * PS + c4);
      acc[0] += t[0] * w; acc[1] += t[1] * w; acc[2] += t[2] * w; acc[3] += t[3] * w;
    }
#if KV_CTAS > 1
    float* prow = Op + ((((long)blockIdx.y * BATCH + batch) * HQ + head) * SQ + (q0 + row)) * (D + 4);
    *(f32x4*)(prow + c4) = acc;
    if (c4 == 0) { prow[D] = m; prow[D + 1] = l; }
#else
    const float inv = 1.0f / l;
    f32x4 y; y[0] = acc[0] * inv; y[1] = acc[1] * inv; y[2] = acc[2] * inv; y[3] = acc[3] * inv;
    *(f32x4*)(Op + O_OFF + (long)batch * O_SB + (long)head * O_SH + (long)(q0 + row) * O_SS + c4) = y;
#endif
  }
}
"""

_LOOP_PLAIN = r"""  #pragma unroll 1
  for (int j = grp; j < nblocks; j += KVS) {
    const bool more = j + KVS < nblocks;
    const int k0 = j * 32;
    asm volatile("s_waitcnt vmcnt(%0)" :: "n"(NIV) : "memory");  // this block's K has landed (its V may still be on its way)
    emh_lds_publish(kl);
    f32x16 s;
    #pragma unroll
    for (int r = 0; r < 16; ++r) s[r] = 0.0f;
    {
      const float* kfrag = kl + n * 8 + h * 4;
      #pragma unroll
      for (int u = 0; u < DP / 8; ++u) {
        const f32x4 kf = *(const f32x4*)(kfrag + u * 256);
        #pragma unroll
        for (int i = 0; i < 4; ++i) s = __builtin_amdgcn_mfma_f32_32x32x2f32(kf[i], qf[u][i], s, 0, 0, 0);
      }
    }
    // the K fragments are in registers (the atoms above consumed them): the region takes the next block
    asm volatile("" :: "v"(s[0]) : "memory");
    if (more) EMH_REQUEST_K(j + KVS)
@SOFTMAX@
    if (more) asm volatile("s_waitcnt vmcnt(%0)" :: "n"(NIK) : "memory");  // V of this block (the next K block may be on its way)
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    emh_lds_publish(vl);
    #pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int row = 8 * (r / 4) + 4 * h + (r % 4);
      const float* vr = vl + row * DPL + (n % 4);
      #pragma unroll
      for (int b = 0; b < NDB; ++b) oacc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(vr[((8 * b + n / 4) ^ emh_vswz(row)) * 4], s[r], oacc[b], 0, 0, 0);
    }
    #pragma unroll
    for (int b = 0; b < NDB; ++b) asm volatile("" :: "v"(oacc[b][0]) : "memory");  // every V fragment has been consumed
    if (more) EMH_REQUEST_V(j + KVS)
  }

"""

# One region a wave: its K block and its V block take turns in it.  A wave then waits for each landing in the open —
# the V block is requested when the scores are done and has only the softmax to land under, the next K block is
# requested after the output atoms — but a wave needs half the LDS, so a SIMD holds two of them and one's atoms fill
# the other's waits.
_LOOP_ONE = r"""  #pragma unroll 1
  for (int j = grp; j < nblocks; j += KVS) {
    const bool more = j + KVS < nblocks;
    const int k0 = j * 32;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this block's K has landed: nothing else is on its way
    emh_lds_publish(kl);
    f32x16 s;
    #pragma unroll
    for (int r = 0; r < 16; ++r) s[r] = 0.0f;
    {
      const float* kfrag = kl + n * 8 + h * 4;
      #pragma unroll
      for (int u = 0; u < DP / 8; ++u) {
        const f32x4 kf = *(const f32x4*)(kfrag + u * 256);
        #pragma unroll
        for (int i = 0; i < 4; ++i) s = __builtin_amdgcn_mfma_f32_32x32x2f32(kf[i], qf[u][i], s, 0, 0, 0);
      }
    }
    // the K fragments are in registers (the atoms above consumed them): the region takes this block's V
    asm volatile("" :: "v"(s[0]) : "memory");
    EMH_REQUEST_V(j)
@SOFTMAX@
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    emh_lds_publish(vl);
    #pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int row = 8 * (r / 4) + 4 * h + (r % 4);
      const float* vr = vl + row * DPL + (n % 4);
      #pragma unroll
      for (int b = 0; b < NDB; ++b) oacc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(vr[((8 * b + n / 4) ^ emh_vswz(row)) * 4], s[r], oacc[b], 0, 0, 0);
    }
    #pragma unroll
    for (int b = 0; b < NDB; ++b) asm volatile("" :: "v"(oacc[b][0]) : "memory");  // every V fragment has been consumed
    if (more) EMH_REQUEST_K(j + KVS)
  }

"""

# The software-pipelined order of the key-split form: the output atoms of block t-1 run under the softmax of block t
# (one wave per SIMD: nothing else would fill the matrix pipe while the vector pipe takes exponentials).  Per step:
# scores of block t -> request K(t+1) -> { P(t-1) V(t-1) atoms, interleaved with scale / mask / maximum of block t in
# the first half and its exponentials in the second } -> request V(t) -> rescale (rare) -> P(t) becomes P(t-1).
_PIPE_DEFS = r"""
  #define EMH_SCORES(s_) { \
    _Pragma("unroll") for (int r = 0; r < 16; ++r) s_[r] = 0.0f; \
    const float* kfrag = kl + n * 8 + h * 4; \
    _Pragma("unroll") for (int u = 0; u < DP / 8; ++u) { \
      const f32x4 kf = *(const f32x4*)(kfrag + u * 256); \
      _Pragma("unroll") for (int i = 0; i < 4; ++i) s_ = __builtin_amdgcn_mfma_f32_32x32x2f32(kf[i], qf[u][i], s_, 0, 0, 0); \
    } \
    asm volatile("" :: "v"(s_[0]) : "memory");  /* the K fragments are in registers: the region takes the next block */ }
  #if HAS_MASK
  #define EMH_MASK_TERM(key_) + (float)mrow[(key_) < SKV ? (key_) : SKV - 1] * 1.4426950408889634f
  #else
  #define EMH_MASK_TERM(key_)
  #endif
  // element r of a block's scores: key k0 + 8 (r / 4) + 4 h + r % 4 of query qrow, in log2 units from here on
  #define EMH_SCALE_ONE(s_, r, k0_) { \
    const int key_ = (k0_) + 8 * ((r) / 4) + 4 * h + ((r) % 4); \
    float v_ = s_[r] * SCALE_LOG2 EMH_MASK_TERM(key_); \
    if (key_ >= SKV || (CAUSAL && key_ > qrow)) v_ = -__builtin_inff(); \
    s_[r] = v_; mx = fmaxf(mx, v_); }
  // The reference maximum is raised only when a row outgrows it by 2^8 (probabilities stay below 2^8, far inside fp32
  // range), so the rescale of the accumulators is rare.
  #define EMH_MAX_DONE() { \
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64)); \
    raise = mx > m_run + 8.0f;  /* (from -inf any finite maximum raises; a block of masked keys never does) */ \
    alpha = raise ? exp2f(m_run - mx) : 1.0f; \
    m_run = raise ? mx : m_run; \
    l_run *= alpha; \
    m_use = m_run == -__builtin_inff() ? 0.0f : m_run;  /* nothing but masked keys so far: every term is 0 */ }
  // (the empty asm keeps the exponential where it is written: its result is not needed before the next step's atoms, and
  // the compiler would otherwise sink it out of the atoms' shadow)
  #define EMH_EXP_ONE(s_, r) { s_[r] = exp2f(s_[r] - m_use); asm volatile("" : "+v"(s_[r])); l_run += s_[r]; }
  #define EMH_RESCALE() if (__any(raise)) { \
    _Pragma("unroll") for (int b = 0; b < NDB; ++b) _Pragma("unroll") for (int r = 0; r < 16; ++r) oacc[b][r] *= alpha; }
  #define EMH_V_READ(P, r) { \
    const int row_ = 8 * ((r) / 4) + 4 * h + ((r) % 4); \
    const float* vr_ = vl + row_ * DPL + (n % 4); \
    _Pragma("unroll") for (int b = 0; b < NDB; ++b) vf[P][b] = vr_[((8 * b + n / 4) ^ emh_vswz(row_)) * 4]; }
  #define EMH_PV_MMA(P, p_, r) { \
    _Pragma("unroll") for (int b = 0; b < NDB; ++b) oacc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(vf[P][b], p_[r], oacc[b], 0, 0, 0); }
  #define EMH_V_CONSUMED() { _Pragma("unroll") for (int b = 0; b < NDB; ++b) asm volatile("" :: "v"(oacc[b][0]) : "memory"); }
"""


def _pipelined_loop() -> str:
    o: list[str] = [_PIPE_DEFS]
    a = o.append
    a("  if (grp < nblocks) {")
    a("    f32x16 p, s;")
    a("    float vf[2][NDB];")
    a("    float mx, alpha, m_use; bool raise;")
    a("    // first block: scores and softmax, nothing to overlap yet")
    a('    asm volatile("s_waitcnt vmcnt(%0)" :: "n"(NIV) : "memory");')
    a("    emh_lds_publish(kl);")
    a("    EMH_SCORES(p)")
    a("    if (grp + KVS < nblocks) EMH_REQUEST_K(grp + KVS)")
    a("    mx = -__builtin_inff();")
    for r in range(16):
        a(f"    EMH_SCALE_ONE(p, {r}, grp * 32)")
    a("    EMH_MAX_DONE()")
    for r in range(16):
        a(f"    EMH_EXP_ONE(p, {r})")
    a("    // the accumulators are still zero: a raise from -inf needs no rescale")
    a("    #pragma unroll 1")
    a("    for (int j = grp + KVS; j < nblocks; j += KVS) {")
    a("      const bool more = j + KVS < nblocks;")
    a("      const int k0 = j * 32;")
    a("      // this block's K has landed; the first time round the V block before it is older than it and lands with it")
    a('      if (j == grp + KVS) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");')
    a('      else asm volatile("s_waitcnt vmcnt(%0)" :: "n"(NIV) : "memory");')
    a("      emh_lds_publish(kl);")
    a("      EMH_SCORES(s)")
    a("      if (more) EMH_REQUEST_K(j + KVS)")
    a('      if (more) asm volatile("s_waitcnt vmcnt(%0)" :: "n"(NIK) : "memory");  // V of the block before (the next K block may be on its way)')
    a('      else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");')
    a("      emh_lds_publish(vl);")
    a("      mx = -__builtin_inff();")
    a("      EMH_V_READ(0, 0)")
    for r in range(16):
        # the V fragments of the next key are read before this key's atoms; a step's vector work stays behind its atoms
        if r < 15:
            a(f"      EMH_V_READ({(r + 1) % 2}, {r + 1})")
        a(f"      EMH_PV_MMA({r % 2}, p, {r})")
        if r < 8:
            a(f"      EMH_SCALE_ONE(s, {2 * r}, k0) EMH_SCALE_ONE(s, {2 * r + 1}, k0)")
        if r == 8:
            a("      EMH_MAX_DONE()")
        if r >= 8:
            a(f"      EMH_EXP_ONE(s, {2 * (r - 8)}) EMH_EXP_ONE(s, {2 * (r - 8) + 1})")
        a("      __builtin_amdgcn_sched_barrier(0);")
    a("      EMH_V_CONSUMED()")
    a("      EMH_REQUEST_V(j)")
    a("      EMH_RESCALE()  // the atoms above added P(t-1) V(t-1) relative to the old reference maximum")
    a("      p = s;")
    a("    }")
    a("    // last block: its output atoms")
    a('    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");')
    a("    emh_lds_publish(vl);")
    a("    EMH_V_READ(0, 0)")
    for r in range(16):
        if r < 15:
            a(f"    EMH_V_READ({(r + 1) % 2}, {r + 1})")
        a(f"    EMH_PV_MMA({r % 2}, p, {r})")
    a("  }")
    return "\n".join(o) + "\n"



def f32_supported(head_dim: int) -> bool:
    return 1 <= head_dim <= MAX_HEAD_DIM


def on_f32_atoms(body: Flash) -> bool:
    """Whether ``body`` is this emitter's: fp32 operands, or 16-bit rows that are not whole 16-byte chunks (the 16-bit
    kernel pads whole chunks only), which are converted to fp32 as they are staged."""
    return body.dtype.name == "f32" or (body.dtype.name in ("bf16", "f16") and body.head_dim % 8 != 0 and body.head_dim_real is None)


def emit_flash_f32(body: Flash, name: str, ctx: Context = Context()) -> HipOp:
    D = body.head_dim
    if body.dtype.name not in ("f32", "bf16", "f16"):
        raise LoweringError("flash (fp32 atoms): fp32, bf16 or fp16 operands")
    narrow = body.dtype.name != "f32"  # 16-bit operands (rows the 16-bit kernel has no chunks for): converted as they are staged
    if not f32_supported(D) or body.head_dim_real not in (None, D):
        raise LoweringError(f"flash (fp32 form): head_dim {D} outside 1..{MAX_HEAD_DIM}")
    if body.q_heads % body.kv_heads:
        raise LoweringError("flash: q heads must be a multiple of kv heads")
    if body.pair or body.ws or body.mfma_sum or (body.sp and body.kv_split < 2):
        raise LoweringError("flash (fp32 form): no mirrored pairs; the software-pipelined order is the key-split form's")
    split = int(body.kv_ctas or 1)
    if split > 1:
        sym_ = getattr(body, "sym", None)
        if body.partials is None:
            raise LoweringError("flash: a cross-workgroup key split (REDUCE=g<n>k) is lowered as a partial kernel plus a combine (passes.lower), not by this emitter alone")
        if body.kv_split < 2 or body.causal or body.mask is not None or (sym_ is not None and sym_.fields) or body.dtype.name != "f32" or D % 4:
            raise LoweringError("flash (fp32 form): the cross-workgroup key split is the key-split form's, without masks or symbolic lengths")
        step_keys = body.kv_split * body.block_kv
        kv_chunk = -(-(-(-body.kv_len // split)) // step_keys) * step_keys  # whole key steps per slice
        split = -(-body.kv_len // kv_chunk)  # slices that hold keys
    waves, kvs = body.waves, body.kv_split
    private = kvs > 1
    if (not private and waves not in (1, 2, 4)) or (private and (waves != 1 or kvs not in (2, 4, 8))):
        raise LoweringError(f"flash (fp32 form): w{waves}/s{kvs} is neither 1, 2 or 4 row groups nor one row group of 2, 4 or 8 key-split waves")
    DP = padded_head_dim(D)
    DPL = 1 << (DP - 1).bit_length()
    lds = private_lds_bytes(D, kvs, bool(body.one_region)) if private else lds_bytes(D)
    if lds > ctx.lds_bytes_per_cu:
        raise LoweringError(f"flash (fp32 form): {lds} B of LDS exceeds {ctx.lds_bytes_per_cu} B per CU")
    sym = getattr(body, "sym", None)
    symf = sym.fields if sym is not None else {}
    for key in symf:
        if key not in ("q_len", "kv_len") and not (key.split(".")[0] in ("q_strides", "k_strides", "v_strides", "o_strides", "mask_strides") and key.split(".")[1] in ("0", "1", "2")):
            raise LoweringError(f"flash: {key} cannot follow a symbolic axis")
    vec_in, vec_out = (False, False) if narrow else whole_chunk_rows(body)
    if private and not (vec_in and vec_out and D % 8 == 0):
        raise LoweringError("flash (fp32 form): the key-split form needs rows of whole, aligned pairs of 16-byte chunks")

    def stride(field: str, i: int):
        return symf.get(f"{field}.{i}", getattr(body, field)[i])

    has_mask = body.mask is not None
    if has_mask and body.mask_dtype.name not in ("bf16", "f16", "f32"):
        raise LoweringError("flash: the mask must be a floating-point tensor")
    BQ = 32 * waves
    NT = 64 * kvs if private else THREADS
    defs = {
        "KNAME": name, "ELT": rt.type_name(body.dtype.name), "NT": NT, "WAVES": waves, "KVS": kvs, "BQ": BQ, "BKV": BLOCK_KV, "D": D, "DR": D, "DP": DP, "DPL": DPL,
        "VEC4": int(vec_in), "OVEC4": int(vec_out), "PRE": int(DP <= 128), "ONE_REGION": int(bool(body.one_region) and private),
        "SQ": c_value(symf.get("q_len", body.q_len)),
        **({"SKV_ALL": body.kv_len, "KV_CHUNK": kv_chunk, "BATCH": body.batch} if split > 1 else {"SKV": c_value(symf.get("kv_len", body.kv_len))}),
        "KV_CTAS": split,
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
    head = f"// {name}: fp32 B={body.batch} Hq={body.q_heads} Hkv={body.kv_heads} Sq={body.q_len} Skv={body.kv_len} D={D} causal={body.causal}\n"
    head += "".join(f"#define {k} {v}\n" for k, v in defs.items())
    qblocks = -(-body.q_len // BQ)
    piped = private and bool(body.sp)
    one = private and bool(body.one_region)
    if piped and one:
        raise LoweringError("flash (fp32 form): the software-pipelined order keeps a K and a V block at once")
    src = (_SRC_PRIVATE.replace("@LOOP@", _pipelined_loop() if piped else (_LOOP_ONE if one else _LOOP_PLAIN)) if private else _SRC).replace("@SOFTMAX@", _SOFTMAX)
    return HipOp(
        kernel_source=(prelude.header(prelude.DMA) if private else prelude.header()) + head + src,
        kernel_name=name,
        arg_order=(body.q, body.k, body.v, *((body.mask,) if has_mask else ()), body.partials if split > 1 else body.out),
        grid=((CeilDiv(symf["q_len"], BQ), body.q_heads * body.batch) if "q_len" in symf else (qblocks * body.q_heads * body.batch,), (split,), (1,)),
        block=((NT,), (1,), (1,)),
        lds_bytes=lds,
        runtime_args=(sym.name,) if symf else (),
        comment=f"flash fp32 Sq={body.q_len} Skv={body.kv_len} D={D} causal={body.causal} waves={waves} split={kvs}",
        algo_bytes=body.algo_bytes(),
        algo_flops=body.algo_flops(),
        knobs={"FLASH": (f"f32/s{kvs}" + ("/sp" if piped else "") + ("/o" if one else "")) if private else f"f32/w{waves}", **({"REDUCE": f"g{split}k"} if split > 1 else {})},
    )


def whole_chunk_rows(body: Flash) -> tuple[bool, bool]:
    """``(operands, output)``: whether every row of q / k / v, and of the output, is whole 16-byte chunks on 16-byte
    boundaries — at every size a symbolic stride can take."""
    sym = getattr(body, "sym", None)
    symf = sym.fields if sym is not None else {}

    def ok(field: str, offset: int, heads: int) -> bool:
        vals = [symf.get(f"{field}.2", getattr(body, field)[2]), offset]
        vals += [symf.get(f"{field}.1", getattr(body, field)[1])] if heads > 1 else []
        vals += [symf.get(f"{field}.0", getattr(body, field)[0])] if body.batch > 1 else []
        return all((v.a % 4 == 0 and v.b % 4 == 0) if isinstance(v, Affine) else (isinstance(v, int) and v % 4 == 0) for v in vals)

    whole = body.head_dim % 4 == 0
    return (whole and ok("q_strides", body.q_offset, body.q_heads) and ok("k_strides", body.k_offset, body.kv_heads) and ok("v_strides", body.v_offset, body.kv_heads),
            whole and ok("o_strides", body.o_offset, body.q_heads))  # fmt: skip


def private_lds_bytes(head_dim: int, kvs: int, one_region: bool = False) -> int:
    dp = padded_head_dim(head_dim)
    dpl = 1 << (dp - 1).bit_length()
    if one_region:  # (the partials of the close are a little wider than a block)
        return kvs * (32 * (dpl + 4) + 64) * 4
    return kvs * 32 * (dp + dpl) * 4


def max_key_split(head_dim: int, lds_limit: int, one_region: bool = False) -> int:
    """Most key-split waves (8, 4, 2, or 1 = none) whose private K / V regions fit the LDS; none beyond 128 columns, where
    a wave's query and output registers leave no room for the form's fragments."""
    if padded_head_dim(head_dim) > 128:
        return 1
    return next((k for k in (8, 4, 2) if private_lds_bytes(head_dim, k, one_region) <= lds_limit), 1)


__all__ = ["emit_flash_f32", "f32_supported", "on_f32_atoms", "lds_bytes", "padded_head_dim", "whole_chunk_rows", "max_key_split", "MAX_HEAD_DIM"]
