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
* ``V`` stays ``[key][d]`` in LDS; its operand fragments come from the gfx950
  transposing LDS read (``ds_read_b64_tr_b16``): two reads per fragment, no
  register shuffling.
* One workgroup = ``waves`` groups of 32 query rows x ``kv_split`` wave groups that
  share those rows and split the key blocks between them, so each SIMD hosts
  several waves whose MFMA, LDS and softmax phases overlap in hardware; the
  groups' ``(m, l, O)`` are merged through LDS at the end.  K/V blocks are staged
  with direct-to-LDS loads one step ahead (K XOR-swizzled for conflict-free
  16-byte fragment reads, V swizzled for the transposing reads).
* The exponentials are taken against a reference maximum that is only raised
  when a row outgrows it by 2^8, which makes the accumulator rescale rare; the
  score scale is folded into the exponent's fma.  Causal workgroups stop at the
  diagonal, mask only diagonal blocks, and are launched heaviest-first.
"""

from __future__ import annotations

import math

from deplodock_amd.context import Context
from deplodock_amd.emit import prelude
from deplodock_amd.render_target import rt
from deplodock_amd.emit.errors import LoweringError
from deplodock_amd.ir.expr import float_literal
from deplodock_amd.ir.hip import HipOp
from deplodock_amd.ir.sym import Affine, CeilDiv, c_value, param_name
from deplodock_amd.ir.tile import Flash

# The key range of a workgroup's query rows is split over KVS wave groups.  Group g
# owns key blocks g, g+KVS, ...; the groups hold the same query rows, so every
# SIMD hosts KVS waves whose MFMA, LDS and softmax phases interleave in hardware.
# Each group keeps its own (m, l, O); they are merged through LDS at the end with
# the same exp-family combine the streaming loop uses.  KVS = 1 is the plain form.
_SRC = r"""
// K rows are XOR-swizzled per 256-byte bank line (KRPL rows of it), so the 16 rows
// a fragment read touches at one k position land in 16 different bank groups.
EMH_DEV int emh_kswz(int row, int c) { return c ^ ((row / KRPL) % CPR); }
// V keeps [key][d] order; its 16-byte chunks are XOR-swizzled in groups of four
// so the four consecutive key rows one transposing read touches sit in four
// different bank quarters.
#define EMH_VROT(row) (D >= 128 ? ((row) % 4) : (((row) >> 1) & 1))  /* 128-byte rows: two rows share a bank line */
EMH_DEV int emh_vswz(int row, int c) { return c ^ (EMH_VROT(row) << 2); }
EMH_DEV float emh_xor32(float v) { return __shfl_xor(v, 32, 64); }
// Rows of DR < D values (a head_dim between the kernel's widths): the 16-byte chunks past the row's end are fetched from
// the row's first chunk instead — finite values of the same row — and never count: q's are zeroed in registers, so k's
// vanish in the scores, and v's only reach output columns that are not stored.
EMH_DEV int emh_gchunk(int c) { return (DR == D || c < DR / 8) ? c : 0; }
typedef short emh_s16x4 __attribute__((ext_vector_type(4)));
#define KBYTES (BKV * D * 2)
#define WQ (NT / 64 / KVS)           /* waves (32-row groups) per key-split group */
#define SETB (KVS * KBYTES)          /* one ring slot: the K (or V) blocks of a step, one per key-split group */
#define V_RING (RK * SETB)           /* LDS: [K ring: RK slots][V ring: RV slots] */
#define EMH_SLOT(st, R) ((R) == 2 ? ((st) & 1) : ((st) % (R)))  /* two slots: the step's parity, known when the loop runs in pairs */
#define QCHUNKS (BQ * CPR)             /* 16-byte chunks of a workgroup's Q (and O) tile */
#define RPL (D / 32 * 16)              /* output registers per lane */
#define RPG (RPL / KVS)                /* ... of which each key-split group finishes this many */
#define OSW (D / 4 < 32 ? D / 4 : 32)  /* rows over which the O tile's 8-byte slots are XOR-swizzled */
#define OACC(f) oacc[(f) / 16][(f) % 16]

extern "C" __global__ __launch_bounds__(NT) void KNAME(const ELT* __restrict__ Q, const ELT* __restrict__ Kp,
                                                      const ELT* __restrict__ Vp MASK_PARAM, OUT_T* __restrict__ Op SYM_PARAM) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];  // [2 buffers][group][K | V][key][d]
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  const int grp = wave / WQ, wq = wave % WQ;
  const int lq = lane % 32, lh = lane / 32;
  // PAIR: a workgroup takes query block b from the heavy end and then its
  // mirror from the light end, so under a causal mask every workgroup streams
  // the same number of key blocks (QBLOCKS + 1) whatever b is.
  // Workgroup ids go round-robin over the XCDs, each with its own L2.  Consecutive
  // logical ids (the query blocks of one head, then the next head of the same KV
  // group) are dealt to one XCD, so a KV head's keys and values are fetched from
  // HBM by one L2 instead of by all of them.
  const int bid = GRID % XCDS == 0 ? (int)(blockIdx.x % XCDS) * (GRID / XCDS) + (int)(blockIdx.x / XCDS) : (int)blockIdx.x;
  const int slot = bid % QSLOTS;
  const int head = (bid / QSLOTS) % HQ;
  const int batch = bid / (QSLOTS * HQ);
  const int kvh = head / GROUP;
  const ELT* qbase = Q + Q_OFF + (long)batch * Q_SB + (long)head * Q_SH;
#if KV_CTAS > 1
  // Cross-workgroup key split: slice blockIdx.y of the keys, [kv0, kv0 + SKV), is this workgroup's whole key range.
  // Key indices below are relative to the slice; the causal comparison shifts the query index instead.
  const int kv0 = (int)blockIdx.y * KV_CHUNK;
  const int skv_slice = SKV_ALL - kv0 < KV_CHUNK ? SKV_ALL - kv0 : KV_CHUNK;
  #define SKV skv_slice
  #define QSHIFT kv0
#else
  #define QSHIFT 0
#endif
  const ELT* kbase = Kp + K_OFF + (long)batch * K_SB + (long)kvh * K_SH + (long)QSHIFT * K_SS;
  const ELT* vbase = Vp + V_OFF + (long)batch * V_SB + (long)kvh * V_SH + (long)QSHIFT * V_SS;
  // Measurement build (-DEMH_STAMP=1 or 2 among the compiler options): the first thread of workgroup 0 sums the clocks
  // its key steps spend per phase (1: score phase / softmax / output MFMAs / end-of-step hand-over, averaged per step) or
  // its passes spend per part (2: prologue / key loop / close / store) and leaves four floats in the first 16 bytes it
  // stored itself; the rest of the output is the attention result as usual.
#ifndef EMH_STAMP
#define EMH_STAMP 0
#endif
#define EMH_STAMP_AT(i) if (EMH_STAMP == 1) { const unsigned long long now_ = __builtin_readcyclecounter(); st_acc[i] += (unsigned)(now_ - st_last); st_last = now_; st_acc[4 + (i)] += 1u; }
#define EMH_PHASE_AT(i) if (EMH_STAMP == 2) { const unsigned long long now_ = __builtin_readcyclecounter(); st_acc[i] += (unsigned)(now_ - st_last); st_last = now_; st_acc[4 + (i)] = 1u; }
  unsigned st_acc[8] = {0u, 0u, 0u, 0u, 0u, 0u, 0u, 0u};
  unsigned long long st_last = EMH_STAMP ? __builtin_readcyclecounter() : 0ull;
  #pragma unroll 1
  for (int pass = 0; pass < (PAIR ? 2 : 1); ++pass) {
  if (PAIR && pass) __syncthreads();  // every thread is done copying the first block's O tile out of LDS
  const int qb = pass == 0 ? (QBLOCKS - 1) - slot : slot;
  const int q0 = qb * BQ;
  const int qw0 = q0 + wq * 32;
  const int qrow = qw0 + lq;
  const int qw0_k = qw0 - QSHIFT, qrow_k = qrow - QSHIFT;  // the same rows as positions among this workgroup's keys

  // A lane's Q fragments are 16-byte pieces of one row: read straight from global
  // memory a wave's load touches 32 rows per instruction.  With LDS to spare the
  // tile comes in through the same swizzled direct-to-LDS path as a K block (whole
  // rows per instruction) and the fragments are read from there.
  FRAG qf[D / 16];
  if (Q_LDS) {
    #pragma unroll
    for (int c0 = 0; c0 < QCHUNKS; c0 += NT) {
      if (QCHUNKS % NT == 0 || c0 + (tid - lane) < QCHUNKS) {  // whole waves: QCHUNKS is a multiple of 64
        const int r_ = (c0 + tid) / CPR, p_ = (c0 + tid) % CPR;
        const int qr_ = q0 + r_ < SQ ? q0 + r_ : SQ - 1;
        emh_dma16(qbase + (long)qr_ * Q_SS + emh_gchunk(emh_kswz(r_, p_)) * 8, lds + Q_OFF_LDS + (c0 + tid - lane) * 16);
      }
    }
  } else {
    const int qr = qrow < SQ ? qrow : SQ - 1;
    const ELT* qp = qbase + (long)qr * Q_SS + 8 * lh;
    #pragma unroll
    for (int kk = 0; kk < D / 16; ++kk) qf[kk] = *(const FRAG*)(qp + 8 * (emh_gchunk(2 * kk + lh) - lh));
  }
  int ntiles = (SKV + BKV - 1) / BKV;
  if (CAUSAL) {
    const int last_ = (q0 + BQ - 1 < SQ - 1 ? q0 + BQ - 1 : SQ - 1) - QSHIFT;  // the last key any row of the block may see
    const int lim = last_ < 0 ? 0 : last_ / BKV + 1;
    if (lim < ntiles) ntiles = lim;
  }
  const int nsteps = (ntiles + KVS - 1) / KVS;

  // Direct-to-LDS staging.  A step holds KVS key blocks; their K and V chunks
  // (16 bytes each) are dealt over all threads.  Every wave-level load fills 64
  // consecutive LDS slots, so for K the XOR swizzle is applied by choosing which
  // global chunk each lane fetches.
  constexpr int CHUNKS = BKV * D / 8;          // per block, per operand
  constexpr int PER_T = KVS * CHUNKS / NT;     // chunks per thread, per operand
  // Chunk q = tid + i*NT of a step: block g = q / CHUNKS, row (q % CHUNKS) / CPR,
  // slot q % CPR = tid % CPR.  CHUNKS is a multiple of NT, so g and the row offset
  // of iteration i are compile-time.
  const int st_row = tid / CPR, st_pos = tid % CPR;
  const unsigned lds0 = emh_lds_addr(lds);
  const int wave_u = __builtin_amdgcn_readfirstlane(tid / 64);  // wave-uniform by construction; says so to the compiler
  // A request is a scalar base (the head's K or V plane, moved along the keys per step in scalar registers), a
  // 32-bit lane offset and a scalar LDS target: no vector arithmetic per request.  The lane offsets are the same
  // for every step whose keys all lie inside the sequence.  Only the last step can hang over the end: before its
  // requests are issued EMH_CLAMP_K / _V(st) recomputes the offsets once with each lane's row clamped to the last
  // key (a duplicate row the score mask discards), so the requests themselves never branch on the length.
  unsigned kvo[PER_T], vvo[PER_T];
  #define EMH_LANE_OFFSETS(off_, stride_, swz_, lim_) \
    _Pragma("unroll") for (int i = 0; i < PER_T; ++i) { \
      const int g_ = (i * NT) / CHUNKS, ro_ = ((i * NT) % CHUNKS) / CPR; \
      const int row_ = g_ * BKV + ro_ + st_row; \
      off_[i] = (unsigned)((row_ < (lim_) ? row_ : (lim_)) * (stride_) + emh_gchunk(swz_(st_row + ro_, st_pos)) * 8) * 2u; }
  EMH_LANE_OFFSETS(kvo, K_SS, emh_kswz, 0x7fffffff)
  EMH_LANE_OFFSETS(vvo, V_SS, emh_vswz, 0x7fffffff)
  #define EMH_RAGGED(st) (!WHOLE_STEPS && ((st) + 1) * (KVS * BKV) > SKV)
  #define EMH_CLAMP_K(st) if (EMH_RAGGED(st)) { const int lim_ = SKV - 1 - (st) * (KVS * BKV); EMH_LANE_OFFSETS(kvo, K_SS, emh_kswz, (lim_ < 0 ? 0 : lim_)) }
  #define EMH_CLAMP_V(st) if (EMH_RAGGED(st)) { const int lim_ = SKV - 1 - (st) * (KVS * BKV); EMH_LANE_OFFSETS(vvo, V_SS, emh_vswz, (lim_ < 0 ? 0 : lim_)) }
  // EMH_STEP_BASES(st) names the scalar parts of the requests of step st once (K and V plane bases moved to the
  // step's keys, the ring slots' LDS addresses); EMH_STAGE_K / _V(st, i) then issue request i against them.
  #define EMH_STEP_BASES(tag, st) \
      const unsigned char* kb##tag = emh_uniform((const unsigned char*)kbase + (long)(st) * (KVS * BKV) * K_SS * 2); \
      const unsigned char* vb##tag = emh_uniform((const unsigned char*)vbase + (long)(st) * (KVS * BKV) * V_SS * 2); \
      const unsigned kl##tag = emh_uniform(lds0 + EMH_SLOT(st, RK) * SETB + wave_u * 1024); \
      const unsigned vl##tag = emh_uniform(lds0 + V_RING + EMH_SLOT(st, RV) * SETB + wave_u * 1024);
  #define EMH_STAGE_ONE(st, i, sb_, lb_, off_) { \
      const int g_ = ((i) * NT) / CHUNKS; \
      emh_dma16s(sb_, off_[i], (lb_) + g_ * KBYTES + (((i) * NT) % CHUNKS) * 16); }
  #define EMH_STAGE_K(tag, st, i) EMH_STAGE_ONE(st, i, kb##tag, kl##tag, kvo)
  #define EMH_STAGE_V(tag, st, i) EMH_STAGE_ONE(st, i, vb##tag, vl##tag, vvo)
  // Requests are issued between MFMAs, spread evenly over a chain of NQ_SLOTS of them (request i behind MFMA
  // number EMH_SLOT_OF(i)): they trickle into the memory pipeline instead of arriving as one burst from every wave.
  #define NQ_SLOTS ((BKV / 32) * (D / 16))
  #define EMH_SLOT_OF(i) (((i) * NQ_SLOTS) / PER_T)
  #define EMH_STAGE_ALL_K(st) { EMH_STEP_BASES(_a, st) _Pragma("unroll") for (int i = 0; i < PER_T; ++i) EMH_STAGE_K(_a, st, i) (void)vb_a; (void)vl_a; }
  #define EMH_STAGE_ALL_V(st) { EMH_STEP_BASES(_a, st) _Pragma("unroll") for (int i = 0; i < PER_T; ++i) EMH_STAGE_V(_a, st, i) (void)kb_a; (void)kl_a; }

  // Publishing direct-to-LDS data: the request counter reaching its target does not yet mean the
  // data is visible to other waves' LDS reads (measured: stale reads right after
  // the barrier).  An LDS read of this wave queues behind its own DMA writes, so
  // waiting for that read orders them before the barrier.  Requests retire in issue order: "at most c * PER_T
  // outstanding" means everything issued before the last c request groups has landed.
  #define EMH_WAIT_VM(n) ((((n) & 0xF) | ((((n) >> 4) & 0x3) << 14)) | 0x0070)  /* vmcnt <= n, lgkmcnt = 0 */
  #define EMH_LAND(c) { \
    switch (c) { \
      case 0: __builtin_amdgcn_s_waitcnt(EMH_WAIT_VM(0)); break; \
      case 1: __builtin_amdgcn_s_waitcnt(EMH_WAIT_VM(PER_T)); break; \
      case 2: __builtin_amdgcn_s_waitcnt(EMH_WAIT_VM(2 * PER_T)); break; \
      case 3: __builtin_amdgcn_s_waitcnt(EMH_WAIT_VM(3 * PER_T)); break; \
      default: __builtin_amdgcn_s_waitcnt(EMH_WAIT_VM(4 * PER_T)); break; } \
    emh_lds_publish(lds + tid * 4); \
    __syncthreads(); }

  f32x16 oacc[D / 32];
  #pragma unroll
  for (int t = 0; t < D / 32; ++t)
  #pragma unroll
  for (int r = 0; r < 16; ++r) oacc[t][r] = 0.0f;
  float m_ref = -1.0e30f, l_run = 0.0f;
  // MSUM: the row sums come out of the matrix pipe.  An all-ones A operand against the P fragments the output MFMAs
  // already hold gives, in every row of a 32 x 32 tile, the sum over the 32 keys of each query column (both lane
  // halves included): two MFMAs per 32-key sub-block replace 16 adds per lane, and the sum is of the rounded
  // probabilities the output itself is made of.
  f32x16 lacc;
  FRAG ones_f;
  if (MSUM) {
    #pragma unroll
    for (int r = 0; r < 16; ++r) lacc[r] = 0.0f;
    #pragma unroll
    for (int e = 0; e < 8; ++e) ones_f[e] = (ELT)1.0f;
  }

  // ds_read_b64_tr_b16: within 16 lanes, lane i receives element (i % 4) of the
  // 8-byte chunks addressed by lanes i/4, i/4 + 4, i/4 + 8, i/4 + 12.  Lane i
  // therefore points at key row (i / 4) and d-chunk 4*(i % 4) of its half tile,
  // and receives four consecutive keys of its own d = 32*T + (l % 32): the V
  // operand fragment of an MFMA step is two such reads and no shuffling.
  const int i16 = lane % 16, q4 = i16 / 4;
  const int v_lane = (4 * lh + q4) * (D * 2) + ((lane % 32) / 16) * 32 + (i16 % 4) * 8;
  int v_tile[TG];
  #pragma unroll
  for (int T = 0; T < TG; ++T) v_tile[T] = v_lane + ((T ^ EMH_VROT(q4)) * 64);

  // DEEP: K runs through a ring of three slots, V through one of two.  K(j) is read by the score MFMAs of step j,
  // V(j) by its output MFMAs; both are dead at the barrier that ends the step.  During step st the waves request
  // V(st + 1) (between the score MFMAs) and then K(st + 2) (between the output MFMAs), and the step's end waits
  // only for what is older than K(st + 2): the V block has the memory pipeline to itself for most of the step,
  // and a K block has two steps to land.  Otherwise (two slots each): K(st + 1) and V(st + 1) are requested
  // together during step st and both are waited for at its end.
  // Issue order: K0 V0 [K1] | step 0: V1, K2 | step 1: V2, K3 | ...
  EMH_CLAMP_K(0)
  EMH_CLAMP_V(0)
  EMH_STAGE_ALL_K(0);
  EMH_STAGE_ALL_V(0);
  if (DEEP) {
    if (1 < nsteps) { EMH_CLAMP_K(1) EMH_STAGE_ALL_K(1); }
    EMH_LAND((int)(1 < nsteps));
  } else {
    EMH_LAND(0);
  }
  if (Q_LDS) {
    const int qr_ = wq * 32 + lq;
    #pragma unroll
    for (int kk = 0; kk < D / 16; ++kk) qf[kk] = *(const FRAG*)(lds + Q_OFF_LDS + qr_ * (D * 2) + emh_kswz(qr_, kk * 2 + lh) * 16);
  }
  if (DR < D) {  // the columns past the row's end count as zeros
    #pragma unroll
    for (int kk = 0; kk < D / 16; ++kk)
      if (2 * kk + lh >= DR / 8) {
        #pragma unroll
        for (int e = 0; e < 8; ++e) qf[kk][e] = (ELT)0.0f;
      }
  }

  EMH_PHASE_AT(0)
  // Steps run in pairs so that a step's ring slots (its parity) are known when the code is generated: the LDS
  // addresses of the fragment reads are then a loop-invariant lane offset plus an immediate, with no vector
  // arithmetic per step.
#if PAIRSTEP
  #pragma unroll 1
  for (int st2 = 0; 2 * st2 < nsteps; ++st2)
  #pragma unroll
  for (int par = 0; par < 2; ++par) {
    const int st = 2 * st2 + par;
    if (st >= nsteps) break;
#else
  for (int st = 0; st < nsteps; ++st) {
#endif
    // The next step's blocks are requested between this step's score MFMAs: the
    // matrix pipe works through the chain while the wave issues the loads.
    const bool more = st + 1 < nsteps;
    const int jt = st * KVS + grp;
    const int k0 = jt * BKV;
    const bool active = (jt < ntiles) && (!CAUSAL || (k0 <= qw0_k + 31));
    EMH_STEP_BASES(1, st + 1)
    EMH_STEP_BASES(2, st + 2)
    // this step requests V(st + 1) and K(st + 1) (DEEP: K(st + 2)); a step past the sequence's last one is never requested
    EMH_CLAMP_V(st + 1)
    if (DEEP) { EMH_CLAMP_K(st + 2) } else { EMH_CLAMP_K(st + 1) }
    (void)kb2; (void)kl2; (void)vb2; (void)vl2; (void)kb1; (void)kl1;
    if (!active) {
      if (more) { EMH_STAGE_ALL_V(st + 1); if (!DEEP) EMH_STAGE_ALL_K(st + 1); }
      if (DEEP && st + 2 < nsteps) EMH_STAGE_ALL_K(st + 2);
    } else {
      const unsigned char* sK = lds + EMH_SLOT(st, RK) * SETB + grp * KBYTES;
      const unsigned char* sV = lds + V_RING + EMH_SLOT(st, RV) * SETB + grp * KBYTES;
      f32x16 sacc[BKV / 32];
      #pragma unroll
      for (int u = 0; u < BKV / 32; ++u) {
        #pragma unroll
        for (int r = 0; r < 16; ++r) sacc[u][r] = 0.0f;
        // All fragments of a 32-key sub-block are fetched before its MFMAs, so the
        // LDS latency is paid once per sub-block rather than once per MFMA pair.
        const int krow = u * 32 + lq;
        FRAG kf[D / 16];
        #pragma unroll
        for (int kk = 0; kk < D / 16; ++kk) kf[kk] = *(const FRAG*)(sK + krow * (D * 2) + emh_kswz(krow, kk * 2 + lh) * 16);
        __builtin_amdgcn_sched_barrier(0);
        #pragma unroll
        for (int kk = 0; kk < D / 16; ++kk) {
          sacc[u] = MFMA(kf[kk], qf[kk], sacc[u], 0, 0, 0);
          if (more) {
            #pragma unroll
            for (int i = 0; i < PER_T; ++i) if (EMH_SLOT_OF(i) == u * (D / 16) + kk) { EMH_STAGE_V(1, st + 1, i); if (!DEEP) EMH_STAGE_K(1, st + 1, i); }
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      EMH_STAMP_AT(0)
      // The V operand fragments of the output MFMAs are requested here, behind the score MFMAs (where a lane
      // has the registers for them): they land while the matrix pipe works through the scores and the softmax
      // runs, instead of in front of each output MFMA.
      u32x4 vfr[V_PRE ? (BKV / 32) * 2 * (D / 32) : 1];
      if (V_PRE) {
        #pragma unroll
        for (int u = 0; u < BKV / 32; ++u)
        #pragma unroll
        for (int s = 0; s < 2; ++s)
        #pragma unroll
        for (int dt = 0; dt < D / 32; ++dt) {
          const unsigned char* vp = sV + (32 * u + 16 * s) * (D * 2) + (dt / TG) * 256 + v_tile[dt % TG];
          const emh_s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) emh_s16x4*)(vp));
          const emh_s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) emh_s16x4*)(vp + 8 * (D * 2)));
          const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
          u32x4 av;
          av[0] = l2[0]; av[1] = l2[1]; av[2] = h2[0]; av[3] = h2[1];
          vfr[(u * 2 + s) * (D / 32) + dt] = av;
        }
        __builtin_amdgcn_sched_barrier(0);
      }
#if HAS_MASK
      {
        // The additive mask: this lane's query row, the keys of its accumulator rows (runs of four consecutive
        // keys).  Added before the scale is applied, divided by it, so the exponent's fma sees s * scale + mask.
        const MELT* mrow_ = Mp + M_OFF + (long)batch * M_SB + (long)head * M_SH + (long)(qrow < SQ ? qrow : SQ - 1) * M_SS;
        #pragma unroll
        for (int u = 0; u < BKV / 32; ++u)
        #pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
          const int key0 = k0 + 32 * u + 8 * g4 + 4 * lh;
          if (MASK_VEC && key0 + 3 < SKV) {
            const MVEC4 mv_ = *(const MVEC4*)(mrow_ + key0);
            #pragma unroll
            for (int j = 0; j < 4; ++j) sacc[u][4 * g4 + j] += (float)mv_[j] * INV_SCALE;
          } else {
            #pragma unroll
            for (int j = 0; j < 4; ++j) if (key0 + j < SKV) sacc[u][4 * g4 + j] += (float)mrow_[key0 + j] * INV_SCALE;
          }
        }
      }
#endif
      float mx = -1.0e30f;
      if ((CAUSAL && (k0 + BKV - 1 > qw0_k)) || (k0 + BKV > SKV)) {
        #pragma unroll
        for (int u = 0; u < BKV / 32; ++u)
        #pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int key = k0 + 32 * u + 8 * (r / 4) + 4 * lh + (r % 4);
          if ((CAUSAL && key > qrow_k) || key >= SKV) sacc[u][r] = -1.0e30f;
          mx = fmaxf(mx, sacc[u][r]);
        }
      } else {
        #pragma unroll
        for (int u = 0; u < BKV / 32; ++u)
        #pragma unroll
        for (int r = 0; r < 16; ++r) mx = fmaxf(mx, sacc[u][r]);
      }
      mx *= SCALE_LOG2;
      if (__any(mx > m_ref + RESCALE_SLACK)) {  // a vote over both halves of every row: the halves meet only when it passes
        mx = fmaxf(mx, emh_xor32(mx));
        const float m_new = fmaxf(m_ref, mx);
        const float alpha = EXP2(m_ref - m_new);
        m_ref = m_new;
        l_run *= alpha;
        #pragma unroll
        for (int t = 0; t < D / 32; ++t)
        #pragma unroll
        for (int r = 0; r < 16; ++r) oacc[t][r] *= alpha;
        if (MSUM) {
          #pragma unroll
          for (int r = 0; r < 16; ++r) lacc[r] *= alpha;
        }
      }
      float psum = 0.0f;
      #pragma unroll
      for (int u = 0; u < BKV / 32; ++u)
      #pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float p = EXP2(__builtin_fmaf(sacc[u][r], SCALE_LOG2, -m_ref));
        sacc[u][r] = p;
        if (!MSUM) psum += p;
      }
      l_run += psum;
      EMH_STAMP_AT(1)
      #pragma unroll
      for (int u = 0; u < BKV / 32; ++u)
      #pragma unroll
      for (int s = 0; s < 2; ++s) {
        FRAG pf;
        #pragma unroll
        for (int t = 0; t < 8; ++t) pf[t] = (ELT)sacc[u][8 * s + t];
        if (MSUM) lacc = MFMA(ones_f, pf, lacc, 0, 0, 0);
        #pragma unroll
        for (int dt = 0; dt < D / 32; ++dt) {
          u32x4 av;
          if (V_PRE) {
            av = vfr[(u * 2 + s) * (D / 32) + dt];
          } else {
            const unsigned char* vp = sV + (32 * u + 16 * s) * (D * 2) + (dt / TG) * 256 + v_tile[dt % TG];
            const emh_s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) emh_s16x4*)(vp));
            const emh_s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) emh_s16x4*)(vp + 8 * (D * 2)));
            const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
            av[0] = l2[0]; av[1] = l2[1]; av[2] = h2[0]; av[3] = h2[1];
          }
          oacc[dt] = MFMA(__builtin_bit_cast(FRAG, av), pf, oacc[dt], 0, 0, 0);
          if (DEEP && st + 2 < nsteps) {
            #pragma unroll
            for (int i = 0; i < PER_T; ++i) if ((i * ((BKV / 32) * 2 * (D / 32))) / PER_T == (u * 2 + s) * (D / 32) + dt) EMH_STAGE_K(2, st + 2, i);
          }
        }
      }
    }
    EMH_STAMP_AT(2)
    // end of the step: everything but K(st + 2) has landed; every wave is done with K(st) and V(st)
    EMH_LAND((int)(DEEP && st + 2 < nsteps));
    EMH_STAMP_AT(3)
  }
  EMH_PHASE_AT(1)

  // ---- close.  The key-split groups share the final combine: group g finishes
  // registers [g*RPG, (g+1)*RPG) of its rows' RPL output registers.  Every group
  // parks the registers the others own, and its (m, l); after one barrier each
  // combines its share with the same exp-family merge the streaming loop uses,
  // scales by 1/l and puts the 16-bit result into the O tile in LDS, which leaves
  // through 16-byte stores of whole rows.  (The rings are dead after the loop's last barrier.)
  if (MSUM) l_run = 0.5f * lacc[0];  // every element of the tile's column is the whole sum: half each, as the two lane halves are added below
  if (KVS > 1) {
    float* park = (float*)lds;
    float* pml = (float*)(lds + PARK_ML) + ((grp * WQ + wq) * 2) * 64 + lane;
    pml[0] = m_ref;
    pml[64] = l_run;
    #pragma unroll
    for (int g = 0; g < KVS; ++g) {
      if (g == grp) {
        #pragma unroll
        for (int h = 0; h < KVS; ++h) {
          if (h != g) {
            float* pw = park + (((h * (KVS - 1) + (g - (g > h ? 1 : 0))) * WQ + wq) * RPG) * 64 + lane * 4;
            #pragma unroll
            for (int r4 = 0; r4 < RPG / 4; ++r4) {
              f32x4 t;
              #pragma unroll
              for (int j = 0; j < 4; ++j) t[j] = OACC(h * RPG + 4 * r4 + j);
              *(f32x4*)(pw + r4 * 256) = t;
            }
          }
        }
      }
    }
    __syncthreads();
  }
  #pragma unroll
  for (int g = 0; g < KVS; ++g) {
    if (g == grp) {
      float a_own = 1.0f, l_tot = l_run, m_row = m_ref;
      float a_o[KVS];
      if (KVS > 1) {
        const float* pml = (const float*)(lds + PARK_ML) + lane;
        float m_all = m_ref, m_o[KVS], l_o[KVS];
        #pragma unroll
        for (int h = 0; h < KVS; ++h) {
          if (h != g) {
            m_o[h] = pml[((h * WQ + wq) * 2) * 64];
            l_o[h] = pml[((h * WQ + wq) * 2 + 1) * 64];
            m_all = fmaxf(m_all, m_o[h]);
          }
        }
        a_own = EXP2(m_ref - m_all);
        m_row = m_all;
        l_tot = l_run * a_own;
        #pragma unroll
        for (int h = 0; h < KVS; ++h) {
          if (h != g) {
            a_o[h] = EXP2(m_o[h] - m_all);
            l_tot += l_o[h] * a_o[h];
          }
        }
      }
      l_tot += emh_xor32(l_tot);
      const float inv = 1.0f / l_tot;
      const int orow = wq * 32 + lq;
#if KV_CTAS > 1
      // The slice's state goes to the workspace as it is: per query row D unnormalised output values (at the scale of the
      // row's reference maximum over the slice), then that maximum (log2 units, score scale folded in) and the row sum.
      float* prow = Op + ((((long)blockIdx.y * BATCH + batch) * HQ + head) * SQ + (q0 + orow < SQ ? q0 + orow : SQ - 1)) * (D + 4);
      if (q0 + orow < SQ && g == 0 && lh == 0) { prow[D] = m_row; prow[D + 1] = l_tot; }
#endif
      #pragma unroll
      for (int r4 = 0; r4 < RPG / 4; ++r4) {
        f32x4 acc;
        #pragma unroll
        for (int j = 0; j < 4; ++j) acc[j] = OACC(g * RPG + 4 * r4 + j) * a_own;
        if (KVS > 1) {
          #pragma unroll
          for (int h = 0; h < KVS; ++h) {
            if (h != g) {
              const f32x4 t = *(const f32x4*)((const float*)lds + (((g * (KVS - 1) + (h - (h > g ? 1 : 0))) * WQ + wq) * RPG) * 64 + lane * 4 + r4 * 256);
              #pragma unroll
              for (int j = 0; j < 4; ++j) acc[j] += t[j] * a_o[h];
            }
          }
        }
        // Registers 4i .. 4i+3 of tile T are d = 32*T + 8*i + 4*lh + (0..3): 8-byte slot 8*T + 2*i + lh of the row.
        const int f = g * RPG + 4 * r4;
#if KV_CTAS > 1
        (void)inv;
        if (q0 + orow < SQ) *(f32x4*)(prow + 32 * (f / 16) + 8 * ((f % 16) / 4) + 4 * lh) = acc;
#else
        PACK4 y;
        #pragma unroll
        for (int j = 0; j < 4; ++j) y[j] = (ELT)(acc[j] * inv);
        const int sl = 8 * (f / 16) + 2 * ((f % 16) / 4) + lh;
        *(PACK4*)(lds + O_OFF_LDS + orow * (D * 2) + ((sl ^ (orow % OSW)) * 8)) = y;
#endif
      }
    }
  }
  EMH_PHASE_AT(2)
#if KV_CTAS == 1
  __syncthreads();
  {
    ELT* obase = Op + O_OFF + (long)batch * O_SB + (long)head * O_SH;
    #pragma unroll
    for (int c0 = 0; c0 < QCHUNKS; c0 += NT) {
      const int c = c0 + tid;
      if (QCHUNKS % NT == 0 || c < QCHUNKS) {
        const int r = c / CPR, pc = c % CPR, x = r % OSW;
        // slots 2*pc and 2*pc + 1 of the row sit XOR x away: the same 16 bytes, halves swapped when x is odd
        const u32x4 t = *(const u32x4*)(lds + O_OFF_LDS + r * (D * 2) + ((pc ^ (x >> 1)) * 16));
        u32x4 y;
        y[0] = (x & 1) ? t[2] : t[0]; y[1] = (x & 1) ? t[3] : t[1];
        y[2] = (x & 1) ? t[0] : t[2]; y[3] = (x & 1) ? t[1] : t[3];
        if (q0 + r < SQ && (DR == D || pc < DR / 8)) *(u32x4*)(obase + (long)(q0 + r) * O_SS + pc * 8) = y;
      }
    }
    EMH_PHASE_AT(3)
    if (EMH_STAMP && bid == 0 && tid == 0 && pass == (PAIR ? 1 : 0)) {  // over the 16 bytes this thread has just stored: the first of row q0
      #pragma unroll
      for (int i = 0; i < 4; ++i) ((float*)(obase + (long)q0 * O_SS))[i] = (float)st_acc[i] / (float)(st_acc[4 + i] ? st_acc[4 + i] : 1u);
    }
  }
#endif
  }
}
"""


_V_PRE = True
_PAIRSTEP = True


def lds_plan(waves: int, kvs: int, bkv: int, head_dim: int, limit: int, deep: bool = False) -> dict:
    """LDS layout of a workgroup: ``[K ring | V ring | Q tile]``.

    A ring slot holds the K (or V) blocks of one step, one per key-split group.  ``deep``: three K slots and two V
    slots (a K block is requested two steps ahead, and a step's end waits for the next V block only) instead of
    two and two.

    After the key loop the rings hold the parked partial results of the key-split groups (``(kvs-1) * waves *
    registers`` lane-vectors and an ``(m, l)`` table) and, behind them, the O tile.  The Q tile is staged through
    LDS only when it fits behind all of that; ``q_off`` is ``None`` when the fragments are read from global
    memory instead."""
    slot = kvs * bkv * head_dim * 2
    rk, rv = (3, 2) if deep else (2, 2)
    ring = (rk + rv) * slot
    regs = head_dim // 32 * 16
    park_ml = (kvs - 1) * waves * regs * 256
    park = park_ml + (kvs * waves * 512 if kvs > 1 else 0)
    tile = 32 * waves * head_dim * 2
    o_off = park
    end = max(ring, o_off + tile)
    q_off = end if end + tile <= limit else None
    return {"bytes": end + (tile if q_off is not None else 0), "q_off": q_off, "o_off": o_off, "park_ml": park_ml, "rk": rk, "rv": rv, "deep": deep}


def emit_flash(body: Flash, name: str, ctx: Context = Context()) -> HipOp:
    from deplodock_amd.emit.flash_f32 import emit_flash_f32, on_f32_atoms

    if on_f32_atoms(body):
        return emit_flash_f32(body, name, ctx)
    if body.private:
        from deplodock_amd.emit.flash_pv import emit_flash_pv

        return emit_flash_pv(body, name, ctx)
    if body.ws or body.sp:
        from deplodock_amd.emit.flash_ws import emit_flash_ws

        return emit_flash_ws(body, name, ctx)
    D = body.head_dim
    if body.dtype.name not in ("bf16", "f16"):
        raise LoweringError("flash: MFMA tier needs 16-bit operands")
    if D not in (64, 128, 256):
        raise LoweringError(f"flash: head_dim {D} must be 64, 128 or 256 on this tier")
    DR = body.head_dim_real or D
    if DR > D or DR % 8 or DR < 8:
        raise LoweringError(f"flash: rows of {DR} values do not pad to head_dim {D} in whole 16-byte chunks")
    if body.q_heads % body.kv_heads:
        raise LoweringError("flash: q heads must be a multiple of kv heads")
    waves = body.waves
    kvs = body.kv_split
    BQ = 32 * waves
    BKV = body.block_kv
    if BKV % 32 or BKV < 32:
        raise LoweringError("flash: key block must be a multiple of 32")
    NT = waves * kvs * 64
    if NT > ctx.max_threads_per_block:
        raise LoweringError(f"flash: {waves} x {kvs} waves exceed {ctx.max_threads_per_block} threads")
    if (BKV * D // 8) % NT:
        raise LoweringError("flash: a key block's 16-byte chunks must be a multiple of the workgroup's threads")
    if (D // 32 * 16) % (4 * kvs):
        raise LoweringError(f"flash: {kvs} key-split groups cannot share the {D // 32 * 16} output registers of a lane")
    plan = lds_plan(waves, kvs, BKV, D, ctx.lds_bytes_per_cu, deep=body.deep)
    lds = plan["bytes"]
    if lds > ctx.lds_bytes_per_cu:
        raise LoweringError(f"flash: {lds} B of LDS exceeds {ctx.lds_bytes_per_cu} B per CU")
    for st in (body.q_strides, body.k_strides, body.v_strides):
        if st[2] % 8:
            raise LoweringError("flash: sequence strides must keep 16-byte row alignment")
    for st, heads in ((body.q_strides, body.q_heads), (body.k_strides, body.kv_heads), (body.v_strides, body.kv_heads), (body.o_strides, body.q_heads)):
        if st[2] % 8 or (heads > 1 and st[1] % 8) or (body.batch > 1 and st[0] % 8):
            raise LoweringError("flash: batch / head / sequence strides must keep 16-byte alignment")
    if any(o % 8 for o in (body.q_offset, body.k_offset, body.v_offset, body.o_offset)):
        raise LoweringError("flash: offsets break 16-byte alignment")
    qblocks = -(-body.q_len // BQ)
    pair = bool(body.pair)
    split = int(getattr(body, "kv_ctas", 1) or 1)
    if split > 1:
        if body.partials is None:
            raise LoweringError("flash: a cross-workgroup key split (REDUCE=g<n>k) is lowered as a partial kernel plus a combine (passes.lower), not by this emitter alone")
        if pair or body.mask is not None or (getattr(body, "sym", None) is not None and body.sym.fields):
            raise LoweringError("flash: the cross-workgroup key split takes no mirrored pairs, mask operand or symbolic lengths")
        step_keys = kvs * BKV
        kv_chunk = -(-(-(-body.kv_len // split)) // step_keys) * step_keys  # whole key steps per slice
        split = -(-body.kv_len // kv_chunk)  # slices that hold keys
    # Symbolic lengths (``body.sym``): SQ / SKV, the query-block count, the launch size and a [B, H, S, D] tensor's
    # batch stride become expressions over the kernel's trailing ``int`` parameter; every guard the loop has for
    # ragged lengths (row clamps, key masks, the causal block limit) already reads them at run time.
    sym = getattr(body, "sym", None)
    symf = sym.fields if sym is not None else {}
    if symf:
        if pair:
            raise LoweringError("flash: mirrored query-block pairs need a block count known when the kernel is built")
        for key in symf:
            if key not in ("q_len", "kv_len") and not (key.split(".")[0] in ("q_strides", "k_strides", "v_strides", "o_strides", "mask_strides") and key.split(".")[1] in ("0", "1", "2")):
                raise LoweringError(f"flash: {key} cannot follow a symbolic axis")
            if isinstance(symf[key], Affine) and "strides" in key and not key.startswith("mask_") and (symf[key].a % 8 or symf[key].b % 8):
                raise LoweringError(f"flash: {key} = {symf[key]} does not keep 16-byte alignment at every size")
    if pair and not (body.causal and qblocks % 2 == 0):
        raise LoweringError("flash: pairing mirrored query blocks needs a causal mask and an even block count")
    qslots = qblocks // 2 if pair else qblocks
    bf16 = body.dtype.name == "bf16"
    has_mask = body.mask is not None
    if has_mask:
        if body.mask_dtype.name not in ("bf16", "f16", "f32"):
            raise LoweringError("flash: the mask must be a floating-point tensor")
        if body.scale == 0.0:
            raise LoweringError("flash: a mask with a zero scale is not supported")
        m_strides = [symf.get(f"mask_strides.{i}", v) for i, v in enumerate(body.mask_strides)]
    defs = {
        "KNAME": name,
        "NT": NT,
        "D": D,
        "DR": DR,
        "BQ": BQ,
        "BKV": BKV,
        "KVS": kvs,
        "CPR": D // 8,
        "KRPL": max(1, 16 // (D // 8)),
        "TG": min(4, D // 32),
        "SQ": c_value(symf.get("q_len", body.q_len)),
        **({"SKV_ALL": body.kv_len, "KV_CHUNK": kv_chunk, "BATCH": body.batch} if split > 1 else {"SKV": c_value(symf.get("kv_len", body.kv_len))}),
        "KV_CTAS": split,
        # every key step lies inside the sequence (or the slice of it), known when the kernel is built
        "WHOLE_STEPS": 1 if "kv_len" not in symf and body.kv_len % (kvs * BKV) == 0 else 0,
        "OUT_T": "float" if split > 1 else rt.type_name(body.dtype.name),
        "HQ": body.q_heads,
        "GROUP": body.q_heads // body.kv_heads,
        "QBLOCKS": "((SQ + BQ - 1) / BQ)" if "q_len" in symf else qblocks,
        "QSLOTS": "QBLOCKS" if "q_len" in symf else qslots,
        "SYM_PARAM": f", int {param_name(sym.name)}" if symf else "",
        "HAS_MASK": 1 if has_mask else 0,
        "MASK_PARAM": f", const {rt.type_name(body.mask_dtype.name)}* __restrict__ Mp" if has_mask else "",
        **({"MELT": rt.type_name(body.mask_dtype.name), "MVEC4": rt.vector_type(body.mask_dtype.name, 4)[0],
            # four keys per load (8 or 16 bytes) when every row of the mask starts on a four-element boundary: known when
            # the kernel is built for static strides, one scalar test per launch when a stride follows a symbolic length
            "MASK_VEC": "((((M_SB) | (M_SH) | (M_SS) | (M_OFF)) & 3) == 0)" if any(isinstance(v, Affine) for v in m_strides) else int(all(v % 4 == 0 for v in (*m_strides, body.mask_offset))),
            "M_SB": c_value(m_strides[0]), "M_SH": c_value(m_strides[1]), "M_SS": c_value(m_strides[2]), "M_OFF": body.mask_offset,
            "INV_SCALE": float_literal(1.0 / body.scale)} if has_mask else {}),
        "PAIR": 1 if pair else 0,
        "MSUM": 1 if body.mfma_sum else 0,
        # steps in parity pairs (static ring slots) unless the whole key range is one or two steps
        "PAIRSTEP": 1 if _PAIRSTEP and body.pair_steps and (bool(symf) or -(-(kv_chunk if split > 1 else body.kv_len) // (kvs * BKV)) > 2) else 0,
        "V_PRE": 1 if _V_PRE and (BKV // 32) * 2 * (D // 32) * 4 <= 32 else 0,  # the prefetched V fragments take at most 32 registers
        "RK": plan["rk"], "RV": plan["rv"], "DEEP": 1 if plan["deep"] else 0,
        "Q_LDS": 1 if plan["q_off"] is not None else 0,
        "Q_OFF_LDS": plan["q_off"] or 0,
        "O_OFF_LDS": plan["o_off"],
        "PARK_ML": plan["park_ml"],
        "CAUSAL": 1 if body.causal else 0,
        "SCALE_LOG2": float_literal(body.scale * math.log2(math.e)),
        "Q_SB": c_value(symf.get("q_strides.0", body.q_strides[0])), "Q_SH": c_value(symf.get("q_strides.1", body.q_strides[1])), "Q_SS": c_value(symf.get("q_strides.2", body.q_strides[2])), "Q_OFF": body.q_offset,
        "K_SB": c_value(symf.get("k_strides.0", body.k_strides[0])), "K_SH": c_value(symf.get("k_strides.1", body.k_strides[1])), "K_SS": c_value(symf.get("k_strides.2", body.k_strides[2])), "K_OFF": body.k_offset,
        "V_SB": c_value(symf.get("v_strides.0", body.v_strides[0])), "V_SH": c_value(symf.get("v_strides.1", body.v_strides[1])), "V_SS": c_value(symf.get("v_strides.2", body.v_strides[2])), "V_OFF": body.v_offset,
        "O_SB": c_value(symf.get("o_strides.0", body.o_strides[0])), "O_SH": c_value(symf.get("o_strides.1", body.o_strides[1])), "O_SS": c_value(symf.get("o_strides.2", body.o_strides[2])), "O_OFF": body.o_offset,
        "ELT": rt.type_name(body.dtype.name),
        "FRAG": rt.vector_type(body.dtype.name, 8)[0],
        "PACK4": rt.vector_type(body.dtype.name, 4)[0],
        "MFMA": "__builtin_amdgcn_mfma_f32_32x32x16_bf16" if bf16 else "__builtin_amdgcn_mfma_f32_32x32x16_f16",
        # 2^x straight on the transcendental unit; inputs are <= 0 and the result
        # feeds a 16-bit operand, so the fast form loses nothing that survives.
        "EXP2": rt.intrinsic("fast_exp2", "f32"),
        # log2-domain slack before the accumulators are rescaled to a new maximum:
        # probabilities stay below 2^8, far inside fp32 / bf16 range.
        "RESCALE_SLACK": "8.0f",
    }  # fmt: skip
    head = f"// {name}: B={body.batch} Hq={body.q_heads} Hkv={body.kv_heads} Sq={body.q_len} Skv={body.kv_len} D={D} causal={body.causal}\n"
    head += "".join(f"#define {k} {v}\n" for k, v in defs.items())
    grid = qslots * body.q_heads * body.batch
    head += f"#define GRID {'((int)gridDim.x)' if 'q_len' in symf else grid}\n#define XCDS {ctx.xcds}\n"
    source = prelude.header(prelude.DMA) + head + _SRC
    return HipOp(
        kernel_source=source,
        kernel_name=name,
        arg_order=(body.q, body.k, body.v, *((body.mask,) if has_mask else ()), body.partials if split > 1 else body.out),
        grid=((CeilDiv(symf["q_len"], BQ), body.q_heads * body.batch) if "q_len" in symf else (grid,), (split,), (1,)),
        block=((NT,), (1,), (1,)),
        lds_bytes=lds,
        runtime_args=(sym.name,) if symf else (),
        comment=f"flash Sq={body.q_len} Skv={body.kv_len} D={D} causal={body.causal} waves={waves} bkv={BKV} split={kvs} pair={int(pair)}",
        algo_bytes=body.algo_bytes(),
        algo_flops=body.algo_flops(),
        knobs={"FLASH": f"w{waves}/kv{BKV}/s{kvs}" + ("/p" if pair else "") + ("/k3" if plan["deep"] else "") + ("/ms" if body.mfma_sum else ""), **({"REDUCE": f"g{split}k"} if split > 1 else {})},
    )


def flash_partial_slices(body: Flash) -> int:
    """Key slices the partial kernel of ``body``'s cross-workgroup split actually runs (slices are whole key steps, so
    fewer than asked for can hold all the keys)."""
    step_keys = body.kv_split * body.block_kv
    chunk = -(-(-(-body.kv_len // body.kv_ctas)) // step_keys) * step_keys
    return -(-body.kv_len // chunk)


def emit_flash_combine(body: Flash, ws: str, name: str, ctx: Context = Context()) -> HipOp:
    """Merge of the key slices' ``(m, l, O)``: per query row ``m = max m_s``, ``l = sum l_s 2^(m_s - m)``,
    ``out = sum O_s 2^(m_s - m) / l`` — the exp-family combine the streaming loop uses, applied across workgroups (the
    reference's kernel finalize of the twisted carrier, passes/lowering/tile/030_split.py:217-334).  One thread per four
    consecutive output values; the workspace row is ``head_dim`` values, then ``m`` (log2 units) and ``l``."""
    D, S = body.head_dim, flash_partial_slices(body)
    DR = body.head_dim_real or D  # the workspace rows are D wide; only the first DR columns are output
    rows = body.batch * body.q_heads * body.q_len
    elt, pack4 = rt.type_name(body.dtype.name), rt.vector_type(body.dtype.name, 4)[0]
    groups = rows * (DR // 4)
    o: list[str] = []
    a = o.append
    a(f"// {name}: combine of {S} key slices of attention B={body.batch} Hq={body.q_heads} Sq={body.q_len} D={D}")
    a(f'extern "C" __global__ __launch_bounds__(256) void {name}(const float* __restrict__ WS, {elt}* __restrict__ O) {{')
    a("  const long q = (long)blockIdx.x * 256 + threadIdx.x;")
    a(f"  if (q >= {groups}L) return;")
    a(f"  const long row = q / {DR // 4}; const int c = (int)(q % {DR // 4}) * 4;")
    a(f"  const long s_ = row % {body.q_len}, h_ = (row / {body.q_len}) % {body.q_heads}, b_ = row / {body.q_len * body.q_heads};")
    a(f"  const float* w0 = WS + row * {D + 4};")
    a("  float m = w0[" + str(D) + "];")
    for s in range(1, S):
        a(f"  m = fmaxf(m, w0[{s * rows * (D + 4) + D}L]);")
    a("  float l = 0.0f; f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};")
    for s in range(S):
        a(f"  {{ const float* w = w0 + {s * rows * (D + 4)}L; const float e = exp2f(w[{D}] - m); l += w[{D + 1}] * e; const f32x4 t = *(const f32x4*)(w + c); acc[0] += t[0] * e; acc[1] += t[1] * e; acc[2] += t[2] * e; acc[3] += t[3] * e; }}")
    a("  const float inv = 1.0f / l;")
    a(f"  {pack4} y; y[0] = ({elt})(acc[0] * inv); y[1] = ({elt})(acc[1] * inv); y[2] = ({elt})(acc[2] * inv); y[3] = ({elt})(acc[3] * inv);")
    a(f"  *({pack4}*)(O + {body.o_offset}L + b_ * {body.o_strides[0]}L + h_ * {body.o_strides[1]}L + s_ * {body.o_strides[2]}L + c) = y;")
    a("}")
    return HipOp(
        kernel_source=prelude.header() + "\n".join(o) + "\n",
        kernel_name=name,
        arg_order=(ws, body.out),
        grid=((-(-groups // 256),), (1,), (1,)),
        block=((256,), (1,), (1,)),
        comment=f"combine of {S} key slices of attention Sq={body.q_len} Skv={body.kv_len} D={D}",
        algo_bytes=S * rows * (D + 4) * 4 + rows * DR * body.dtype.nbytes,
        algo_flops=0,
        knobs={"REDUCE": f"g{S}k"},
    )
