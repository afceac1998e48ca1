"""Wave-specialised form of the fused attention kernel (``FLASH=.../ws``).

Same algebra, operand layouts, swizzles and close as ``emit/flash.py`` (the transposed-score MFMA form of
the reference's warp-flash realisation, emmy/compiler/pipeline/passes/lowering/kernel/_twist.py:229-363);
what changes is who does what, and when:

* **Eight waves, two roles.**  Waves 0-3 (one per SIMD) are *consumers*: 32 query rows each, ``waves`` row
  groups x ``kv_split`` key-split groups, ``waves * kv_split == 4``.  Waves 4-7 (one per SIMD) are *stagers*:
  they issue every direct-to-LDS request, wait for their own requests by count and publish them.  A request
  blocks its wave at issue while the memory pipeline is full, which at this kernel's K/V rate is most of the
  time; on a stager that costs nothing, in a consumer's stream it holds back the MFMAs queued behind it.
* **A consumer's instruction stream is software-pipelined over 32-key sub-blocks.**  In iteration t it issues
  the output MFMAs of sub-block t-1 and the score MFMAs of sub-block t+1, and between every two MFMAs a slice
  of the softmax of sub-block t (``sched_barrier`` pins the interleaving): the vector pipe works in the shadow
  of the matrix pipe from one wave, with no second wave per SIMD and no phase alignment between waves.
* **Rings of ``ring`` sub-steps per operand, one workgroup barrier per iteration.**  A sub-step is the 32-key
  blocks of all key-split groups.  In iteration t the stagers request K(t+ring) into the slot whose last
  reader (the score MFMAs of sub-block t, in iteration t-1) is done, and V(t+ring-2) likewise; the barrier that
  ends iteration t waits for K(t+2) and V(t): ``ring - 2`` iterations of lead for every request.

The unrolled iterations carry their ring slots as immediates (``lcm(2, ring)`` copies: slot and the parity
of the score / probability double buffers); the last active sub-block of a wave — the only one a causal or
ragged mask can touch — runs in a tail with run-time slots and the masked softmax.
"""

from __future__ import annotations

import math

from deplodock_amd.context import Context
from deplodock_amd.emit import prelude
from deplodock_amd.emit.errors import LoweringError
from deplodock_amd.emit.flash import lds_plan as _close_plan
from deplodock_amd.ir.expr import float_literal
from deplodock_amd.ir.hip import HipOp
from deplodock_amd.ir.tile import Flash
from deplodock_amd.render_target import rt

CONSUMER_WAVES = 4
STAGER_WAVES = 4
_PREFETCH = 3  # fragment reads are issued this many MFMAs ahead of their use

# issue cost of the softmax's vector instructions, in clocks of the SIMD's vector pipe (a transcendental
# takes four passes); only the ratios matter, they decide how the instructions are dealt over the slices
_COST = {"max": 4, "misc": 4, "exp": 20, "cvt": 2, "add": 4}


def ws_lds_plan(waves: int, kvs: int, head_dim: int, limit: int, rings: tuple[int, ...] = (4, 3)) -> dict:
    """``[K ring | V ring | Q tile]``; after the key loop the rings hold the parked partial results and the O
    tile (the layout of ``flash.lds_plan``).  The ring depth is the largest of ``rings`` that fits."""
    slot = kvs * 32 * head_dim * 2
    tile = 32 * waves * head_dim * 2
    close = _close_plan(waves, kvs, 32, head_dim, 1 << 30)
    close_bytes = close["o_off"] + tile
    for ring in rings:
        both = 2 * ring * slot
        if both + tile <= limit and close_bytes <= both:
            return {"bytes": both + tile, "ring": ring, "slot": slot, "q_off": both, "o_off": close["o_off"], "park_ml": close["park_ml"]}
    raise LoweringError(f"flash: rings of {min(rings)} {slot}-byte sub-steps per operand and a {tile}-byte Q tile exceed {limit} B of LDS")


class _Lines:
    def __init__(self) -> None:
        self.out: list[str] = []
        self.depth = 1

    def __call__(self, text: str = "") -> None:
        self.out.append("  " * self.depth + text if text else "")

    def open(self, text: str) -> None:
        self(text + " {")
        self.depth += 1

    def close(self, tail: str = "") -> None:
        self.depth -= 1
        self("}" + tail)


def _v_reads(a: _Lines, tag: str, D: int, s: int, dt: int, slot) -> None:
    """The two transposing reads of the V fragment of output MFMA (s, dt): keys 16 s .. 16 s + 15 of the wave's
    32-key block, d tile dt."""
    tg = min(4, D // 32)
    off = f"{slot} * SLOT + {(16 * s) * (D * 2) + (dt // tg) * 256}" if isinstance(slot, int) else f"{slot} + {(16 * s) * (D * 2) + (dt // tg) * 256}"
    a(f"const emh_s16x4 {tag}l = EMH_ABLATE == 4 ? emh_abl4 : EMH_TR16(vb[{dt % tg}] + ({off}));")
    a(f"const emh_s16x4 {tag}h = EMH_ABLATE == 4 ? emh_abl4 : EMH_TR16(vb[{dt % tg}] + ({off}) + {8 * D * 2});")


def _v_mfma(a: _Lines, tag: str, dt: int, pfrag: str) -> None:
    a(f"{{ const u32x2 l2_ = __builtin_bit_cast(u32x2, {tag}l), h2_ = __builtin_bit_cast(u32x2, {tag}h); u32x4 av_; av_[0] = l2_[0]; av_[1] = l2_[1]; av_[2] = h2_[0]; av_[3] = h2_[1];")
    a(f"  oacc[{dt}] = MFMA(__builtin_bit_cast(FRAG, av_), __builtin_bit_cast(FRAG, {pfrag}), oacc[{dt}], 0, 0, 0); }}")


def _k_read(a: _Lines, tag: str, kk: int, slot) -> None:
    off = f"{slot} * SLOT" if isinstance(slot, int) else f"{slot}"
    a(f"const FRAG {tag} = EMH_ABLATE == 4 ? qf[{kk}] : *(const FRAG*)(kb[{kk}] + ({off}));")


def _max_chain(src: str) -> list[str]:
    """The maximum of the lane's 16 scores in two chains (a dependent instruction waits for its operand, and a single
    wave per SIMD has no other wave to fill the gap), in the exponent's log2 units."""
    out = [f"float mx = fmaxf({src}[0], {src}[1]), my = fmaxf({src}[2], {src}[3]);"]
    for r in range(4, 16, 4):
        out.append(f"mx = fmaxf(fmaxf(mx, {src}[{r}]), {src}[{r + 1}]); my = fmaxf(fmaxf(my, {src}[{r + 2}]), {src}[{r + 3}]);")
    out.append("mx = fmaxf(mx, my) * SCALE_LOG2;")
    return out


def _pack(dst: str, r: int, pin: bool = True) -> str:
    """Two probabilities per 32-bit word of the operand fragment.  The empty asm pins the conversion where it is written
    (a vector assembled element by element is converted where its last element is written, with all sixteen fp32 values
    live until then)."""
    w = f"{dst}[{r // 8}][{(r % 8) // 2}]"
    return f"{{ PACK2 h_; h_[0] = (ELT)p{r}; h_[1] = (ELT)p{r + 1}; {w} = __builtin_bit_cast(unsigned, h_);" + (f' asm volatile("" : "+v"({w}));' if pin else "") + " }"


def _softmax_ticks(src: str, dst: str) -> list[tuple[str, int]]:
    """Exponentials, 16-bit probabilities (into ``dst``) and the row sum of one 32-key sub-block against ``m_ref``, as
    ``(statements, cost)`` ticks.  The chain of a score — exponent (fma), exponential, conversion / row sum — is skewed:
    at tick k the exponent of score k, the exponential of score k - 2, and the conversion and sum of the pair that was
    finished two ticks before, so no instruction reads what the one just before it wrote."""
    body: list[tuple[str, int]] = []
    for k in range(16 + 6):
        tick: list[str] = []
        cost = 0
        if k < 16:
            tick.append(f"const float e{k} = __builtin_fmaf({src}[{k}], SCALE_LOG2, -m_ref);")
            cost += _COST["misc"]
        if 0 <= k - 2 < 16:
            tick.append(f"const float p{k - 2} = EXP2(e{k - 2});")
            cost += _COST["exp"] - _COST["misc"]
        j, odd = divmod(k - 5, 2)  # pair j = scores 2j, 2j + 1: its second exponential was issued at tick 2j + 3
        if 0 <= j < 8 and odd == 0:
            r = 2 * j
            tick.append(_pack(dst, r))
            tick.append(f"psum {'=' if r == 0 else '+='} p{r} + p{r + 1}; asm volatile(\"\" : \"+v\"(psum));")  # pinned: the sum belongs in the shadow of the MFMAs
            cost += 2 * _COST["cvt"] + 2 * _COST["add"]
        if tick:
            body.append(("\n".join(tick), cost))
    return body


_RESCALE_IN_PLACE = (
    # in place (tied operands): a conditional product the compiler is free to put elsewhere costs a second set of accumulators
    'asm volatile("s_nop 15\\n\\ts_nop 15");  // the accumulators\' last MFMAs have left the matrix pipe (the compiler does not see into the statements below)\n'
    '_Pragma("unroll") for (int t_ = 0; t_ < D / 32; ++t_) _Pragma("unroll") for (int r_ = 0; r_ < 16; ++r_) asm volatile("v_mul_f32 %0, %1, %0" : "+v"(oacc[t_][r_]) : "v"(alpha));'
)


def _classic_softmax(a: _Lines, D: int, src: str, dst: str, *, masked: bool) -> None:
    """The softmax of a sub-block, unsliced: the row maximum, the vote on raising the reference maximum, the rescale of
    what has been accumulated (at once: the output MFMAs before it have been issued), then exponentials, probabilities
    and row sum.  For a wave's last sub-block (``masked``: the causal diagonal, the end of the keys)."""
    if masked:
        for r in range(16):
            a(f"{{ const int key_ = k0t + {8 * (r // 4) + (r % 4)} + 4 * lh; if ((CAUSAL && key_ > qrow) || key_ >= SKV) {src}[{r}] = -1.0e30f; }}")
    for line in _max_chain(src):
        a(line)
    a("if (__any(mx > m_ref + RESCALE_SLACK)) {  // a vote over both halves of every row: the halves meet only when it passes")
    a("  mx = fmaxf(mx, emh_xor32(mx)); const float mn_ = fmaxf(m_ref, mx); alpha = EXP2(m_ref - mn_); m_ref = mn_; l_run *= alpha;")
    for line in _RESCALE_IN_PLACE.split("\n"):
        a("  " + line)
    a("}")
    for r in range(16):
        a(f"const float p{r} = EXP2(__builtin_fmaf({src}[{r}], SCALE_LOG2, -m_ref));")
    for r in range(0, 16, 2):
        a(_pack(dst, r, pin=False))
    a("psum = " + " + ".join(f"(p{r} + p{r + 1})" for r in range(0, 16, 2)) + ";")
    a("l_run += psum;")


_LEAD_TICKS = 7  # ticks of vector work issued while the iteration's first fragment reads are in flight


def _request_statements(per_s: int) -> list[str]:
    """The requests one staging thread issues in an iteration, in issue order: the V sub-step first, then the K one
    (``EMH_SUB_BASES`` has named their scalar parts under the tags ``v`` and ``k``)."""
    return [f"EMH_REQ_I(v, {i}, vvo0, vbase, V_SS, emh_vswz, V_RING)" for i in range(per_s)] + [f"EMH_REQ_I(k, {i}, kvo0, kbase, K_SS, emh_kswz, 0)" for i in range(per_s)]


def _iteration(a: _Lines, D: int, *, par: int, has_pv: bool, kslot, vslot, t_expr: str | None = None, per_s: int = 0) -> None:
    """One steady consumer iteration on sub-block t (scores in ``sc<par>``): output MFMAs of sub-block t-1 (its
    probabilities in ``pq<par^1>``, V slot ``vslot``; none when ``has_pv`` is false: t = 0), the softmax of t
    (probabilities into ``pq<par>``), score MFMAs of sub-block t+1 (K slot ``kslot``) into ``sc<par^1>``.  Slots are ints
    (immediates) or the names of run-time byte offsets.

    A raised reference maximum (``resc`` / ``alpha``, decided by the vote in this iteration's lead) reaches the output
    accumulators in the lead of the *next* iteration, before that iteration's output MFMAs: the probabilities those
    multiply were taken against the raised maximum, everything accumulated so far against the one before."""
    src, dst, nxt, old = f"sc{par}", f"pq{par}", f"sc{par ^ 1}", f"pq{par ^ 1}"
    # The score MFMAs of a sub-block accumulate into one tile: each depends on the one before it, and a dependent MFMA
    # waits until that one has left the matrix pipe (twice its issue interval).  Interleaved with the output MFMAs (four
    # tiles, eight MFMAs) the chain's links sit two issue slots apart and the pipe stays full from a single wave.
    pv = [("pv", (s, dt)) for s in range(2) for dt in range(D // 32)] if has_pv else []
    qk = [("qk", (kk,)) for kk in range(D // 16)]
    jobs: list[tuple[str, tuple]] = []
    for i in range(max(len(pv), len(qk))):
        jobs += pv[i : i + 1] + qk[i : i + 1]
    body = _softmax_ticks(src, dst)
    # self-staging waves: this iteration's requests, one behind each of the first MFMAs (a request that finds the memory
    # pipeline full blocks its wave at issue; the other wave of the SIMD goes on)
    reqs = _request_statements(per_s) if t_expr is not None else []
    a.open("")
    a("float psum;")
    a("EMH_STAMP_AT(3)  // since the end of the iteration before: the barrier")
    if reqs:
        a(f"EMH_SUB_BASES(v, ({t_expr}) + RING - 2, vbase, V_SS, V_RING)")
        a(f"EMH_SUB_BASES(k, ({t_expr}) + RING, kbase, K_SS, 0)")

    def read(j: int) -> None:
        kind, arg = jobs[j]
        if kind == "pv":
            _v_reads(a, f"vf{j}_", D, arg[0], arg[1], vslot)
        else:
            _k_read(a, f"kf{j}_", arg[0], kslot)

    def mfma(j: int) -> None:
        kind, arg = jobs[j]
        if kind == "pv":
            _v_mfma(a, f"vf{j}_", arg[1], f"{old}[{arg[0]}]")
        else:
            acc = nxt if arg[0] else "emh_zero16"
            a(f"{nxt} = MFMA(kf{j}_, qf[{arg[0]}], {acc}, 0, 0, 0);")

    def ticks(n: int) -> None:
        nonlocal idx, done
        for _ in range(n):
            if idx < len(body):
                for line in body[idx][0].split("\n"):
                    a(line)
                a("__builtin_amdgcn_sched_barrier(0);")
                done += body[idx][1]
                idx += 1

    idx, done = 0, 0.0
    if has_pv:
        a("if (resc) {  // what the vote of the iteration before decided (rare after the first sub-blocks)")
        for line in _RESCALE_IN_PLACE.split("\n"):
            a("  " + line)
        a("  resc = false; }")
    for j in range(min(_PREFETCH, len(jobs))):
        read(j)
    for line in _max_chain(src):
        a(line)
    a("if (__any(mx > m_ref + RESCALE_SLACK)) {  // a vote over both halves of every row: the halves meet only when it passes")
    a("  mx = fmaxf(mx, emh_xor32(mx)); const float mn_ = fmaxf(m_ref, mx); alpha = EXP2(m_ref - mn_); m_ref = mn_; l_run *= alpha; resc = true; }")
    a("__builtin_amdgcn_sched_barrier(0);")
    ticks(_LEAD_TICKS if has_pv else 2)
    a("EMH_STAMP_AT(0)  // the lead: first fragment reads in flight, vector work only")
    lead_cost = done
    total = sum(c for _, c in body) - lead_cost
    for j in range(len(jobs)):
        if j + _PREFETCH < len(jobs):
            read(j + _PREFETCH)
        mfma(j)
        if j < len(reqs):
            a(reqs[j])
        target = lead_cost + total * (j + 1) / len(jobs)
        while idx < len(body) and (done + body[idx][1] / 2 <= target or j == len(jobs) - 1):
            ticks(1)
        if has_pv and j == len(jobs) // 2 - 1:
            a("EMH_STAMP_AT(1)  // the first half of the slices")
        a("__builtin_amdgcn_sched_barrier(0);")
    for r in reqs[len(jobs):]:
        a(r)
    a("EMH_STAMP_AT(2)  // the second half of the slices")
    a("l_run += psum; asm volatile(\"\" : \"+v\"(l_run));")
    if not has_pv:
        a("resc = false;  // nothing has been accumulated yet: there is nothing to rescale")
    a.close()


def _consumer(a: _Lines, D: int, ring: int, per_s: int = 0) -> None:
    """The consumer role.  Naming is canonical at every loop boundary — the scores of the sub-block about to be
    reduced in ``sc0``, the probabilities of the one before it in ``pq1`` — so the unrolled loop has one entry, one
    back edge and one exit: ``lcm(2, ring)`` iterations per trip with ring slots and the double buffers' parity
    resolved in the text; what is left of a wave's full iterations runs in a loop with run-time slots that copies
    the buffers back to their canonical names.

    ``per_s`` > 0: the waves stage for themselves (no staging role): every iteration t, whatever the wave computes in
    it, carries the wave's share of the requests of sub-steps V(t + ring - 2) and K(t + ring) and ends in ``EMH_LAND(t)``
    (wait for what must have landed, publish, barrier) instead of a bare barrier."""
    sp = per_s > 0
    L = ring * 2 // math.gcd(ring, 2)
    jobs = [(s, dt) for s in range(2) for dt in range(D // 32)]

    def end(t_expr: str) -> None:
        a(f"EMH_LAND({t_expr})" if sp else "EMH_BARRIER();")

    def requests_now(t_expr: str) -> None:
        if sp:
            a(f"{{ EMH_SUB_BASES(v, ({t_expr}) + RING - 2, vbase, V_SS, V_RING) EMH_SUB_BASES(k, ({t_expr}) + RING, kbase, K_SS, 0)")
            for r in _request_statements(per_s):
                a("  " + r)
            a("}")

    a("// ---- consumers: 32 query rows x the key blocks of one key-split group each")
    if sp:
        a("EMH_PROLOGUE_REQUESTS()")
        a("EMH_LAND(-1)    // P: the Q tile and the first sub-steps of K have landed")
    else:
        a("EMH_BARRIER();  // P: the Q tile and the first sub-steps of K have landed")
    a("FRAG qf[D / 16];")
    a("{ const int qr_ = wq * 32 + lq;")
    a("  _Pragma(\"unroll\") for (int kk = 0; kk < D / 16; ++kk) qf[kk] = *(const FRAG*)(lds + Q_OFF_LDS + qr_ * (D * 2) + emh_kswz(qr_, kk * 2 + lh) * 16); }")
    a("f32x16 sc0 = emh_zero16, sc1 = emh_zero16;")
    a("bool resc = false; float alpha = 1.0f;  // a raised maximum waiting to be applied to the output accumulators")
    a("u32x4 pq0[2], pq1[2];  // the probabilities of a sub-block as the two operand fragments of its output MFMAs")
    a("_Pragma(\"unroll\") for (int s_ = 0; s_ < 2; ++s_) _Pragma(\"unroll\") for (int e_ = 0; e_ < 4; ++e_) { pq0[s_][e_] = 0u; pq1[s_][e_] = 0u; }")
    a.open("if (nact > 0)")
    a("// scores of sub-block 0 (K slot 0)")
    for kk in range(D // 16):
        _k_read(a, f"kf{kk}_", kk, 0)
    for kk in range(D // 16):
        a(f"sc1 = MFMA(kf{kk}_, qf[{kk}], {'sc1' if kk else 'emh_zero16'}, 0, 0, 0);")
    a.close()
    a("EMH_BARRIER();  // B0: slot 0 of the K ring may be requested again")
    a("EMH_PHASE_AT(0)")
    a("int t = 0;")
    a.open("if (nact >= 2)")
    a("// sub-block 0: softmax, and the scores of sub-block 1; no probabilities to multiply yet")
    _iteration(a, D, par=1, has_pv=False, kslot=1 % ring, vslot=None, t_expr="0" if sp else None, per_s=per_s)
    end("0")
    a("t = 1;")
    a("#pragma unroll 1")
    a.open(f"for (; t + {L} < nact; t += {L})")
    for i in range(L):
        _iteration(a, D, par=i & 1, has_pv=True, kslot=(i + 2) % ring, vslot=i % ring, t_expr=f"t + {i}" if sp else None, per_s=per_s)
        end(f"t + {i}")
    a.close()
    a("#pragma unroll 1")
    a.open("for (; t + 1 < nact; ++t)")
    a("const int kso = ((t + 1) % RING) * SLOT, vso = ((t + RING - 1) % RING) * SLOT;")
    _iteration(a, D, par=0, has_pv=True, kslot="kso", vslot="vso", t_expr="t" if sp else None, per_s=per_s)
    a("sc0 = sc1; pq1[0] = pq0[0]; pq1[1] = pq0[1];")
    end("t")
    a.close()
    a.close(" else { sc0 = sc1; }")
    a("EMH_PHASE_AT(1)")
    a.open("if (nact > 0)")
    a("// the wave's last active sub-block: the one a causal diagonal or the end of the keys can cut.  Run-time ring")
    a("// slots; the output MFMAs of the sub-block before it, the masked softmax, and after the barrier its own output MFMAs.")
    a("const int k0t = t * SUBK + grp * 32;")
    a("const int vso_prev = ((t + RING - 1) % RING) * SLOT, vso = (t % RING) * SLOT;")
    requests_now("t")
    a("if (resc) {  // left by the vote of the last steady iteration")
    for line in _RESCALE_IN_PLACE.split("\n"):
        a("  " + line)
    a("}")
    a.open("if (t > 0)")
    for j, (s, dt) in enumerate(jobs):
        _v_reads(a, f"vp{j}_", D, s, dt, "vso_prev")
    for j, (s, dt) in enumerate(jobs):
        _v_mfma(a, f"vp{j}_", dt, f"pq1[{s}]")
    a.close()
    # scores in sc0, probabilities back into pq1 (its old value has been consumed above)
    a.open("")
    a("float psum;")
    _classic_softmax(a, D, "sc0", "pq1", masked=True)
    a.close()
    end("t")  # V(t) has landed
    for j, (s, dt) in enumerate(jobs):
        _v_reads(a, f"vq{j}_", D, s, dt, "vso")
    for j, (s, dt) in enumerate(jobs):
        _v_mfma(a, f"vq{j}_", dt, f"pq1[{s}]")
    a.close()
    a("// sub-steps the causal mask leaves this wave out of")
    a.open("for (int i_ = nact; i_ < nsub; ++i_)")
    requests_now("i_")
    end("i_")
    a.close()


_HEAD = r"""
// K rows are XOR-swizzled per 256-byte bank line (KRPL rows of it), so the 16 rows
// a fragment read touches at one k position land in 16 different bank groups.
EMH_DEV int emh_kswz(int row, int c) { return c ^ ((row / KRPL) % CPR); }
// V keeps [key][d] order; its 16-byte chunks are XOR-swizzled in groups of four
// so the four consecutive key rows one transposing read touches sit in four
// different bank quarters.
#define EMH_VROT(row) (D >= 128 ? ((row) % 4) : (((row) >> 1) & 1))  /* 128-byte rows: two rows share a bank line */
EMH_DEV int emh_vswz(int row, int c) { return c ^ (EMH_VROT(row) << 2); }
EMH_DEV float emh_xor32(float v) { return __shfl_xor(v, 32, 64); }
typedef short emh_s16x4 __attribute__((ext_vector_type(4)));
#define EMH_TR16(p) __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) emh_s16x4*)(p))
#define KBYTES (32 * D * 2)            /* one key-split group's 32-key block */
#define SLOT (KVS * KBYTES)            /* one ring slot: a sub-step, the 32-key blocks of all key-split groups */
#define SUBK (KVS * 32)                /* keys per sub-step */
#define V_RING (RING * SLOT)           /* LDS: [K ring][V ring][Q tile] */
#define ST (SP ? NT : 256)             /* staging threads: every wave (SP), or waves 4-7 beside the consumer waves 0-3 */
#define QCHUNKS (BQ * CPR)             /* 16-byte chunks of a workgroup's Q (and O) tile */
#define RPL (D / 32 * 16)              /* output registers per lane */
#define RPG (RPL / KVS)                /* ... of which each key-split group finishes this many */
#define OSW (D / 4 < 32 ? D / 4 : 32)  /* rows over which the O tile's 8-byte slots are XOR-swizzled */
#define OACC(f) oacc[(f) / 16][(f) % 16]
#define CHUNKS (32 * D / 8)            /* 16-byte chunks of one 32-key block */
#define PER_S (KVS * CHUNKS / ST)      /* requests per staging thread, per operand and sub-step */
#ifndef EMH_ABLATE
#define EMH_ABLATE 0  /* -DEMH_ABLATE=1|2 through EMMY_HIPRTC_FLAGS: timing experiments whose results are not attention */
#endif
#ifndef EMH_STAMP
#define EMH_STAMP 0  /* -DEMH_STAMP=1: wave 0 of workgroup 0 sums the clocks its iterations spend per phase and leaves the sums in the output's first words */
#endif
#define EMH_PHASE_AT(i) if (EMH_STAMP == 2) { const unsigned long long now_ = __builtin_readcyclecounter(); st_acc[i] += (unsigned)(now_ - st_last); st_last = now_; st_acc[4 + (i)] = 1u; }  /* =2: totals per phase of a pass: prologue, loops, tail, close */
#define EMH_STAMP_AT(i) if (EMH_STAMP == 1) { const unsigned long long now_ = __builtin_readcyclecounter(); st_acc[i] += (unsigned)(now_ - st_last); st_last = now_; st_acc[4 + (i)] += 1u; }
#define EMH_BARRIER() { asm volatile("" ::: "memory"); __builtin_amdgcn_s_barrier(); asm volatile("" ::: "memory"); }
#define EMH_WAIT_VM(n) ((((n) & 0xF) | ((((n) >> 4) & 0x3) << 14)) | 0x0070)  /* vmcnt <= n, lgkmcnt = 0 */

extern "C" __global__ __launch_bounds__(NT) void KNAME(const ELT* __restrict__ Q, const ELT* __restrict__ Kp,
                                                      const ELT* __restrict__ Vp, ELT* __restrict__ Op) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  const int tid = threadIdx.x, lane = tid % 64;
  const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
  const bool consumer = SP || wave < 4;
  const int grp = (wave % (WQ * KVS)) / WQ, wq = (wave % (WQ * KVS)) % WQ;  // consumers: key-split group, row group
  const int lq = lane % 32, lh = lane / 32;
  const f32x16 emh_zero16 = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
  // Workgroup ids go round-robin over the XCDs, each with its own L2: consecutive logical ids (the query
  // blocks of one head, then the next head of the same KV group) are dealt to one XCD.
  const int bid = GRID % XCDS == 0 ? (int)(blockIdx.x % XCDS) * (GRID / XCDS) + (int)(blockIdx.x / XCDS) : (int)blockIdx.x;
  const int slot_id = bid % QSLOTS;
  const int head = (bid / QSLOTS) % HQ;
  const int batch = bid / (QSLOTS * HQ);
  const int kvh = head / GROUP;
  const ELT* qbase = Q + Q_OFF + (long)batch * Q_SB + (long)head * Q_SH;
  const ELT* kbase = Kp + K_OFF + (long)batch * K_SB + (long)kvh * K_SH;
  const ELT* vbase = Vp + V_OFF + (long)batch * V_SB + (long)kvh * V_SH;
  const unsigned lds0 = emh_lds_addr(lds);
  // ds_read_b64_tr_b16: within 16 lanes, lane i receives element (i % 4) of the 8-byte chunks addressed by
  // lanes i/4, i/4 + 4, i/4 + 8, i/4 + 12: lane i points at key row (i / 4) and d-chunk 4*(i % 4) of its half
  // tile and receives four consecutive keys of its own d.
  const int i16 = lane % 16, q4 = i16 / 4;
  const unsigned char* vb[TG];
  #pragma unroll
  for (int T = 0; T < TG; ++T) vb[T] = lds + V_RING + grp * KBYTES + (4 * lh + q4) * (D * 2) + ((lane % 32) / 16) * 32 + (i16 % 4) * 8 + ((T ^ EMH_VROT(q4)) * 64);
  const unsigned char* kb[D / 16];
  #pragma unroll
  for (int kk = 0; kk < D / 16; ++kk) kb[kk] = lds + grp * KBYTES + lq * (D * 2) + emh_kswz(lq, kk * 2 + lh) * 16;
  // ---- staging.  A sub-step's K (or V) chunks are dealt over the ST staging threads; every wave-level load fills 64
  // consecutive 16-byte LDS slots, so the swizzle is applied by choosing which global chunk each lane fetches.  A request
  // is a scalar base (the operand plane moved along the keys to the sub-step, plus the request's row offset: whole
  // multiples of 16 rows, which leave the swizzle of a lane's chunk unchanged), one loop-invariant 32-bit lane offset per
  // operand and a scalar LDS target; only a sub-step that hangs over the end of the keys clamps its rows per lane.
  const int stid = SP ? tid : tid - 256, sw = SP ? wave : wave - 4;
  const int st_row = stid / CPR, st_pos = stid % CPR;
  const unsigned kvo0 = (unsigned)(st_row * K_SS + emh_kswz(st_row, st_pos) * 8) * 2u;
  const unsigned vvo0 = (unsigned)(st_row * V_SS + emh_vswz(st_row, st_pos) * 8) * 2u;
  #define EMH_SUB_BASES(tag, s_, base_, stride_, ring0_) \
    const int sub_##tag = (s_); \
    const bool ok_##tag = sub_##tag >= 0 && sub_##tag < nsub; \
    const bool whole_##tag = SKV % SUBK == 0 || (sub_##tag + 1) * SUBK <= SKV; \
    const unsigned char* sb_##tag = emh_uniform((const unsigned char*)(base_) + (long)sub_##tag * SUBK * (stride_) * 2); \
    const unsigned lb_##tag = emh_uniform(lds0 + (ring0_) + ((sub_##tag + RING) % RING) * SLOT + sw * 1024);
  #define EMH_REQ_I(tag, i, voff_, base_, stride_, swz_, ring0_) { \
    const int g_ = ((i) * ST) / CHUNKS, ro_ = (((i) * ST) % CHUNKS) / CPR; \
    if (ok_##tag) { \
      if (whole_##tag) { \
        emh_dma16s(sb_##tag + (long)(g_ * 32 + ro_) * (stride_) * 2, voff_, lb_##tag + g_ * KBYTES + (((i) * ST) % CHUNKS) * 16); \
      } else { \
        long krow_ = (long)sub_##tag * SUBK + g_ * 32 + ro_ + st_row; \
        if (krow_ > SKV - 1) krow_ = SKV - 1; \
        emh_dma16((base_) + krow_ * (stride_) + swz_(st_row + ro_, st_pos) * 8, lds + (ring0_) + (sub_##tag % RING) * SLOT + g_ * KBYTES + (((i) * ST) % CHUNKS) * 16 + sw * 1024); } } }
  // Requests retire in issue order.  In "iteration" tau (the prologue is iterations -RING .. -1) a staging thread issues
  // V(tau + RING - 2) and then K(tau + RING), where they exist.  The barrier that ends iteration t_ needs K(t_ + 2) and
  // V(t_): everything issued up to iteration t_ + 2 - RING.  What may still be outstanding is what iterations
  // t_ + 3 - RING .. t_ issued.  Reaching the count does not yet make direct-to-LDS data visible to other waves: an LDS
  // read of this wave queues behind its own writes, so waiting for it orders them before the barrier.
  #define EMH_LAND(t_) { \
    int cnt_ = 0; \
    _Pragma("unroll") for (int d_ = 0; d_ < RING - 2; ++d_) { \
      const int tau_ = (t_) - d_; \
      cnt_ += (tau_ + RING - 2 >= 0 && tau_ + RING - 2 < nsub) + (tau_ + RING < nsub); } \
    switch (cnt_) { \
      case 0: __builtin_amdgcn_s_waitcnt(EMH_WAIT_VM(0)); break; \
      case 1: __builtin_amdgcn_s_waitcnt(EMH_WAIT_VM(PER_S)); break; \
      case 2: __builtin_amdgcn_s_waitcnt(EMH_WAIT_VM(2 * PER_S)); break; \
      case 3: __builtin_amdgcn_s_waitcnt(EMH_WAIT_VM(3 * PER_S)); break; \
      default: __builtin_amdgcn_s_waitcnt(EMH_WAIT_VM(4 * PER_S)); break; } \
    emh_lds_publish(lds + tid * 4); \
    EMH_BARRIER(); }
  // the Q tile (whole rows per instruction, swizzled like a K block) and the sub-steps that fill the rings before the loop
  #define EMH_PROLOGUE_REQUESTS() { \
    _Pragma("unroll") for (int c0 = 0; c0 < QCHUNKS; c0 += ST) { \
      if (QCHUNKS % ST == 0 || c0 + (stid - lane) < QCHUNKS) {  /* whole waves: QCHUNKS is a multiple of 64 */ \
        const int r_ = (c0 + stid) / CPR, p_ = (c0 + stid) % CPR; \
        const int qr_ = q0 + r_ < SQ ? q0 + r_ : SQ - 1; \
        emh_dma16(qbase + (long)qr_ * Q_SS + emh_kswz(r_, p_) * 8, lds + Q_OFF_LDS + (c0 + stid - lane) * 16); } } \
    _Pragma("unroll") for (int tau = -RING; tau < 0; ++tau) { \
      EMH_SUB_BASES(v, tau + RING - 2, vbase, V_SS, V_RING) EMH_SUB_BASES(k, tau + RING, kbase, K_SS, 0) \
      _Pragma("unroll") for (int i = 0; i < PER_S; ++i) EMH_REQ_I(v, i, vvo0, vbase, V_SS, emh_vswz, V_RING) \
      _Pragma("unroll") for (int i = 0; i < PER_S; ++i) EMH_REQ_I(k, i, kvo0, kbase, K_SS, emh_kswz, 0) } }
  unsigned st_acc[8] = {0u, 0u, 0u, 0u, 0u, 0u, 0u, 0u};
  unsigned long long st_last = EMH_STAMP ? __builtin_readcyclecounter() : 0ull;
  #pragma unroll 1
  for (int pass = 0; pass < (PAIR ? 2 : 1); ++pass) {
  if (PAIR && pass) __syncthreads();  // every thread is done copying the first block's O tile out of LDS
  const int qb = pass == 0 ? (QBLOCKS - 1) - slot_id : slot_id;
  const int q0 = qb * BQ;
  const int qw0 = q0 + wq * 32;
  const int qrow = qw0 + lq;
  int keys = SKV;
  if (CAUSAL) {
    const int lim = (q0 + BQ - 1 < SQ - 1 ? q0 + BQ - 1 : SQ - 1) + 1;
    if (lim < keys) keys = lim;
  }
  const int nsub = __builtin_amdgcn_readfirstlane((keys + SUBK - 1) / SUBK);
  // sub-blocks this wave takes part in: those of its key-split group that start inside the keys and, under a
  // causal mask, not beyond its last row
  int nact = SKV > grp * 32 ? (SKV - grp * 32 + SUBK - 1) / SUBK : 0;
  if (CAUSAL) {
    const int cl = qw0 + 31 - grp * 32 >= 0 ? (qw0 + 31 - grp * 32) / SUBK + 1 : 0;
    if (cl < nact) nact = cl;
  }
  if (nsub < nact) nact = nsub;
  nact = __builtin_amdgcn_readfirstlane(nact);
  if (EMH_ABLATE == 2) nact = 0;  // measurement only: staging alone, the consumers just keep the barriers

  f32x16 oacc[D / 32];
  #pragma unroll
  for (int t_ = 0; t_ < D / 32; ++t_) oacc[t_] = emh_zero16;
  const emh_s16x4 emh_abl4 = {(short)lane, 1, 2, 3};  // (measurement only: stands in for fragment reads under -DEMH_ABLATE=4)
  float m_ref = -1.0e30f, l_run = 0.0f;

  if (consumer) {
    __builtin_amdgcn_s_setprio(CONSUMER_PRIO);
"""

_STAGER = r"""
    __builtin_amdgcn_s_setprio(0);
  } else {
    // ---- stagers: every direct-to-LDS request of the workgroup
    EMH_PROLOGUE_REQUESTS()
    EMH_LAND(-1)     // P
    EMH_BARRIER();   // B0
    #pragma unroll 1
    for (int t = 0; t < nsub; ++t) {
      if (EMH_ABLATE != 1) {  // (1, measurement only: no requests inside the loop, the consumers work on what the prologue left)
        EMH_SUB_BASES(v, t + RING - 2, vbase, V_SS, V_RING) EMH_SUB_BASES(k, t + RING, kbase, K_SS, 0)
        #pragma unroll
        for (int i = 0; i < PER_S; ++i) EMH_REQ_I(v, i, vvo0, vbase, V_SS, emh_vswz, V_RING)
        #pragma unroll
        for (int i = 0; i < PER_S; ++i) EMH_REQ_I(k, i, kvo0, kbase, K_SS, emh_kswz, 0)
      }
      EMH_LAND(t)
    }
  }
  EMH_BARRIER();  // every wave is done reading the rings: the close may overwrite them
  EMH_PHASE_AT(2)

  // ---- close.  The key-split groups share the final combine: group g finishes registers [g*RPG, (g+1)*RPG) of its
  // rows' RPL output registers.  Every group parks the registers the others own, and its (m, l); after one barrier
  // each combines its share with the same exp-family merge the streaming loop uses, scales by 1/l and puts the 16-bit
  // result into the O tile in LDS, which leaves through 16-byte stores of whole rows by all eight waves.
  if (KVS > 1 && consumer) {
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
  }
  if (KVS > 1) __syncthreads();
  if (consumer) {
  #pragma unroll
  for (int g = 0; g < KVS; ++g) {
    if (g == grp) {
      float a_own = 1.0f, l_tot = l_run;
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
        PACK4 y;
        #pragma unroll
        for (int j = 0; j < 4; ++j) y[j] = (ELT)(acc[j] * inv);
        // Registers 4i .. 4i+3 of tile T are d = 32*T + 8*i + 4*lh + (0..3): 8-byte slot 8*T + 2*i + lh of the row.
        const int f = g * RPG + 4 * r4;
        const int sl = 8 * (f / 16) + 2 * ((f % 16) / 4) + lh;
        *(PACK4*)(lds + O_OFF_LDS + orow * (D * 2) + ((sl ^ (orow % OSW)) * 8)) = y;
      }
    }
  }
  }
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
        if (q0 + r < SQ) *(u32x4*)(obase + (long)(q0 + r) * O_SS + pc * 8) = y;
      }
    }
  }
  EMH_PHASE_AT(3)
  }
  if (EMH_STAMP && bid == 0 && tid == 0) {  // over the 16 bytes this thread stored itself (row 0 of the first head, in the pair's second pass)
    #pragma unroll
    for (int i = 0; i < 4; ++i) ((float*)(Op + O_OFF))[i] = (float)st_acc[i] / (float)(st_acc[4 + i] ? st_acc[4 + i] : 1u);
  }
}
"""


def _shape(body: Flash) -> tuple[bool, int, tuple[int, ...]]:
    """``(self-staging, consumer waves, ring depths to try)`` of the form ``body`` asks for."""
    sp = bool(getattr(body, "sp", False))
    return sp, (8 if sp else CONSUMER_WAVES), ((4, 3, 2) if sp else (4, 3))


def ws_supported(body: Flash, ctx: Context = Context()) -> str | None:
    """``None`` when the software-pipelined forms (``ws``: four consumer waves and four staging waves; ``sp``: eight
    consumer waves that stage for themselves) can take ``body`` with its current ``waves`` / ``kv_split``; else why not."""
    sp, consumers, rings = _shape(body)
    if body.dtype.name not in ("bf16", "f16"):
        return "16-bit operands only"
    if body.head_dim not in (64, 128) or body.head_dim_real not in (None, body.head_dim):
        return "head_dim 64 or 128"
    if body.mask is not None:
        return "no mask operand"
    if getattr(body, "sym", None) is not None and body.sym.fields:
        return "lengths known when the kernel is built"
    if body.waves * body.kv_split != consumers:
        return f"row groups x key-split groups must be {consumers} ({'two consumer waves' if sp else 'one consumer wave'} per SIMD)"
    if (body.head_dim // 32 * 16) % (4 * body.kv_split):
        return "the key-split groups cannot share a lane's output registers"
    if (body.kv_split * 32 * body.head_dim // 8) % (512 if sp else 256):
        return "a sub-step's chunks must be a multiple of the staging threads"
    try:
        ws_lds_plan(body.waves, body.kv_split, body.head_dim, ctx.lds_bytes_per_cu, rings)
    except LoweringError as exc:
        return str(exc)
    return None


def emit_flash_ws(body: Flash, name: str, ctx: Context = Context()) -> HipOp:
    why = ws_supported(body, ctx)
    if why is not None:
        raise LoweringError(f"flash/{'sp' if getattr(body, 'sp', False) else 'ws'}: {why}")
    sp, consumers, rings = _shape(body)
    D = body.head_dim
    if body.q_heads % body.kv_heads:
        raise LoweringError("flash: q heads must be a multiple of kv heads")
    waves, kvs = body.waves, body.kv_split
    BQ = 32 * waves
    NT = 64 * (consumers if sp else CONSUMER_WAVES + STAGER_WAVES)
    plan = ws_lds_plan(waves, kvs, D, ctx.lds_bytes_per_cu, rings)
    for st, heads in ((body.q_strides, body.q_heads), (body.k_strides, body.kv_heads), (body.v_strides, body.kv_heads), (body.o_strides, body.q_heads)):
        if st[2] % 8 or (heads > 1 and st[1] % 8) or (body.batch > 1 and st[0] % 8):
            raise LoweringError("flash: batch / head / sequence strides must keep 16-byte alignment")
    if any(o % 8 for o in (body.q_offset, body.k_offset, body.v_offset, body.o_offset)):
        raise LoweringError("flash: offsets break 16-byte alignment")
    qblocks = -(-body.q_len // BQ)
    pair = bool(body.pair)
    if pair and not (body.causal and qblocks % 2 == 0):
        raise LoweringError("flash: pairing mirrored query blocks needs a causal mask and an even block count")
    qslots = qblocks // 2 if pair else qblocks
    bf16 = body.dtype.name == "bf16"
    grid = qslots * body.q_heads * body.batch
    per_s = kvs * (32 * D // 8) // NT if sp else 0
    defs = {
        "KNAME": name, "NT": NT, "SP": 1 if sp else 0, "D": D, "BQ": BQ, "KVS": kvs, "WQ": waves, "RING": plan["ring"],
        "CPR": D // 8, "KRPL": max(1, 16 // (D // 8)), "TG": min(4, D // 32),
        "SQ": body.q_len, "SKV": body.kv_len, "HQ": body.q_heads, "GROUP": body.q_heads // body.kv_heads,
        "QBLOCKS": qblocks, "QSLOTS": qslots, "PAIR": 1 if pair else 0, "CAUSAL": 1 if body.causal else 0,
        "Q_OFF_LDS": plan["q_off"], "O_OFF_LDS": plan["o_off"], "PARK_ML": plan["park_ml"],
        "SCALE_LOG2": float_literal(body.scale * math.log2(math.e)),
        "Q_SB": body.q_strides[0], "Q_SH": body.q_strides[1], "Q_SS": body.q_strides[2], "Q_OFF": body.q_offset,
        "K_SB": body.k_strides[0], "K_SH": body.k_strides[1], "K_SS": body.k_strides[2], "K_OFF": body.k_offset,
        "V_SB": body.v_strides[0], "V_SH": body.v_strides[1], "V_SS": body.v_strides[2], "V_OFF": body.v_offset,
        "O_SB": body.o_strides[0], "O_SH": body.o_strides[1], "O_SS": body.o_strides[2], "O_OFF": body.o_offset,
        "PACK2": rt.vector_type(body.dtype.name, 2)[0],
        "ELT": rt.type_name(body.dtype.name), "FRAG": rt.vector_type(body.dtype.name, 8)[0], "PACK4": rt.vector_type(body.dtype.name, 4)[0],
        "MFMA": "__builtin_amdgcn_mfma_f32_32x32x16_bf16" if bf16 else "__builtin_amdgcn_mfma_f32_32x32x16_f16",
        "EXP2(x)": f"(EMH_ABLATE == 3 ? (x) : {rt.intrinsic('fast_exp2', 'f32')}(x))",
        "RESCALE_SLACK": "8.0f",
        "CONSUMER_PRIO": 0 if sp else 1,
        "GRID": grid, "XCDS": ctx.xcds,
    }  # fmt: skip
    form = "self-staging, software-pipelined" if sp else "wave-specialised"
    head = f"// {name}: B={body.batch} Hq={body.q_heads} Hkv={body.kv_heads} Sq={body.q_len} Skv={body.kv_len} D={D} causal={body.causal} ({form})\n"
    head += "".join(f"#define {k} {v}\n" for k, v in defs.items())
    lines = _Lines()
    lines.depth = 2
    _consumer(lines, D, plan["ring"], per_s)
    source = prelude.header(prelude.DMA) + head + _HEAD + "\n".join(lines.out) + _STAGER
    return HipOp(
        kernel_source=source,
        kernel_name=name,
        arg_order=(body.q, body.k, body.v, body.out),
        grid=((grid,), (1,), (1,)),
        block=((NT,), (1,), (1,)),
        lds_bytes=plan["bytes"],
        comment=f"flash/{'sp' if sp else 'ws'} Sq={body.q_len} Skv={body.kv_len} D={D} causal={body.causal} waves={waves} split={kvs} pair={int(pair)} ring={plan['ring']}",
        algo_bytes=body.algo_bytes(),
        algo_flops=body.algo_flops(),
        knobs={"FLASH": f"w{waves}/kv32/s{kvs}" + ("/p" if pair else "") + ("/sp" if sp else "/ws")},
    )


__all__ = ["emit_flash_ws", "ws_lds_plan", "ws_supported"]
