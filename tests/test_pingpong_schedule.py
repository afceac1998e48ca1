"""The barrier schedule of ``STAGE .../pp`` (emit.contraction._emit_pingpong_loop), checked on the emitted text.

The k loop runs three roles (two consumer groups and the staging waves) through different instruction streams
that meet at one workgroup barrier a slab.  A miscount hangs the workgroup, a misplaced request overwrites a slab
that is still being read, a wait count that is too large lets a wave read a slab that has not landed — none of
which a CPU can run, all of which follow from the text.  The emitted loop is expanded role by role into events
(request, wait-until-landed, fragment read, MFMA step, barrier) and replayed period by period:

* every role executes the same number of barriers;
* a request goes into the ring buffer of its slab, and only after the barrier that follows the last read of the
  slab it replaces, by both groups;
* a fragment read finds its slab complete: every request of it older than the producer's wait count allowed, at a
  barrier before the read;
* each group reads and computes slab j in period j (group 0 reads one period ahead), every slab exactly once.
"""

from __future__ import annotations

import re

import pytest

from deplodock_amd.emit.contraction import _emit_pingpong_loop


def interp(lines, R, KT):
    ev = []
    def sub(e, kt): return eval(e.replace('DEPTH', str(R)), {}, {'kt': kt})
    def stmt(ln, kt):
        ln = ln.strip()
        m = re.search(r'EMH_DPART_[AB]\((.*), (.*), (\d+)\);', ln)
        if m: ev.append(('dma', sub(m.group(1), kt), sub(m.group(2), kt))); return
        m = re.match(r'EMH_READ\((\d+), (.*), (\d+)\);', ln)
        if m: ev.append(('read', sub(m.group(2), kt), int(m.group(3)))); return
        m = re.match(r'EMH_SLAB_SYNC\((\d+)\);', ln)
        if m: ev.append(('land', int(m.group(1)))); ev.append(('bar',)); return
        if 'EMH_PHASE_END()' in ln and not ln.startswith('#define'): ev.append(('bar',)); return
        if ln.startswith('EMH_MMA'): ev.append(('mma',)); return
    def block(i, kt):
        """run lines from i until the matching close; returns index after"""
        while i < len(lines):
            ln = lines[i].strip()
            m = re.match(r'for \(int kt = 0; kt < (\d+); \+\+kt\) \{', ln)
            if m:
                end = None
                for k in range(int(m.group(1))):
                    end = block(i + 1, k)
                if int(m.group(1)) == 0:
                    end = skip(i + 1)
                i = end; continue
            m = re.match(r'if \((.*)\) \{$', ln)
            if m:
                if sub(m.group(1), kt): i = block(i + 1, kt)
                else: i = skip(i + 1)
                continue
            if ln == '{': i = block(i + 1, kt); continue
            if ln.startswith('}'):
                stmt(ln[1:], kt)   # e.g. "EMH_PHASE_END(); }" handled below; "} // c" nothing
                return i + 1
            if ln.endswith('}') and '{' not in ln:
                stmt(ln[:-1], kt); return i + 1
            stmt(ln, kt); i += 1
        return i
    def skip(i):
        depth = 1
        while depth:
            ln = lines[i].strip()
            depth += ln.count('{') - ln.count('}')
            i += 1
        return i
    block(0, None)
    return ev

def check(KT, R, nparts=10):
    out = []
    parts = [f"EMH_DPART_A({{slab}}, {{buf}}, {i});" for i in range(4)] + [f"EMH_DPART_B({{slab}}, {{buf}}, {i});" for i in range(nparts - 4)]
    _emit_pingpong_loop(out.append, KT=KT, KS=2, depth=R, parts=parts)
    text = "\n".join(out).split("\n")
    i0 = next(i for i, l in enumerate(text) if l.strip().startswith('if (role == 2) {'))
    i1 = next(i for i, l in enumerate(text) if l.strip().startswith('} else if (role == 0) {'))
    i2 = next(i for i, l in enumerate(text) if l.strip().startswith('} else {'))
    prod, g0, g1 = interp(text[i0 + 1:i1], R, KT), interp(text[i1 + 1:i2], R, KT), interp(text[i2 + 1:len(text) - 1], R, KT)
    nb = [sum(1 for e in x if e[0] == 'bar') for x in (prod, g0, g1)]
    assert nb[0] == nb[1] == nb[2] == KT + 1, (KT, R, nb)
    issued = [s for s in range(min(R - 1, KT)) for _ in range(nparts)]
    visible = {0}
    buf_slab = {s % R: s for s in range(min(R - 1, KT))}
    last_read = {}
    pos = [0, 0, 0]
    roles = (prod, g0, g1)
    mma = [0, 0]
    for phase in range(KT + 1):
        newly = None
        for r in range(3):
            while True:
                e = roles[r][pos[r]]; pos[r] += 1
                if e[0] == 'bar': break
                if e[0] == 'dma':
                    assert r == 0
                    _, slab, buf = e
                    assert 0 <= slab < KT and buf == slab % R, (KT, R, e)
                    old = buf_slab.get(buf)
                    if old is not None and old != slab:
                        for g in (1, 2):
                            assert (g, old) in last_read and last_read[(g, old)] < phase, (KT, R, 'overwrite before last read', e, phase, last_read)
                    buf_slab[buf] = slab
                    issued.append(slab)
                elif e[0] == 'read':
                    slab = buf_slab[e[1]]
                    assert slab in visible, (KT, R, 'read of a slab not complete', e, slab, phase)
                    last_read[(r, slab)] = phase
                    # list index `phase` is phase number phase - 1
                    want = phase if r == 1 else phase - 1
                    assert slab == want, (KT, R, 'wrong slab', r, phase, slab, want)
                elif e[0] == 'land':
                    assert r == 0
                    done = issued[:len(issued) - e[1]] if e[1] else list(issued)
                    newly = {s for s in set(done) if done.count(s) == nparts}
                elif e[0] == 'mma':
                    mma[r - 1] += 1
        if newly is not None:
            visible |= newly
    assert all(p == len(x) for p, x in zip(pos, roles)), (KT, R, pos)
    assert mma == [2 * KT, 2 * KT], (KT, R, mma)
    assert sorted(set(issued)) == list(range(KT)) and all(issued.count(s) == nparts for s in range(KT)), (KT, R)
    for s in range(KT):
        for g in (1, 2):
            assert (g, s) in last_read



@pytest.mark.parametrize("depth", [3, 4, 5])
def test_every_slab_count_replays_without_a_hazard(depth):
    for slabs in range(1, 24):
        for requests in (5, 10):
            check(slabs, depth, requests)


def test_the_replay_sees_a_wrong_wait_count_and_a_wrong_buffer(monkeypatch):
    """The checker itself: mutated emitters (a wait that allows one slab too many in flight, a request into the
    next buffer, group 0 reading the slab it just computed) must each trip it."""
    import inspect

    import deplodock_amd.emit.contraction as C

    src = inspect.getsource(C._emit_pingpong_loop)
    mutants = {
        "late landing": src.replace("return max(0, last - (q + 2)) * len(parts)", "return (max(0, last - (q + 2)) + 1) * len(parts)"),
        "wrong buffer": src.replace('buf=f"((({q}) + {R - 1}) % DEPTH)"', 'buf=f"((({q}) + {R}) % DEPTH)"'),
        "wrong slab": src.replace('    fetch("kt + 1")\n', '    fetch("kt")\n'),
    }
    for what, mutant in mutants.items():
        assert mutant != src, what
        ns: dict = {}
        exec(mutant, dict(vars(C)), ns)
        monkeypatch.setitem(globals(), "_emit_pingpong_loop", ns["_emit_pingpong_loop"])
        with pytest.raises(AssertionError):
            for slabs in range(1, 12):
                check(slabs, 4)
