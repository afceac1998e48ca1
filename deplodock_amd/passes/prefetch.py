"""Weight prefetch across launches: a kernel's spare lanes touch the *next* launch's weights.

A model whose weights exceed the last-level cache streams every weight matrix from HBM exactly once per forward pass, and
at decode sizes each launch is a latency chain: its first loads miss all the way to HBM while most of the machine idles,
then the next launch starts cold again.  The launches of a program are known when it is lowered, so each kernel can be
given the address of the constant its successor will stream and a few lanes that do nothing but touch it — one 4-byte
load per 128-byte line, results unused — while the kernel's own waves work.  The successor then finds its weights in
the L2 of the XCD that will ask for them (when its workgroup -> rows mapping is known: ``HipOp.weight_slices``) or at
least in the memory-side cache.

Two forms, both a textual change of the rendered kernel (a new parameter, a guard in front of the body, a larger launch):

* ``wave``: every workgroup gets one more wave (``threadIdx.x >= T``) that prefetches and ends; the kernel's own waves never
  see it (a wave that has ended does not count for barriers).  For kernels whose workgroups cover the machine;
* ``workgroups``: the grid gets extra workgroups (``blockIdx.x >= G``) that prefetch and end.  For kernels with few
  workgroups and little LDS (an extra workgroup asks for the launch's LDS size too, so beside a large one it would wait
  for a CU instead of running at once).

A load returns into its destination register whenever the memory system gets to it, and the compiler knows nothing of
that for a load written as an ``asm`` statement: it would hand the register to the next value it computes (an address of
the following iteration, overwritten in mid-use when the data arrives).  So every prefetch load of a wave names the same
variable as input *and* output — one register that stays allocated from before the first load until the wave has waited
for all of them — and the wave ends only after that wait.

The pass runs after lowering and is on by default only where it can pay: a program whose constants exceed the
last-level cache, and in it a consumer between ``MIN_INTENSITY`` and ``MAX_INTENSITY`` flop per byte (``EMMY_PREFETCH=1`` /
``0`` force it on for every consumer / off).  Measured on the 28-layer Qwen3-0.6B-architecture model (880 MB of weights;
us per forward as one graph replay, without / with): 1 token 735 / 776, 16 tokens 842 / 846, 32 tokens 959 / 929,
128 tokens 1090 / 1019, 256 tokens 1284 / 1180, 384 tokens 1477 / 1459, 512 tokens 1519 / 1489 — below about 32 rows a launch
is too short to hide its successor's lines behind and the extra wave or workgroups cost more than the warm start gains; from
512 rows on the consumers are busy with arithmetic and the gain is down to 1-2 % (an upper bound of 200 flop per byte left the
256-token gate / up projection, at 219, without its prefetch: 1234).
"""

from __future__ import annotations

import hashlib
import math
import re

from deplodock_amd import config
from deplodock_amd.context import Context
from deplodock_amd.graph import Graph
from deplodock_amd.ir.base import ConstantOp
from deplodock_amd.ir.hip import HipOp

#: constants smaller than this are not worth a prefetch (they arrive within one round trip anyway)
MIN_BYTES = 512 * 1024
#: ... and larger ones would push the running kernel's own lines out of the caches
MAX_BYTES = 64 * 1024 * 1024
#: the memory-side cache: programs whose constants fit it find them there after the first pass
LAST_LEVEL_CACHE_BYTES = 256 * 1024 * 1024
#: flop per byte of the consumer (about its row count, for a weight-streaming contraction) between which a prefetch pays
MIN_INTENSITY = 24.0
MAX_INTENSITY = 400.0
#: LDS up to which extra workgroups run beside the kernel's own on a CU (two of them fit a CU's 160 KiB)
_SMALL_LDS = 76 * 1024
LINE = 128


def _static_int(spec) -> int | None:
    if isinstance(spec, int):
        return spec
    total = 1
    for f in spec:
        if not isinstance(f, int):
            return None
        total *= f
    return total


def _signature(src: str, name: str) -> tuple[int, int, int] | None:
    """``(index of the parameter list's closing parenthesis, index of the body's opening brace, index of the
    ``__launch_bounds__`` argument's closing parenthesis)`` of kernel ``name`` in ``src``."""
    g = src.find("__global__")
    if g < 0 or src.find("__global__", g + 1) >= 0:
        return None  # one kernel per source
    lb = src.find("__launch_bounds__(", g)
    v = src.find(" void ", g)
    if lb < 0 or v < 0 or lb > v:
        return None
    lb_close = src.find(")", lb)
    open_ = src.find("(", v)
    depth, i = 0, open_
    while i < len(src):
        if src[i] == "(":
            depth += 1
        elif src[i] == ")":
            depth -= 1
            if depth == 0:
                break
        i += 1
    brace = src.find("{", i)
    if depth != 0 or brace < 0 or src[i + 1 : brace].strip():
        return None
    return i, brace, lb_close


def _guard(form: str, own: int, prefetchers: int, lanes: int, nbytes: int, slices: tuple[int, int] | None, xcds: int) -> str:
    """The statements in front of the kernel body.  ``own``: the kernel's own threads per workgroup (``wave``) or its
    own workgroups (``workgroups``); ``prefetchers`` of ``lanes`` lanes each share the lines."""
    lines = -(-nbytes // LINE)
    if form == "wave":
        head = f"  if (threadIdx.x >= {own}u) {{\n    const unsigned p_ = blockIdx.x, t_ = threadIdx.x - {own}u;\n"
    else:
        head = f"  if (blockIdx.x >= {own}u) {{\n    const unsigned p_ = blockIdx.x - {own}u, t_ = threadIdx.x;\n"
    body = "    // touch the next launch's weights, one load per 128-byte line, all into one register that nothing else may take\n    unsigned v_ = 0u;\n"
    if slices is not None and prefetchers >= xcds:
        sl, ns = slices  # lines per slice, slices; the consumer's workgroup j reads slice j and runs on XCD j % xcds
        q_total = prefetchers // xcds
        body += (
            f"    const unsigned xcd_ = blockIdx.x % {xcds}u, q_ = p_ / {xcds}u;\n"
            f"    const unsigned nsx_ = xcd_ < {ns}u ? ({ns}u - xcd_ + {xcds - 1}u) / {xcds}u : 0u;  // slices xcd_, xcd_ + {xcds}, ...\n"
            f"    if (q_ < {q_total}u)\n"
            f"    for (unsigned i_ = q_ * {lanes}u + t_; i_ < nsx_ * {sl}u; i_ += {q_total * lanes}u) {{\n"
            f"      const unsigned line_ = (xcd_ + {xcds}u * (i_ / {sl}u)) * {sl}u + i_ % {sl}u;\n"
            f"      if (line_ < {lines}u) asm volatile(\"global_load_dword %0, %1, off\" : \"+v\"(v_) : \"v\"(emh_pf + (unsigned long)line_ * {LINE // 4}));\n"
            "    }\n"
        )
    else:
        body += (
            f"    for (unsigned line_ = p_ * {lanes}u + t_; line_ < {lines}u; line_ += {prefetchers * lanes}u) {{\n"
            f"      asm volatile(\"global_load_dword %0, %1, off\" : \"+v\"(v_) : \"v\"(emh_pf + (unsigned long)line_ * {LINE // 4}));\n"
            "    }\n"
        )
    return head + body + "    asm volatile(\"s_waitcnt vmcnt(0)\" : \"+v\"(v_));\n    return;\n  }\n"


def with_prefetch(op: HipOp, target: str, nbytes: int, slices: tuple[int, int] | None, ctx: Context) -> HipOp | None:
    """``op`` with lanes that touch ``nbytes`` of buffer ``target`` (its last pointer argument), or ``None`` when the
    kernel does not take the change (a launch sized at run time, a kernel that reads its own launch size)."""
    gx, gy, gz = (_static_int(s) for s in op.grid)
    bx, by, bz = (_static_int(s) for s in op.block)
    if None in (gx, gy, gz, bx, by, bz) or gy != 1 or gz != 1 or by != 1 or bz != 1 or op.runtime_args:
        return None
    src = op.kernel_source
    if "gridDim" in src or "blockDim" in src or "emh_pf" in src:
        return None
    sig = _signature(src, op.kernel_name)
    if sig is None:
        return None
    close, brace, lb_close = sig
    few = gx * 2 <= ctx.compute_units
    if few and op.lds_bytes <= _SMALL_LDS and bx >= 64:
        form, extra = "workgroups", ctx.compute_units
        guard = _guard(form, gx, extra, bx, nbytes, slices, ctx.xcds)
        grid, block = ((gx + extra,), (1,), (1,)), op.block
    elif bx + 64 <= 1024 and bx % 64 == 0:
        form = "wave"
        guard = _guard(form, bx, gx, 64, nbytes, slices, ctx.xcds)
        grid, block = op.grid, ((bx + 64,), (1,), (1,))
    else:
        return None
    new_src = src[:brace + 1] + "\n" + guard + src[brace + 1 :]
    new_src = new_src[:close] + ", const unsigned* __restrict__ emh_pf" + new_src[close:]
    if form == "wave":
        new_src = new_src[:lb_close] + " + 64" + new_src[lb_close:]
    digest = hashlib.sha1(new_src.encode()).hexdigest()[:4]
    name = f"{op.kernel_name}_pf{digest}"
    new_src = re.sub(rf"\b{re.escape(op.kernel_name)}\b", name, new_src)
    new = HipOp(
        kernel_source=new_src, kernel_name=name, arg_order=(*op.arg_order, target), grid=grid, block=block, lds_bytes=op.lds_bytes,
        zero_outputs=op.zero_outputs, comment=op.comment + f" + prefetch of {target} ({form})", runtime_args=op.runtime_args,
        algo_bytes=op.algo_bytes, algo_flops=op.algo_flops,
    )  # fmt: skip
    for attr in ("knobs", "source", "weight_slices"):
        if hasattr(op, attr):
            setattr(new, attr, getattr(op, attr))
    new.knobs = {**getattr(op, "knobs", {}), "PREFETCH": form}
    return new


def _nbytes(node) -> int | None:
    shape = node.output.shape
    if not all(isinstance(d, int) for d in shape):
        return None
    return math.prod(int(d) for d in shape) * node.output.dtype.nbytes


def enabled(graph: Graph) -> bool | None:
    """``True``: every consumer of a large constant gets a prefetch; ``None``: those the intensity rule picks; ``False``: none."""
    pin = config.knob_raw("PREFETCH")
    if pin is not None and pin != "":
        return pin not in ("0", "off", "OFF", "false")
    if getattr(graph, "symbolic", None) is not None:
        return False
    # what a pass streams whole: constants a kernel reads from end to end (a gathered table, larger than any weight, is not)
    sizes = [_nbytes(graph.nodes[nid]) or 0 for nid, op in graph.constant_ops() if op.value is None]
    return None if sum(b for b in sizes if MIN_BYTES <= b <= MAX_BYTES) > LAST_LEVEL_CACHE_BYTES else False


def _builds_clean(op: HipOp, ctx: Context) -> bool:
    """The changed kernel builds without vector-register spills (one more wave per workgroup lowers the register
    budget of a lane).  Without a launcher library nothing can be compiled here and the answer is yes: the program's
    load step compiles the same source."""
    from deplodock_amd.backend.hip import hiprtc, launcher

    try:
        return hiprtc.spilled_vgprs(op.kernel_source, op.kernel_name, arch=ctx.arch) == 0
    except launcher.CompileError:
        raise
    except launcher.LauncherError:
        return True


def add_weight_prefetch(graph: Graph, ctx: Context | None = None) -> Graph:
    """Give every kernel whose successor streams a large constant the lanes that touch it first (in place)."""
    ctx = ctx or Context()
    mode = enabled(graph)
    if mode is False:
        return graph
    order = [nid for nid in graph.topological_order() if isinstance(graph.nodes[nid].op, HipOp)]
    for cur, nxt in zip(order, order[1:]):
        consumer: HipOp = graph.nodes[nxt].op
        weights = [(a, _nbytes(graph.nodes[a])) for a in consumer.arg_order if isinstance(graph.nodes[a].op, ConstantOp) and graph.nodes[a].op.value is None]
        weights = [(a, b) for a, b in weights if b is not None and MIN_BYTES <= b <= MAX_BYTES]
        if not weights:
            continue
        target, nbytes = max(weights, key=lambda w: w[1])
        if target in graph.nodes[cur].op.arg_order:
            continue  # the running kernel reads it itself
        if mode is None and not (consumer.algo_bytes and MIN_INTENSITY <= consumer.algo_flops / consumer.algo_bytes <= MAX_INTENSITY):
            continue
        slices = None
        ws = getattr(consumer, "weight_slices", None)
        if ws is not None and ws[0] == target and ws[1] % LINE == 0 and ws[1] * ws[2] == nbytes:
            slices = (ws[1] // LINE, ws[2])
        new = with_prefetch(graph.nodes[cur].op, target, nbytes, slices, ctx)
        if new is None or not _builds_clean(new, ctx):
            continue
        graph.nodes[cur].op = new
        if target not in graph.nodes[cur].inputs:
            graph.nodes[cur].inputs.append(target)
    return graph


__all__ = ["add_weight_prefetch", "with_prefetch", "enabled", "MIN_BYTES", "MAX_BYTES", "LAST_LEVEL_CACHE_BYTES"]
