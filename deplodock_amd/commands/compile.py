"""``compile``: trace an inline expression and print the emitted HIP kernels.

Needs no GPU (hipRTC is not even invoked): the output is the source the
backend would compile, one block per launch in program order, as the
reference's ``emmy compile --code`` prints its CUDA
(emmy/commands/compile.py:286-394).  ``--hsaco`` additionally compiles every
kernel for gfx950 and reports code-object sizes.
"""

from __future__ import annotations

import os
import sys
from pathlib import Path

from deplodock_amd import config


def add_common_args(parser) -> None:
    parser.add_argument("input", nargs="?", help="Unsupported here (model IDs and IR files): use --code.")
    parser.add_argument("--code", "-c", help="Inline Python whose last statement is the expression to compile, e.g. 'torch.nn.RMSNorm(2048)(torch.randn(1,32,2048))'.")
    parser.add_argument("--dump-dir", default=None, help="Directory for the graph after each pass and the final kernel sources.")
    parser.add_argument("--knobs", default=None, help="Pin scheduling knobs for this invocation, 'K1=V1,K2=V2' (the EMMY_KNOBS grammar), e.g. 'TILE=a:mfma_32x32x16_bf16/w2x2/f2x3/k4'.")
    parser.add_argument("--hiprtc-flags", default=None, help="Extra hipRTC options (space separated); same as EMMY_HIPRTC_FLAGS.")
    parser.add_argument("--seed", type=int, default=0, help="torch RNG seed applied before the expression is evaluated (default 0).")
    parser.add_argument(
        "--dynamic",
        action="append",
        default=None,
        metavar="NAME@INPUT:AXIS",
        help="Let axis AXIS of forward argument INPUT vary at run time under the name NAME (repeatable), e.g. 'seq_len@x:1'. "
        "Kernels stay specialised per size: another size re-traces and re-lowers on first use.",
    )
    parser.add_argument("--tune-db", default=None, help="Consult this tune database (path, or 'auto' for the per-user default) for knob pins the environment does not set.")
    parser.add_argument("-v", "--verbose", action="count", default=0)


def apply_common_args(args) -> None:
    if args.knobs is not None:
        os.environ[config.KNOBS] = args.knobs
    if args.hiprtc_flags is not None:
        os.environ[config.HIPRTC_FLAGS] = args.hiprtc_flags


def trace_from_args(args):
    """``(graph, program)`` for the parsed arguments, or exit with the reference's codes."""
    from deplodock_amd.commands.code import CodeError, parse_inline
    from deplodock_amd.trace.torch import trace_module

    if args.input and not args.code:
        print("error: model IDs and IR files are not handled by this backend; pass the module with --code", file=sys.stderr)
        sys.exit(2)
    if not args.code:
        print("error: --code is required", file=sys.stderr)
        sys.exit(2)
    import torch

    torch.manual_seed(args.seed)
    try:
        prog = parse_inline(args.code)
    except CodeError as e:
        print(f"error: {e}", file=sys.stderr)
        sys.exit(2)
    return trace_module(prog.module, prog.args, kwargs=prog.kwargs or None, dynamic_shapes=parse_dynamic(args.dynamic)), prog


def parse_dynamic(specs: list[str] | None) -> dict | None:
    """``NAME@INPUT:AXIS`` strings → ``{INPUT: {AXIS: NAME}}``."""
    if not specs:
        return None
    out: dict[str, dict[int, str]] = {}
    for spec in specs:
        try:
            name, rest = spec.split("@", 1)
            arg, axis = rest.rsplit(":", 1)
            out.setdefault(arg, {})[int(axis)] = name
        except ValueError:
            print(f"error: --dynamic expects NAME@INPUT:AXIS, got {spec!r}", file=sys.stderr)
            sys.exit(2)
    return out


def register_compile_command(subparsers) -> None:
    p = subparsers.add_parser("compile", help="Lower an inline torch expression to gfx950 HIP kernels and print them")
    add_common_args(p)
    p.add_argument("--output", "-o", help="Write the kernel sources here instead of stdout")
    p.add_argument("--ir", choices=["torch", "hip"], default="hip", help="Stage to print: the traced graph or the emitted kernels (default).")
    p.add_argument("--json", default=None, metavar="PATH", help="Also write the selected stage as a JSON graph (a reproducer `run --ir PATH` replays on random data).")
    p.add_argument("--hsaco", action="store_true", help="Also compile each kernel with hipRTC for gfx950 and report code-object sizes.")
    p.set_defaults(func=handle_compile)


def handle_compile(args) -> None:
    from deplodock_amd.backend.hip.backend import HipBackend
    from deplodock_amd.ir.hip import HipOp
    from deplodock_amd.pipeline import format_kernels

    apply_common_args(args)
    graph, _prog = trace_from_args(args)
    staged = graph
    if args.ir == "torch":
        text = graph.pretty_print() + "\n"
    else:
        compiled = HipBackend(dump=Path(args.dump_dir) if args.dump_dir else None, tune_db=getattr(args, "tune_db", None)).compile(graph)
        text = format_kernels(compiled)
        staged = compiled
        if args.hsaco:
            from deplodock_amd.backend.hip import hiprtc

            seen = set()
            for nid in compiled.topological_order():
                op = compiled.nodes[nid].op
                if isinstance(op, HipOp) and op.kernel_name not in seen:
                    seen.add(op.kernel_name)
                    path = hiprtc.compile_to_hsaco(op.kernel_source, op.kernel_name)
                    print(f"// {op.kernel_name}: {path.stat().st_size} bytes of gfx950 code object ({path.name})", file=sys.stderr)
    if args.json:
        from deplodock_amd import serialize

        serialize.save(staged, args.json)
    if args.output:
        Path(args.output).write_text(text)
    else:
        sys.stdout.write(text)
