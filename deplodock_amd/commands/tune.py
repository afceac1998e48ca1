"""``tune``: sweep knob pins for an inline expression on the GPU and store the winners.

The role of the reference's ``emmy tune`` (emmy/commands/tune.py): fill the
database the cold schedule pick consults.  The search here is the exhaustive
candidate sweep of :mod:`deplodock_amd.tune`.
"""

from __future__ import annotations

import sys
from pathlib import Path

from deplodock_amd.commands.compile import add_common_args, apply_common_args, trace_from_args
from deplodock_amd.commands.table import render_table


def register_tune_command(subparsers) -> None:
    p = subparsers.add_parser("tune", help="Sweep knob pins for an inline torch expression and store the best per kernel shape")
    add_common_args(p)
    p.add_argument("--db", default="auto", help="Tune database (SQLite) to update; 'auto' = the per-user default (EMMY_TUNE_DB overrides).")
    p.add_argument("--rounds", type=int, default=None, help="Stop after this many candidate rounds (default: the whole candidate list).")
    p.add_argument("--warmup", type=int, default=3)
    p.add_argument("--iters", type=int, default=10)
    p.add_argument("--min-gain", type=float, default=1.02, help="Store a pin only if it beats the heuristic pick by this factor (default 1.02).")
    p.set_defaults(func=handle_tune)


def handle_tune(args) -> None:
    import torch

    from deplodock_amd.backend.hip.backend import HipBackend
    from deplodock_amd.commands.run import _flatten_tensors, _to_device
    from deplodock_amd.tune import TuneDB, tune_graph

    apply_common_args(args)
    if not torch.cuda.is_available():
        print("error: no HIP device visible; tuning measures on the GPU", file=sys.stderr)
        sys.exit(1)
    device = torch.device("cuda:0")
    torch.cuda.set_device(0)
    graph, prog = trace_from_args(args)
    flat = _flatten_tensors(_to_device(prog.args, device)) + _flatten_tensors(_to_device(prog.kwargs, device))
    db = TuneDB(args.db if args.db == "auto" else Path(args.db))
    be = HipBackend(device_id=0)

    def progress(r, n, pins, verdict):
        if args.verbose:
            print(f"[{r + 1}/{n}] {' '.join(f'{k}={v}' for k, v in pins.items())}: {verdict}", file=sys.stderr)

    report = tune_graph(graph, be, db, input_data=dict(zip(graph.inputs, flat)), warmup=args.warmup, num_iters=args.iters, min_gain=args.min_gain, max_rounds=args.rounds, progress=progress)
    rows = [
        [r.kernel, r.key, f"{r.baseline_us:.2f}", f"{r.best_us:.2f}", f"{r.speedup:.2f}x", str(r.tried), " ".join(f"{k}={v}" for k, v in r.best_knobs.items()), "stored" if r.best_knobs != r.baseline_knobs and r.speedup >= args.min_gain else "kept heuristic"]
        for r in report
    ]  # fmt: skip
    for line in render_table(["Kernel", "Shape key", "heuristic us", "best us", "gain", "tried", "best knobs", "database"], rows, "llrrrrll"):
        print(line)
    print(f"\ndatabase: {db.path} ({len(db.rows())} entries)")
