"""CLI entry point: ``python -m deplodock_amd <command>`` (emmy/emmy.py:25-56)."""

from __future__ import annotations

import argparse


def build_parser() -> argparse.ArgumentParser:
    from deplodock_amd.commands.compile import register_compile_command
    from deplodock_amd.commands.microbench import register_microbench_command
    from deplodock_amd.commands.run import register_run_command
    from deplodock_amd.commands.tune import register_tune_command

    parser = argparse.ArgumentParser(prog="deplodock_amd", description="MI355X kernel backend: compile / run inline torch expressions")
    sub = parser.add_subparsers(dest="command", required=True)
    register_compile_command(sub)
    register_run_command(sub)
    register_tune_command(sub)
    register_microbench_command(sub)
    return parser


def main(argv: list[str] | None = None) -> None:
    args = build_parser().parse_args(argv)
    args.func(args)


if __name__ == "__main__":
    main()
