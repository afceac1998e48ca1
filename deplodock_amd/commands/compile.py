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
    parser.add_argument("input", nargs="?", help="A model: a local directory with a transformers config.json (and weights, else random ones), or 'arch:<name>' for a built-in "
                        "architecture with random weights (arch:qwen3-0.6b, arch:qwen3-tiny, arch:llama-tiny).  Hub model IDs need a download and are refused.  Mutually exclusive with --code.")  # fmt: skip
    parser.add_argument("--layer", type=int, default=None, help="Decoder layer index of the model input (hidden states + rotary tables in); omit for the whole model (token ids in, logits out).")
    parser.add_argument("--seq-len", type=int, default=32, help="Tokens of the example input for a model (default 32).")
    parser.add_argument("--dtype", choices=["bf16", "fp16", "fp32"], default="bf16", help="Parameter / activation type for a model input (default bf16).")
    parser.add_argument("--random-weights", action="store_true", help="Initialise the model from its config instead of loading weights from the directory.")
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

    if args.input and args.code:
        print("error: a model input and --code are mutually exclusive", file=sys.stderr)
        sys.exit(2)
    if args.input:
        return _trace_model(args)
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


ARCHITECTURES = {
    # name -> (transformers config class, its arguments): built from the config alone, random weights
    "qwen3-0.6b": ("Qwen3Config", dict(hidden_size=1024, num_attention_heads=16, num_key_value_heads=8, head_dim=128, intermediate_size=3072, num_hidden_layers=28, vocab_size=151669, rms_norm_eps=1e-6, rope_theta=1e6, max_position_embeddings=32768)),
    "qwen3-tiny": ("Qwen3Config", dict(hidden_size=256, num_attention_heads=4, num_key_value_heads=2, head_dim=64, intermediate_size=512, num_hidden_layers=2, vocab_size=1000)),
    "llama-tiny": ("LlamaConfig", dict(hidden_size=256, num_attention_heads=4, num_key_value_heads=2, intermediate_size=512, num_hidden_layers=2, vocab_size=1000)),
}  # fmt: skip


def _trace_model(args):
    """``(graph, program)`` for a model input, the way the reference's ``compile <model> [--layer N] [--seq-len S]`` traces
    one (emmy/commands/trace.py:61-106): the whole causal LM on token ids, or one decoder layer on hidden states and
    its rotary tables.  The model comes from a local directory or a built-in architecture; nothing is downloaded."""
    import torch
    from torch import nn

    from deplodock_amd.commands.code import InlineProgram, slugify
    from deplodock_amd.trace.torch import trace_module

    try:
        import transformers as tf
    except ImportError:
        print("error: a model input needs the transformers package", file=sys.stderr)
        sys.exit(1)
    dtype = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}[args.dtype]
    torch.manual_seed(args.seed)
    spec = args.input
    if spec.startswith("arch:"):
        name = spec[5:]
        if name not in ARCHITECTURES:
            print(f"error: unknown architecture {name!r}; known: {', '.join(sorted(ARCHITECTURES))}", file=sys.stderr)
            sys.exit(2)
        cfg_cls, kw = ARCHITECTURES[name]
        cfg = getattr(tf, cfg_cls)(pad_token_id=0, eos_token_id=1, bos_token_id=2, **kw)
        model = tf.AutoModelForCausalLM.from_config(cfg)
    elif Path(spec).is_dir():
        if spec.endswith(".json") or not (Path(spec) / "config.json").exists():
            print(f"error: {spec} holds no config.json", file=sys.stderr)
            sys.exit(2)
        cfg = tf.AutoConfig.from_pretrained(spec, local_files_only=True)
        model = None
        if not args.random_weights:
            try:
                # safetensors only: a pickled checkpoint would execute code from the file on load
                model = tf.AutoModelForCausalLM.from_pretrained(spec, local_files_only=True, torch_dtype=dtype, use_safetensors=True, trust_remote_code=False)
            except (OSError, ValueError) as exc:
                print(f"note: no weights loaded from {spec} ({str(exc).splitlines()[0][:120]}); random weights instead", file=sys.stderr)
        if model is None:
            model = tf.AutoModelForCausalLM.from_config(cfg)
    else:
        print(f"error: {spec!r} is neither a local model directory nor 'arch:<name>'; hub model IDs need a download, which this environment does not do "
              "(IR files go to `run --ir`)", file=sys.stderr)  # fmt: skip
        sys.exit(2)
    model.config._attn_implementation = "sdpa"
    model = model.to(dtype).eval()
    seq = int(args.seq_len)
    if args.layer is None:

        class Logits(nn.Module):
            def __init__(self, m):
                super().__init__()
                self.m = m

            def forward(self, input_ids):
                return self.m(input_ids=input_ids).logits

        module, inputs, kwargs = Logits(model).eval(), (torch.randint(0, int(model.config.vocab_size), (1, seq)),), {}
        slug = f"{slugify(spec)}-full-s{seq}"
    else:
        layers = model.model.layers
        if not 0 <= args.layer < len(layers):
            print(f"error: layer {args.layer} not found (the model has {len(layers)})", file=sys.stderr)
            sys.exit(1)

        class Layer(nn.Module):
            def __init__(self, layer):
                super().__init__()
                self.l = layer

            def forward(self, x, cos, sin):
                out = self.l(x, position_embeddings=(cos, sin), attention_mask=None)
                return out[0] if isinstance(out, tuple) else out

        x = torch.randn(1, seq, int(model.config.hidden_size))
        cos, sin = model.model.rotary_emb(x.to(dtype), torch.arange(seq)[None])
        module, inputs, kwargs = Layer(layers[args.layer]).eval(), (x.to(dtype), cos.to(dtype), sin.to(dtype)), {}
        slug = f"{slugify(spec)}-layer{args.layer}-s{seq}"
    graph = trace_module(module, inputs, dynamic_shapes=parse_dynamic(args.dynamic))
    return graph, InlineProgram(module=module, args=inputs, kwargs=kwargs, slug=slug)


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
