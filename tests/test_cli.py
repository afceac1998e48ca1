"""Command-line front end: the ``--code`` grammar and the ``compile`` / ``run`` commands."""

import pytest
import torch

from deplodock_amd.cli import main
from deplodock_amd.commands.code import CodeError, parse_inline, slugify


def test_module_call_keeps_parameters_as_constants():
    p = parse_inline("nn.RMSNorm(64)(torch.randn(2, 4, 64))")
    assert isinstance(p.module, torch.nn.RMSNorm)
    assert [tuple(a.shape) for a in p.args] == [(2, 4, 64)]
    assert p.slug == "nn-rmsnorm-64"


def test_module_call_with_preamble_and_kwargs():
    p = parse_inline("m = nn.Softmax(dim=-1); x = torch.randn(3, 8); m(x)")
    assert isinstance(p.module, torch.nn.Softmax)
    assert tuple(p.args[0].shape) == (3, 8)


def test_expression_lifts_inline_and_named_tensors():
    p = parse_inline("w = torch.randn(8); torch.exp(torch.randn(4, 8)) * w + torch.ones(8)")
    assert set(p.input_names) == {"w", "x0", "x1"}
    want = torch.exp(p.args[p.input_names.index("x0")]) * p.args[p.input_names.index("w")] + 1.0
    got = p.module(*p.args)
    assert torch.allclose(got, want)


def test_single_inline_tensor_is_named_x():
    p = parse_inline("torch.softmax(torch.randn(4, 16), -1)")
    assert p.input_names == ("x",)


@pytest.mark.parametrize("bad", ["x = 1", "def f(:", "1 + 2"])
def test_rejects_unusable_code(bad):
    with pytest.raises(CodeError):
        parse_inline(bad)


def test_slugify():
    assert slugify("torch.nn.RMSNorm(2048)") == "torch-nn-rmsnorm-2048"
    assert slugify("***") == "code"


def test_compile_prints_one_kernel_per_launch(capsys):
    main(["compile", "-c", "nn.RMSNorm(2048)(torch.randn(1,32,2048))"])
    out = capsys.readouterr().out
    assert out.count('extern "C" __global__') == 1
    assert "k_rms_norm_reduce" in out and "REDUCE=b256" in out


def test_compile_torch_stage_and_output_file(tmp_path, capsys):
    dst = tmp_path / "g.txt"
    main(["compile", "--ir", "torch", "-o", str(dst), "-c", "torch.softmax(torch.randn(4,128), -1)"])
    assert capsys.readouterr().out == ""
    assert "SoftmaxOp" in dst.read_text()


def test_compile_knob_pin_reaches_the_schedule(capsys, monkeypatch):
    monkeypatch.delenv("EMMY_KNOBS", raising=False)
    main(["compile", "--knobs", "REDUCE=b64", "-c", "nn.RMSNorm(1024)(torch.randn(8,1024))"])
    monkeypatch.delenv("EMMY_KNOBS", raising=False)
    assert "REDUCE=b64" in capsys.readouterr().out


def test_compile_without_code_exits_2(capsys):
    with pytest.raises(SystemExit) as e:
        main(["compile"])
    assert e.value.code == 2


def test_run_ab_requires_bench():
    with pytest.raises(SystemExit) as e:
        main(["run", "--ab", "REDUCE=b64", "-c", "torch.softmax(torch.randn(4,128), -1)"])
    assert e.value.code == 2


def test_accuracy_verdict_flags_a_wrong_output():
    from deplodock_amd.commands.run import check_accuracy

    want = torch.randn(64, 64)
    ok, _ = check_accuracy(want.clone(), want)
    assert ok
    bad = want.clone()
    bad[3, 5] += 1e-2
    ok, line = check_accuracy(bad, want)
    assert not ok and "1 of 4096" in line
    ok, _ = check_accuracy(torch.full_like(want, float("nan")), want)
    assert not ok


@pytest.mark.gpu
def test_run_checks_against_eager_and_benches(capsys):
    main(["run", "--bench", "--iters", "10", "--warmup", "2", "--ab", "REDUCE=b128", "-c", "nn.RMSNorm(2048)(torch.randn(1,32,2048))"])
    out = capsys.readouterr().out
    assert out.startswith("PASS")
    assert "Eager PyTorch" in out and "emmy (hip)" in out and "emmy [REDUCE=b128]" in out
    assert "k_rms_norm_reduce" in out and "% hbm" in out


@pytest.mark.gpu
def test_run_multi_kernel_expression(capsys):
    main(["run", "-c", "x = torch.randn(64, 512); torch.softmax(x * 0.5, -1)"])
    assert capsys.readouterr().out.count("PASS") == 1


def test_microbench_kernels_compile_for_gfx950():
    from deplodock_amd.backend.hip import hiprtc
    from deplodock_amd.commands.microbench import _kernel_source

    for k, kind, mfma in ((0, "fma", True), (8, "exp", True), (4, "fma", False)):
        name = f"k_coissue_test_{k}_{kind}_{int(mfma)}"
        src = _kernel_source(name, k, kind, 256, mfma)
        assert src.count("__builtin_amdgcn_mfma_f32_32x32x16_bf16") == (2 if mfma else 0)
        assert hiprtc.compile_to_hsaco(src, name).stat().st_size > 0


def test_dynamic_flag_grammar():
    from deplodock_amd.commands.compile import parse_dynamic

    assert parse_dynamic(None) is None
    assert parse_dynamic(["seq_len@x:1", "b@x:0", "seq_len@cos:1"]) == {"x": {1: "seq_len", 0: "b"}, "cos": {1: "seq_len"}}
    with pytest.raises(SystemExit):
        parse_dynamic(["seq_len-x-1"])


@pytest.mark.gpu
def test_run_dynamic_axis_at_other_sizes(capsys):
    main(["run", "--dynamic", "rows@input:1", "--at", "rows=48", "--at", "rows=7", "-c", "nn.Softmax(-1)(torch.randn(2, 32, 512))"])
    out = capsys.readouterr().out
    assert out.count("PASS") == 3 and "at rows=48" in out and "at rows=7" in out


@pytest.mark.gpu
def test_tune_command_fills_a_database_run_then_uses(tmp_path, capsys):
    db = tmp_path / "tune.db"
    main(["tune", "--db", str(db), "--rounds", "4", "--iters", "3", "--warmup", "1", "-c", "nn.RMSNorm(1024)(torch.randn(512, 1024))"])
    out = capsys.readouterr().out
    assert "row_reduce/r512/c1024" in out and f"database: {db}" in out
    main(["run", "--tune-db", str(db), "-c", "nn.RMSNorm(1024)(torch.randn(512, 1024))"])
    assert capsys.readouterr().out.startswith("PASS")


def test_compile_a_built_in_architecture_whole_and_by_layer(capsys):
    """``compile <model> [--layer N] [--seq-len S]`` as the reference's command takes a model
    (emmy/commands/compile.py:66-97), from a built-in architecture with random weights: no download, no GPU."""
    main(["compile", "arch:qwen3-tiny", "--seq-len", "16"])
    out = capsys.readouterr().out
    assert out.count("k_index_rows") >= 1 and out.count("// ---- k_sdpa_reduce") == 2  # embedding gather, two layers
    main(["compile", "arch:qwen3-tiny", "--layer", "1", "--seq-len", "48", "--dtype", "fp32"])
    out = capsys.readouterr().out
    assert "k_index_rows" not in out and out.count("// ---- k_sdpa_reduce") == 1 and "mfma_f32_32x32x2f32" in out  # one layer; fp32 attention streams on fp32 atoms


def test_compile_a_local_model_directory(tmp_path, capsys):
    import transformers as tf

    tf.LlamaConfig(hidden_size=128, num_attention_heads=2, num_key_value_heads=1, intermediate_size=256, num_hidden_layers=1, vocab_size=301, pad_token_id=0, eos_token_id=1, bos_token_id=2).save_pretrained(tmp_path)
    main(["compile", str(tmp_path), "--seq-len", "8"])
    captured = capsys.readouterr()
    assert "random weights instead" in captured.err  # the directory holds a config and no weights
    assert "N=304" in captured.out  # the 301-word vocabulary is padded to whole runs of four columns


@pytest.mark.parametrize("argv, code", [(["compile", "Qwen/Qwen3-Embedding-0.6B"], 2), (["compile", "arch:nope"], 2), (["compile", "arch:qwen3-tiny", "--layer", "9"], 1), (["compile", "arch:qwen3-tiny", "-c", "torch.exp(torch.randn(4))"], 2)])
def test_model_inputs_that_are_refused(argv, code, capsys):
    with pytest.raises(SystemExit) as e:
        main(argv)
    assert e.value.code == code and "error:" in capsys.readouterr().err


@pytest.mark.gpu
def test_run_a_built_in_architecture(capsys):
    main(["run", "--bench", "--iters", "5", "--warmup", "1", "arch:qwen3-tiny", "--seq-len", "40"])
    out = capsys.readouterr().out
    assert out.startswith("PASS") and "mean |ours - fp32 eager|" in out and "emmy (hip)" in out
    main(["run", "arch:llama-tiny", "--dtype", "fp32", "--layer", "0", "--seq-len", "24"])
    assert capsys.readouterr().out.startswith("PASS")


def test_profile_child_command_drops_only_the_profiling_options():
    """``run --profile`` runs the same command line again under the profiler: the interpreter itself, the module, and
    every option except the ones that ask for the profile."""
    import sys

    from deplodock_amd.commands.run import _child_command

    argv = ["run", "--profile", "--pmc", "SQ_INSTS_VALU SQ_INSTS_MFMA", "--bench", "-c", "nn.Softmax(-1)(torch.randn(4, 64))", "--pmc=FETCH_SIZE", "--profile-dir", "out", "--knobs", "REDUCE=b64"]
    assert _child_command(argv) == [sys.executable, "-m", "deplodock_amd", "run", "--bench", "-c", "nn.Softmax(-1)(torch.randn(4, 64))", "--knobs", "REDUCE=b64"]


def test_profile_table_joins_the_trace_with_the_counter_passes(tmp_path):
    """Per emitted kernel: launches and average / minimum duration from the kernel trace, per-launch averages of every
    counter from the counter passes; the runtime's own kernels are left out."""
    from deplodock_amd.commands.run import profile_tables

    trace, pmc0, pmc1 = tmp_path / "trace" / "vm", tmp_path / "pmc0" / "vm", tmp_path / "pmc1" / "vm"
    for d in (trace, pmc0, pmc1):
        d.mkdir(parents=True)
    (trace / "1_kernel_trace.csv").write_text(
        '"Kind","Agent_Id","Queue_Id","Stream_Id","Thread_Id","Dispatch_Id","Kernel_Id","Kernel_Name","Correlation_Id","Start_Timestamp","End_Timestamp"\n'
        '"KERNEL_DISPATCH","Agent 1",1,1,1,1,1,"k_softmax_reduce_abc123",1,1000,3000\n'
        '"KERNEL_DISPATCH","Agent 1",1,1,1,2,1,"k_softmax_reduce_abc123",2,5000,9000\n'
        '"KERNEL_DISPATCH","Agent 1",1,1,1,3,2,"__amd_rocclr_copyBuffer",3,9000,9500\n'
    )
    head = '"Correlation_Id","Dispatch_Id","Agent_Id","Queue_Id","Process_Id","Thread_Id","Grid_Size","Kernel_Id","Kernel_Name","Workgroup_Size","LDS_Block_Size","Scratch_Size","VGPR_Count","Accum_VGPR_Count","SGPR_Count","Counter_Name","Counter_Value","Start_Timestamp","End_Timestamp"\n'
    (pmc0 / "2_counter_collection.csv").write_text(head + '1,1,"Agent 1",1,1,1,256,1,"k_softmax_reduce_abc123",256,0,0,32,0,16,"SQ_INSTS_VALU",100,0,0\n1,2,"Agent 1",1,1,1,256,1,"k_softmax_reduce_abc123",256,0,0,32,0,16,"SQ_INSTS_VALU",300,0,0\n')
    (pmc1 / "3_counter_collection.csv").write_text(head + '1,1,"Agent 1",1,1,1,256,1,"k_softmax_reduce_abc123",256,0,0,32,0,16,"FETCH_SIZE",64,0,0\n1,2,"Agent 1",1,1,1,256,2,"__amd_rocclr_copyBuffer",256,0,0,32,0,16,"FETCH_SIZE",999,0,0\n')
    header, rows = profile_tables(tmp_path / "trace", [tmp_path / "pmc0", tmp_path / "pmc1"])
    assert header == ["kernel", "launches", "avg us", "min us", "FETCH_SIZE", "SQ_INSTS_VALU"]
    assert rows == [["k_softmax_reduce_abc123", "2", "3.00", "2.00", "64", "200"]]
