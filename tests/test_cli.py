"""The command line: random-weights mode on the CPU, generation on the GPU."""
import json
import os
import subprocess
import sys

import pytest

from conftest import TINY_B

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run_cli(*args, stdin=None):
    env = dict(os.environ, PYTHONPATH=ROOT)
    return subprocess.run([sys.executable, "-m", "vt_transformer_amd", *args], capture_output=True, text=True, env=env,
                          input=stdin, timeout=300)


def test_write_random_model(tmp_path):
    cfg = tmp_path / "c.json"
    cfg.write_text(json.dumps(TINY_B))
    out = tmp_path / "m"
    r = run_cli("--write-random-model", str(out), "--config", str(cfg), "--seed", "4")
    assert r.returncode == 0, r.stderr
    assert (out / "config.json").is_file() and (out / "model.safetensors").is_file()
    from vt_transformer_amd.weights import WeightStore
    assert len(WeightStore(str(out)).names()) == 3 + 12 * 3


def test_options_carry_the_reference_names():
    from vt_transformer_amd.__main__ import build_parser
    opts = {o for a in build_parser()._actions for o in a.option_strings}
    for name in ("--model-path", "--model", "--tokenizer-path", "--model-name", "--shell-mode",       # sglfront args
                 "--max-tokens", "--temperature", "--top-k", "--top-p", "--ignore-eos",               # SamplingParams
                 "--max-running-reqs", "--num-pages", "--max-seq-len", "--page-size", "--max-extend-tokens",
                 "--default-max-output"):                                                               # SchedulerConfig
        assert name in opts, name


@pytest.mark.gpu
def test_generate_and_shell(model_folders):
    import plain_model
    pc, pw = plain_model.read_folder(model_folders["B"])
    want = plain_model.greedy(pc, pw, [5, 6, 7], 4)
    r = run_cli("--model", model_folders["B"], "--dtype", "float32", "--prompt-ids", "5,6,7", "--max-tokens", "4",
                "--ignore-eos", "--max-seq-len", "64", "--max-running-reqs", "2")
    assert r.returncode == 0, r.stderr
    lines = r.stdout.strip().splitlines()
    assert lines[0] == ",".join(map(str, want))
    assert lines[-1].startswith("Generated 4 tokens, using ")
    # the shell: greedy when the temperature says so; /reset forgets the history
    r = run_cli("--model", model_folders["B"], "--dtype", "float32", "--shell-mode", "--temperature", "0", "--max-tokens", "4",
                "--ignore-eos", "--max-seq-len", "64", "--max-running-reqs", "2", stdin="5 6 7\n/reset\n5,6,7\n/exit\n")
    assert r.returncode == 0, r.stderr
    outs = [ln.replace("$ ", "") for ln in r.stdout.splitlines() if ln.replace("$ ", "")[:1].isdigit()]
    assert outs == [",".join(map(str, want))] * 2
    assert "Exiting shell..." in r.stdout


def test_dtype_names_of_the_reference_are_understood():
    """fp16, bf16 and fp32 as the reference's verify tool spells them
    (vt-transformer/models/qwen3-0.6b/tools/verify/reference.py:42-46), beside torch's names."""
    import torch
    from vt_transformer_amd.engine import parse_dtype
    assert parse_dtype("fp16") is parse_dtype("float16") is torch.float16
    assert parse_dtype("bf16") is parse_dtype("bfloat16") is torch.bfloat16
    assert parse_dtype("fp32") is parse_dtype("float32") is torch.float32
    with pytest.raises(ValueError, match="int8"):
        parse_dtype("int8")
    r = run_cli("--help")
    assert "fp16" in r.stdout and "float16" in r.stdout


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU: asked for more it says so in one line and exits with 2, before it touches a GPU."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    for extra_env, args in (({}, ["--gpus", "2"]), ({"WORLD_SIZE": "2"}, [])):
        env = dict(os.environ, **extra_env)
        p = subprocess.run([sys.executable, os.path.join(root, "bench.py"), *args], capture_output=True, text=True, env=env,
                           timeout=120)
        assert p.returncode == 2
        assert len(p.stdout.strip().splitlines()) == 1 and "one GPU" in p.stdout
