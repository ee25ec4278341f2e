"""The command line without a device: usage errors exit with 2, info and random-weights work."""
import json
import os
import subprocess
import sys

from helpers import ROOT, TINY

AXON = [sys.executable, os.path.join(ROOT, "bin", "axon")]


def run(*args):
    return subprocess.run(AXON + list(args), capture_output=True, text=True, timeout=120)


def test_usage_errors_exit_with_2(model_dirs):
    d = model_dirs("A")
    for args, fragment in [(["gen", d, "1 2", "--temp", "3000"], "--temp needs a number from 0 to 100"),
                           (["gen", d, "one two"], "token ids"),
                           (["gen", d, "1 2", "--top-p", "1.5"], "--top-p"),
                           (["gen", d, "1 2", "--repeat-penalty", "0"], "above 0"),
                           (["gen", d, "1 2", "-n", "1000"], "positions"),
                           (["gen", "/nonexistent/model", "1 2"], "config.json"),
                           (["frobnicate"], "invalid choice"),
                           (["logits", d], "required")]:
        r = run(*args)
        assert r.returncode == 2, (args, r.stderr)
        assert fragment in r.stderr and "try 'axon --help'" in r.stderr, (args, r.stderr)


def test_info_and_random_weights(tmp_path):
    cfg = tmp_path / "config.json"
    cfg.write_text(json.dumps(TINY["B"]["config"]))
    out = tmp_path / "model"
    r = run("random-weights", str(cfg), str(out), "--seed", "3", "--storage", "bfloat16")
    assert r.returncode == 0, r.stderr
    assert (out / "config.json").exists() and (out / "model.safetensors").exists()
    r = run("info", str(out))
    assert r.returncode == 0 and "Qwen2ForCausalLM" in r.stdout and "num_key_value_heads: 1" in r.stdout
    assert "cache group: 3 layers x 2 x 1 heads x 32" in r.stdout
    r = run("--help")
    assert r.returncode == 0 and "gen" in r.stdout and "logits" in r.stdout


def test_the_benchmark_refuses_more_than_one_gpu():
    """bench.py runs on one GPU: asked for more it says so in one line and exits with 2, before
    anything touches a device."""
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode == 2
    assert len(r.stdout.strip().splitlines()) == 1 and "one GPU" in r.stdout
