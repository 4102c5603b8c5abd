"""The command line on a tiny random-weights folder: the counterpart of the reference's only test, which
runs its command line and checks the exit code and that text came out (tests/test_model_generation.py:94-196)."""
import json
import os
import subprocess
import sys

import pytest

import plain_minicpm as plain
import tiny

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run_cli(*args):
    env = dict(os.environ, PYTHONPATH=ROOT)
    return subprocess.run([sys.executable, "-m", "cpmcu_amd.cli", *args], capture_output=True, text=True, timeout=600, env=env)


def test_cli_generates_from_token_ids(model_dirs, tmp_path):
    cfg, w = tiny.read_model(model_dirs["A"])
    prompts = [tiny.random_tokens(6, 512, 1), tiny.random_tokens(13, 512, 2)]
    ids = tmp_path / "ids.txt"
    ids.write_text("\n".join(" ".join(map(str, p)) for p in prompts) + "\n")
    p = run_cli("--model-path", model_dirs["A"], "--dtype", "float32", "--prompt-ids", str(ids), "--num-generate", "5",
                "--ignore-eos", "true", "--max-tokens", "512", "--use_stream", "false", "--perf")
    assert p.returncode == 0, p.stderr[-1500:]
    assert "prefill_attn" in p.stdout and "decode_ffn" in p.stdout and "GPU memory" in p.stdout      # the timer summary
    lines = [l for l in p.stdout.splitlines() if l.startswith("[")]
    want = [plain.greedy(cfg, w, pr, 5) for pr in prompts]
    assert [[int(t) for t in l.split(") ")[1].split()] for l in lines] == want
    assert "Decode length" in p.stderr and "Prefill length" in p.stderr
    # streaming a single prompt, sampling with a seed, twice the same
    outs = []
    for _ in range(2):
        p = run_cli("--model", model_dirs["A"], "--prompt-ids", str(ids), "--num_generate", "4", "--temperature", "0.9",
                    "--random-seed", "7", "--max-tokens", "512", "--batch", "1", "--use-stream", "false")
        assert p.returncode == 0, p.stderr[-1500:]
        outs.append(p.stdout)
    assert outs[0] == outs[1] and outs[0].strip()


def test_cli_random_weights_mode_and_errors(tmp_path):
    cfgp = tmp_path / "config.json"
    cfgp.write_text(json.dumps(tiny.tiny_b()))
    out = tmp_path / "model"
    p = run_cli("--random-weights", "--config", str(cfgp), "--seed", "3", "--model-path", str(out), "--prompt-lens", "70,5",
                "--num-generate", "3", "--max-tokens", "512")
    assert p.returncode == 0, p.stderr[-1500:]
    assert sorted(os.listdir(out)) == ["config.json", "model.safetensors"]
    assert len([l for l in p.stdout.splitlines() if l.startswith("[")]) == 2
    p = run_cli("--model-path", str(tmp_path / "nowhere"), "--prompt-lens", "3")
    assert p.returncode == 1 and "not found" in p.stderr
    p = run_cli("--model-path", str(out), "--prompt-text", "hello")
    assert p.returncode == 1 and "tokenizer" in p.stderr
