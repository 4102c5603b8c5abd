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
    assert "Decode Length" in p.stderr and "Prefill Speed" in p.stderr and "Prefilling [" in p.stderr
    assert "weights " in p.stderr and "workspace " in p.stderr and "cache " in p.stderr     # the memory figure
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


def write_tokenizer(model_dir, vocab_size):
    """A word-level tokenizer.json and a chat template, made with the `tokenizers` package: text in, text out."""
    from tokenizers import Tokenizer, models, pre_tokenizers
    words = ["<unk>", "<s>", "</s>", "user", "assistant", "hello", "world", "again"]
    vocab = {w: i for i, w in enumerate(words)}
    vocab.update({f"w{i}": i for i in range(len(words), vocab_size)})
    tok = Tokenizer(models.WordLevel(vocab, unk_token="<unk>"))
    tok.pre_tokenizer = pre_tokenizers.WhitespaceSplit()
    tok.save(os.path.join(model_dir, "tokenizer.json"))
    with open(os.path.join(model_dir, "tokenizer_config.json"), "w") as f:
        json.dump({"eos_token": {"content": "</s>"},
                   "chat_template": "{% for m in messages %}{{ m['role'] }} {{ m['content'] }} {% endfor %}"
                                    "{% if add_generation_prompt %}assistant{% endif %}"}, f)
    return {i: w for w, i in vocab.items()}


def test_cli_text_in_text_out_with_a_tokenizer_and_a_chat_template(tmp_path):
    """The text path (cpmcu/cli.py:47-79, cpmcu/llm.py:327-334): the prompt goes through the chat template and the
    tokenizer, the tokens come back as text, streamed piece by piece or whole; the cache is sized from
    --memory-limit (no --max-tokens), which is the command line's default."""
    raw = tiny.tiny_a()
    d = str(tmp_path / "model")
    os.makedirs(d)
    tiny.write_model(raw, d, seed=9, norm_std=0.1)
    cfg, w = tiny.read_model(d)
    word = write_tokenizer(d, raw["vocab_size"])
    text = lambda toks: " ".join(word[t] for t in toks)
    # chat template: "user hello world assistant" = ids 3 5 6 4
    want = plain.greedy(cfg, w, [3, 5, 6, 4], 6)
    p = run_cli("--model-path", d, "--dtype", "float32", "--prompt-text", "hello world", "--num-generate", "6",
                "--ignore-eos", "true", "--memory-limit", "0.05", "--plain-output", "true")
    assert p.returncode == 0, p.stderr[-1500:]
    assert p.stdout.strip() == text(want)                      # streamed pieces join to the whole text
    assert "Input prompt: 'user hello world assistant'" in p.stderr and "Input tokens: [4]" in p.stderr
    assert "Prefill done: 4/4 tokens" in p.stderr and "\r" not in p.stderr and "\033" not in p.stderr
    assert "Performance Summary:" in p.stderr and "  Decode Length: 5 tokens" in p.stderr
    assert "Maximum context length under current memory limit: 256 tokens" in p.stderr
    # without the template, from a file, not streamed; the tokenizer's eos joins the stop tokens
    pf = tmp_path / "prompt.txt"
    pf.write_text("hello again world\n")
    want = plain.greedy(cfg, w, [5, 7, 6], 8)
    stop = want[3]
    word_of_stop = word[stop]
    with open(os.path.join(d, "tokenizer_config.json"), "w") as f:
        json.dump({"eos_token": word_of_stop}, f)
    p = run_cli("--model-path", d, "--dtype", "float32", "--prompt-file", str(pf), "--use-chat-template", "false",
                "--num-generate", "8", "--use-stream", "false", "--max-tokens", "256")
    assert p.returncode == 0, p.stderr[-1500:]
    cut = want[:want.index(stop) + 1]
    assert p.stdout.strip() == f"[0] (stop) {text(cut)}"
    # a template is asked for and the tokenizer has none: the raw prompt is used, with a note
    p = run_cli("--model-path", d, "--dtype", "float32", "--prompt-text", "hello again world", "--num-generate", "2",
                "--ignore-eos", "true", "--max-tokens", "256")
    assert p.returncode == 0 and "Failed to apply chat template" in p.stderr
    assert p.stdout.strip() == text(want[:2])
