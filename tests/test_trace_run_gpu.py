"""bin/trace_run as a user runs it: a subprocess fed steps on standard input (GPU)."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_minicpm as plain
import tiny

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_replay_of_an_unequal_batch(model_dirs, tmp_path, dtype):
    cfg, w = tiny.read_model(model_dirs["B"])
    reqs = {"p": tiny.random_tokens(100, 1000, 1), "q": tiny.random_tokens(75, 1000, 2), "r": tiny.random_tokens(20, 1000, 3)}
    prompt = {"p": 90, "q": 70, "r": 18}
    steps = [{"step": 0, "entries": [{"id": r, "tokens": reqs[r][:prompt[r]], "want": [0, prompt[r] - 1]} for r in reqs],
              "end": []}]
    fed = dict(prompt)
    n = 1
    while any(fed[r] < len(reqs[r]) for r in reqs):
        live = [r for r in reqs if fed[r] < len(reqs[r])]
        ends = [r for r in live if fed[r] + 1 == len(reqs[r])]
        steps.append({"step": n, "entries": [{"id": r, "tokens": [reqs[r][fed[r]]], "want": [0] if n % 2 else []}
                                             for r in live], "end": ends})
        for r in live:
            fed[r] += 1
        n += 1
    # a second wave that takes the freed slots and pages: 256 tokens hold p (2 pages), q (2) and nothing more
    steps.append({"step": n, "entries": [{"id": "again", "tokens": reqs["p"][:64], "want": [63]}], "end": ["again"]})
    out = tmp_path / "out"
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model_dirs["B"],
                           "--dtype", dtype, "--out", str(out), "--max-tokens", "320"],
                          input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert proc.stdout.split("\n")[:-1] == [f"done {s['step']}" for s in steps]
    ref = {r: plain.forward(cfg, w, t).float() for r, t in reqs.items()}
    tol = 2e-5 if dtype == "float32" else 0.02 * max(float(v.abs().max()) for v in ref.values())
    fed = dict(prompt)
    for s in steps[:-1]:
        rows = []
        for e in s["entries"]:
            base = 0 if s["step"] == 0 else fed[e["id"]]
            rows += [ref[e["id"]][base + wpos] for wpos in e["want"]]
        if s["step"] > 0:
            for e in s["entries"]:
                fed[e["id"]] += 1
        path = out / f"{s['step']}.f32"
        if not rows:
            assert not path.exists()
            continue
        got = torch.from_numpy(np.fromfile(path, dtype="<f4").reshape(len(rows), 1000))
        assert float((got - torch.stack(rows)).abs().max()) < tol, f"step {s['step']}"
    got = torch.from_numpy(np.fromfile(out / f"{n}.f32", dtype="<f4").reshape(1, 1000))
    assert float((got[0] - ref["p"][63]).abs().max()) < tol
