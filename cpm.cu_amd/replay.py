"""Trace replay: feed given token ids through a model step by step and write logits.

It samples nothing and has no forward pass, cache or loader of its own: it
builds the engine that generation uses and calls its step function.  The
reference has no such program (its only driver is the command line,
cpmcu/cli.py:304-326).

Input (standard input), one JSON object a line:
    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}
For a step in which something is wanted, OUT/<step>.f32 receives the logits at
the wanted places, in the order of the entries and of ``want``, as little-endian
float32 [wanted, vocab].  After every step a line ``done <step>`` is printed.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
from typing import Dict

import numpy as np


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16",
                    help="bfloat16: the kernels and precisions that serving uses; float32: everything in true 32-bit")
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens that live requests hold at any time (each rounded up to 64); sizes the cache")
    ap.add_argument("--max-step-tokens", type=int, default=2048, help="tokens one forward pass carries")
    ap.add_argument("--device", default="cuda:0")
    args = ap.parse_args(argv)

    import torch  # noqa: F401  (after argument parsing, so that --help is quick)
    from . import Engine, EngineOptions, StepEntry

    os.makedirs(args.out, exist_ok=True)
    print(f"[trace_run] loading {args.model} ({args.dtype})", file=sys.stderr, flush=True)
    engine = Engine.from_dir(args.model, EngineOptions(dtype=args.dtype, max_tokens=max(args.max_tokens, 64),
                                                       max_step_tokens=args.max_step_tokens, device=args.device))
    slots: Dict[str, int] = {}
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        step = rec["step"]
        entries = []
        for e in rec.get("entries", []):
            rid = str(e["id"])
            if rid not in slots:
                slots[rid] = engine.acquire()
            entries.append(StepEntry(slots[rid], e["tokens"], e.get("want", [])))
        if entries:
            logits = engine.step(entries)
            if logits is not None:
                arr = logits.cpu().numpy().astype("<f4", copy=False)
                tmp = os.path.join(args.out, f".{step}.f32.tmp")
                arr.tofile(tmp)
                os.replace(tmp, os.path.join(args.out, f"{step}.f32"))
        for rid in rec.get("end", []):
            rid = str(rid)
            if rid in slots:
                engine.release(slots.pop(rid))
        print(f"done {step}", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
