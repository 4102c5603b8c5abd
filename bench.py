#!/usr/bin/env python3
"""Benchmark: decode tokens/s of a MiniCPM4-8B-shaped model with random weights on one MI355X.

python bench.py --gpus 1 --steps K --warmup W   prints ONE JSON line.  A step is one decode step
of the whole batch, the next token chosen by argmax included (default: batch 8 at context 4,096,
all 32 layers of the 8B shape).  The same line carries the prefill of 2,048 tokens, the decode
step's memory roofline against the published peak and against what a plain read kernel and a
large library product reach on this GPU, and decode at batch 1 and 64.  Before anything is timed,
one decode step from the captured graph is compared with the same step run eagerly.  Weights are
random (N(0, 0.02)), token ids uniform, the cache of the decode runs is filled with noise (what
filled it is not timed): nothing is downloaded.  The engine runs on one GPU only: for --gpus > 1
it says so and exits with 2.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}


def config_8b(layers=None):
    import torch
    g = torch.Generator().manual_seed(1234)
    fac = lambda: [float(x) for x in (1.0 + 3.0 * torch.rand(64, generator=g, dtype=torch.float64))]
    return {
        "architectures": ["MiniCPMForCausalLM"], "model_type": "minicpm",
        "num_hidden_layers": layers or 32, "hidden_size": 4096, "num_attention_heads": 32, "num_key_value_heads": 2,
        "head_dim": 128, "intermediate_size": 16384, "vocab_size": 73448, "rms_norm_eps": 1e-6, "rope_theta": 10000.0,
        "max_position_embeddings": 32768,
        "rope_scaling": {"rope_type": "longrope", "short_factor": fac(), "long_factor": fac(),
                         "original_max_position_embeddings": 32768},
        "scale_emb": 12, "dim_model_base": 256, "scale_depth": 1.4, "tie_word_embeddings": False,
        "hidden_act": "silu", "torch_dtype": "bfloat16",
    }


def config_small():
    """The MiniCPM4-0.5B shape (tied embeddings)."""
    import torch
    g = torch.Generator().manual_seed(4321)
    fac = lambda: [float(x) for x in (1.0 + 3.0 * torch.rand(32, generator=g, dtype=torch.float64))]
    return {
        "architectures": ["MiniCPMForCausalLM"], "model_type": "minicpm",
        "num_hidden_layers": 24, "hidden_size": 1024, "num_attention_heads": 16, "num_key_value_heads": 2,
        "head_dim": 64, "intermediate_size": 4096, "vocab_size": 73448, "rms_norm_eps": 1e-6, "rope_theta": 10000.0,
        "max_position_embeddings": 32768,
        "rope_scaling": {"rope_type": "longrope", "short_factor": fac(), "long_factor": fac(),
                         "original_max_position_embeddings": 32768},
        "scale_emb": 12, "dim_model_base": 256, "scale_depth": 1.4, "tie_word_embeddings": True,
        "hidden_act": "silu", "torch_dtype": "bfloat16",
    }


SPARSE_32K = {"kernel_size": 32, "kernel_stride": 16, "block_size": 64, "init_blocks": 1, "topk": 64,
              "window_size": 2048, "dense_len": 8192}


def weight_bytes_per_step(cfg, esize):
    """Bytes of weights a decode step reads once: every layer's matrices and norms, final norm, lm_head."""
    H, I, V, L = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size, cfg.num_hidden_layers
    qkv = (cfg.num_attention_heads + 2 * cfg.num_key_value_heads) * cfg.head_dim * H
    o = H * cfg.num_attention_heads * cfg.head_dim
    per_layer = (qkv + o + 3 * H * I) * esize + 2 * H * 4
    return L * per_layer + V * H * esize + H * 4


def kv_bytes_per_token(cfg, esize):
    return cfg.num_hidden_layers * 2 * cfg.num_key_value_heads * cfg.head_dim * esize


def prefill_flops(cfg, n):
    H, I, V, L = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size, cfg.num_hidden_layers
    nh, nkv, hd = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
    lin = L * ((nh + 2 * nkv) * hd * H + H * nh * hd + 3 * H * I)
    attn = L * nh * hd * 2 * (n * (n + 1) // 2) * 2          # q.k and p.v over the causal half
    return 2 * n * lin + attn + 2 * V * H


def batch_prefill_flops(cfg, lens):
    """Prompts of several lengths in one step: the products once a token, causal attention a prompt, one head row each."""
    H, I, V, L = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size, cfg.num_hidden_layers
    nh, nkv, hd = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
    lin = L * ((nh + 2 * nkv) * hd * H + H * nh * hd + 3 * H * I)
    attn = sum(L * nh * hd * 2 * (n * (n + 1) // 2) * 2 for n in lens)
    return 2 * sum(lens) * lin + attn + 2 * len(lens) * V * H


def sparse_keys_read(sc, context):
    """Keys a query at the end of `context` tokens attends to under InfLLM-v2: all of them up to dense_len, else
    the chosen blocks and the window."""
    if context <= sc["dense_len"]:
        return context
    return min(context, (sc["topk"] + sc["window_size"] // sc["block_size"]) * sc["block_size"])


def sparse_decode_bytes(cfg, sc, esize, batch, context):
    """What a decode step with block selection has to read: every weight once, and per sequence the attended
    keys and values and the compressed keys that the selection scores."""
    ck = cfg.num_hidden_layers * (context // sc["kernel_stride"]) * cfg.num_key_value_heads * cfg.head_dim * esize
    return weight_bytes_per_step(cfg, esize) + batch * (sparse_keys_read(sc, context) * kv_bytes_per_token(cfg, esize) + ck)


def sparse_prefill_flops(cfg, sc, n):
    """A prompt of n tokens with block selection: products, attention over the keys each query attends to (causal
    up to dense_len), the selection's scores over the compressed keys, one head row."""
    H, I, V, L = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size, cfg.num_hidden_layers
    nh, nkv, hd = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
    lin = L * ((nh + 2 * nkv) * hd * H + H * nh * hd + 3 * H * I)
    dense = min(n, sc["dense_len"])
    keys = dense * (dense + 1) // 2 + sum(sparse_keys_read(sc, p + 1) for p in range(dense, n))
    scores = sum(p // sc["kernel_stride"] for p in range(dense, n))
    return 2 * n * lin + L * nh * hd * 2 * 2 * keys + L * nh * hd * 2 * scores + 2 * V * H


def calibrate_read(dev):
    """GB/s of a kernel that only reads, over 4 GiB (far beyond the caches)."""
    import torch
    from cpmcu_amd import ops
    buf = torch.empty(1 << 30, dtype=torch.int32, device=dev).random_()
    out = torch.zeros(8192, dtype=torch.int32, device=dev)
    best = 0.0
    for _ in range(4):
        torch.cuda.synchronize()
        t = time.perf_counter()
        ops.read_bandwidth(buf, out)
        torch.cuda.synchronize()
        best = max(best, buf.numel() * 4 / (time.perf_counter() - t) / 1e9)
    return best


def timer_table(eng, run, title):
    """The timers by kernel class (average ms a call) for `run()` with the engine's timers switched on; steps
    then run eagerly, so the figures are of the kernels with their launches, not of the graph."""
    from cpmcu_amd.utils.perf import PerfTimers
    import torch
    before = eng.perf
    eng.perf = PerfTimers(enabled=True)
    try:
        run()
        torch.cuda.synchronize()
        rows = eng.perf.summary()
    finally:
        eng.perf = before
    print(f"[bench] timers, {title}:", file=sys.stderr)
    for label, kind, count, total, avg in sorted(rows, key=lambda r: -r[3]):
        print(f"[bench]   {label:<28}{count:>7} calls{total:>11.3f} ms{avg * 1e3:>10.1f} us each", file=sys.stderr)
    return {label: round(avg, 5) for label, kind, count, total, avg in rows}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=4096)
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the model's 32 (named in config)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--no-points", action="store_true", help="skip decode at batch 1 and 64")
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--hip-graph", type=int, default=1)
    ap.add_argument("--no-rehearse", action="store_true",
                    help="build the engine without its rehearsal passes (a profile then holds the benchmark's own "
                         "kernels only; the workspace grows during the warm-up steps instead)")
    ap.add_argument("--perf", action="store_true",
                    help="after the timed runs, a few eager steps with the engine's timers on: average ms by kernel "
                         "class (products / attention / selection / norms / head) on stderr and under 'timers'")
    ap.add_argument("--scenario", default="headline", choices=["headline", "small_batch64", "sparse32k"],
                    help="headline: the 8B shape at batch 8, context 4,096 (the default, the contract's line); "
                         "small_batch64: the 0.5B shape, 64 unequal prompts through the generation loop; sparse32k: "
                         "the 8B shape with InfLLM-v2 at 32k context")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported (no multi-GPU path exists)")
        sys.exit(2)

    import torch
    import cpmcu_amd
    from cpmcu_amd import Engine, EngineOptions, StepEntry
    from cpmcu_amd.config import MiniCPMConfig
    from cpmcu_amd.weights import random_tensors

    dev = "cuda:0"
    if args.scenario != "headline":
        other_scenarios(args, dev)
        return
    raw = config_8b(args.layers)
    cfg = MiniCPMConfig.from_dict(raw)
    esize = 2 if args.dtype == "bfloat16" else 4
    t0 = time.time()
    tensors = random_tensors(cfg, seed=0, device=dev)
    max_b = max(args.batch, 1 if args.no_points else 64)
    per_seq = -(-(args.context + args.steps + args.warmup + 64) // 64) * 64
    eng = Engine.from_tensors(cfg, tensors, EngineOptions(
        dtype=args.dtype, max_tokens=max(max_b * per_seq, args.prefill_tokens + 64), max_slots=max_b,
        max_step_tokens=max(args.prefill_tokens, 2048), device=dev, hip_graph=bool(args.hip_graph), rehearse=not args.no_rehearse))
    del tensors
    torch.cuda.synchronize()
    print(f"[bench] model ready in {time.time() - t0:.1f} s: {cfg.num_hidden_layers} layers, "
          f"{weight_bytes_per_step(cfg, esize) / 1e9:.2f} GB of weights a step", file=sys.stderr, flush=True)
    g = torch.Generator().manual_seed(7)
    rand_ids = lambda n: [int(t) for t in torch.randint(0, cfg.vocab_size, (n,), generator=g)]

    def fill_context(batch, context):
        """Slots that hold `context - 1` tokens of random keys and values: the state a decode step at that
        context length starts from (the timed steps do all of their own work; what filled the cache is not timed)."""
        slots = [eng.acquire() for _ in range(batch)]
        for s in slots:
            eng.cache.extend(s, context - 1)
        eng.cache.sync()
        for grp in eng.cache.groups:
            for st in grp.storage.values():
                for t in st.values():
                    t.normal_(0.0, 0.5)
        return slots

    from cpmcu_amd import ops
    next_tok = torch.zeros(64, dtype=torch.int32, device=dev)

    def decode_run(batch, context, steps, warmup):
        """Seconds for `steps` decode steps of `batch` sequences at `context`: each step runs the model on one
        token a sequence and chooses the next by argmax (on the device; the tokens fed are fixed beforehand so
        that every run does the same work)."""
        slots = fill_context(batch, context)
        toks = [rand_ids(batch) for _ in range(steps + warmup)]
        for i in range(warmup):
            ops.argmax(eng.step([StepEntry(s, [toks[i][j]], [0]) for j, s in enumerate(slots)]), next_tok[:batch])
        torch.cuda.synchronize()
        t = time.perf_counter()
        for i in range(warmup, warmup + steps):
            ops.argmax(eng.step([StepEntry(s, [toks[i][j]], [0]) for j, s in enumerate(slots)]), next_tok[:batch])
        torch.cuda.synchronize()
        dt = time.perf_counter() - t
        for s in slots:
            eng.release(s)
        return dt

    def graph_check(batch, context):
        """One decode step replayed from the captured graph against the same step run eagerly (the cache is
        wound back one token in between): finite and equal up to the order of float sums."""
        if not args.hip_graph:
            return None
        slots = fill_context(batch, context)
        ids = rand_ids(batch)
        entries = [StepEntry(s, [ids[j]], [0]) for j, s in enumerate(slots)]
        eng.options.hip_graph = False
        eager = eng.step(entries).clone()
        eng.options.hip_graph = True
        outs = []
        for _ in range(2):                   # the first captures, the second replays
            for s in slots:
                eng.cache.truncate(s, context - 1)
            outs.append(eng.step(entries).clone())
        for s in slots:
            eng.release(s)
        if not bool(torch.isfinite(eager).all()):
            raise SystemExit("bench.py: the decode step's logits are not finite")
        scale = float(eager.abs().max())
        err = max(float((o - eager).abs().max()) for o in outs)
        if err > 1e-3 * scale:
            raise SystemExit(f"bench.py: a decode step from the captured graph differs from the eager step by {err:.3g} "
                             f"(logits up to {scale:.3g})")
        return err / scale

    def calibrate():
        """What this GPU gives a kernel that only reads (GB/s) and the library's product of two large bf16
        matrices (FLOP/s): the ceilings that memory-bound and matrix-bound work can be held against besides
        the published peaks."""
        best = calibrate_read(dev)
        a = torch.randn(8192, 8192, device=dev, dtype=torch.bfloat16)
        b = torch.randn(8192, 8192, device=dev, dtype=torch.bfloat16)
        c = torch.empty_like(a)
        flops = 0.0
        for _ in range(4):
            torch.cuda.synchronize()
            t = time.perf_counter()
            for _ in range(4):
                torch.mm(a, b.t(), out=c)
            torch.cuda.synchronize()
            flops = max(flops, 4 * 2 * 8192 ** 3 / (time.perf_counter() - t))
        return best, flops

    def step_bytes(batch, context, steps):
        return weight_bytes_per_step(cfg, esize) + batch * (context + steps // 2) * kv_bytes_per_token(cfg, esize)

    read_gbs, mm_flops = calibrate()
    graph_err = graph_check(args.batch, args.context)
    dt = decode_run(args.batch, args.context, args.steps, args.warmup)
    ms_step = dt / args.steps * 1e3
    value = args.batch * args.steps / dt
    achieved = step_bytes(args.batch, args.context, args.steps) / (ms_step * 1e-3) / 1e9
    rec = {
        "metric": f"MiniCPM4-8B decode tok/s @ batch {args.batch}, context {args.context} "
                  f"({'bf16' if args.dtype == 'bfloat16' else 'fp32'}, random weights)",
        "value": round(value, 2), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic",
        "config": {"model": "MiniCPM4-8B shape, random weights N(0,0.02)", "layers": cfg.num_hidden_layers,
                   "layers_full_model": 32, "hidden": cfg.hidden_size, "heads": cfg.num_attention_heads,
                   "kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
                   "intermediate": cfg.intermediate_size, "vocab": cfg.vocab_size, "global_batch": args.batch,
                   "seq_len": args.context, "prefill_tokens": args.prefill_tokens, "parallelism": "1gpu",
                   "page_size": 64, "hip_graph": bool(args.hip_graph), "sampling": "argmax inside the timed step",
                   "cache_fill": "noise (not timed)"},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "read_kernel": round(read_gbs, 1),
                     "frac_of_read_kernel": round(achieved / read_gbs, 4)},
    }
    if graph_err is not None:
        rec["graph_check"] = {"max_rel_diff_to_eager": float(f"{graph_err:.3g}")}
    if not args.no_prefill:
        n = args.prefill_tokens
        times = []
        for it in range(3):
            s = eng.acquire()
            ids = rand_ids(n)
            torch.cuda.synchronize()
            t = time.perf_counter()
            eng.step([StepEntry(s, ids, [n - 1])])
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t)
            eng.release(s)
        pt = min(times[1:])
        peak = PEAK_FLOPS["bf16" if args.dtype == "bfloat16" else "fp32"]
        rec["prefill"] = {"value": round(n / pt, 1), "tokens": n, "ms": round(pt * 1e3, 3),
                          "frac": round(prefill_flops(cfg, n) / pt / peak, 4),
                          "library_product": round(mm_flops / 1e12, 1), "library_product_unit": "TFLOP/s",
                          "frac_of_library_product": round(prefill_flops(cfg, n) / pt / mm_flops, 4)}
    if not args.no_points:
        pts = {}
        for b in (1, 64):
            st = max(args.steps // 2, 8)
            d = decode_run(b, args.context, st, max(args.warmup // 2, 3))
            gbs = step_bytes(b, args.context, st) / (d / st) / 1e9
            pts[f"decode_b{b}"] = round(b * st / d, 2)
            pts[f"decode_b{b}_ms"] = round(d / st * 1e3, 4)
            pts[f"decode_b{b}_frac"] = round(gbs / HBM_PEAK_GBS, 4)
        rec["points"] = pts
    if args.perf:
        def few_steps():
            slots = fill_context(args.batch, args.context)
            for _ in range(4):
                eng.step([StepEntry(s, [1], [0]) for s in slots])
            for s in slots:
                eng.release(s)
            if not args.no_prefill:
                s = eng.acquire()
                eng.step([StepEntry(s, rand_ids(args.prefill_tokens), [args.prefill_tokens - 1])])
                eng.release(s)
        rec["timers"] = timer_table(eng, few_steps, f"batch {args.batch}, context {args.context}")
    print(json.dumps(rec), flush=True)


def other_scenarios(args, dev):
    """The two further workloads, each one JSON line of the same shape."""
    import torch
    from cpmcu_amd import Engine, EngineOptions, StepEntry
    from cpmcu_amd.config import MiniCPMConfig
    from cpmcu_amd.engine.generate import generate
    from cpmcu_amd.weights import random_tensors

    g = torch.Generator().manual_seed(11)
    if args.scenario == "small_batch64":
        cfg = MiniCPMConfig.from_dict(config_small())
        lens = [int(x) for x in torch.randint(128, 2049, (64,), generator=g)]
        new = 256
        eng = Engine.from_tensors(cfg, random_tensors(cfg, 0, device=dev), EngineOptions(
            dtype=args.dtype, max_tokens=sum(-(-(n + new) // 64) * 64 for n in lens), max_slots=64,
            max_step_tokens=8192, device=dev, hip_graph=bool(args.hip_graph), rehearse=not args.no_rehearse))
        prompts = [[int(t) for t in torch.randint(0, cfg.vocab_size, (n,), generator=g)] for n in lens]
        generate(eng, prompts[:4], 8)                                   # warm-up: kernels loaded, graphs of small batches
        outs = generate(eng, prompts, new)
        prefill_s = max(o.prefill_time for o in outs)
        decode_s = max(o.decode_time for o in outs)
        n_dec = sum(len(o.tokens) - 1 for o in outs)
        esize = 2 if args.dtype == "bfloat16" else 4
        ms_step = decode_s / (new - 1) * 1e3
        # a decode step reads every weight once and the live cache: all 64 sequences, half-way through their 256 tokens
        step_b = weight_bytes_per_step(cfg, esize) + sum(n + new // 2 for n in lens) * kv_bytes_per_token(cfg, esize)
        read_gbs = calibrate_read(dev)
        achieved = step_b / (ms_step * 1e-3) / 1e9
        peak = PEAK_FLOPS["bf16" if args.dtype == "bfloat16" else "fp32"]
        rec = {"metric": "MiniCPM4-0.5B shape, 64 unequal prompts (128..2048), 256 new tokens each: decode tok/s through "
                         "the generation loop", "value": round(n_dec / decode_s, 1), "unit": "tokens/s", "n_gpus": 1,
               "steps": new - 1, "warmup": 0, "ms_per_step": round(decode_s / (new - 1) * 1e3, 4),
               "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
               "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic",
               "config": {"model": "MiniCPM4-0.5B shape, random weights N(0,0.02)", "layers": 24, "hidden": 1024,
                          "heads": 16, "kv_heads": 2, "head_dim": 64, "intermediate": 4096, "vocab": 73448,
                          "global_batch": 64, "prompt_tokens": sum(lens), "new_tokens": new, "parallelism": "1gpu",
                          "hip_graph": bool(args.hip_graph)},
               "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                            "frac": round(achieved / HBM_PEAK_GBS, 4), "bytes_per_step": step_b,
                            "read_kernel": round(read_gbs, 1), "frac_of_read_kernel": round(achieved / read_gbs, 4)},
               "prefill": {"value": round(sum(lens) / prefill_s, 1), "tokens": sum(lens), "ms": round(prefill_s * 1e3, 2),
                           "frac": round(batch_prefill_flops(cfg, lens) / prefill_s / peak, 4)}}
        if args.perf:
            rec["timers"] = timer_table(eng, lambda: generate(eng, prompts[:64], 4), "64 unequal prompts, 4 tokens each")
        print(json.dumps(rec), flush=True)
        return
    raw = config_8b(args.layers)
    raw["sparse_config"] = dict(SPARSE_32K)
    cfg = MiniCPMConfig.from_dict(raw)
    n_prompt, new = 32000, 256
    esize = 2 if args.dtype == "bfloat16" else 4
    peak = PEAK_FLOPS["bf16" if args.dtype == "bfloat16" else "fp32"]
    read_gbs = calibrate_read(dev)
    eng = Engine.from_tensors(cfg, random_tensors(cfg, 0, device=dev), EngineOptions(
        dtype=args.dtype, max_tokens=4 * 32768, max_slots=4, max_step_tokens=2048, device=dev,
        hip_graph=bool(args.hip_graph), rehearse=not args.no_rehearse))
    rec = {"metric": "MiniCPM4-8B shape with InfLLM-v2 at 32k context: decode tok/s at batch 1 after a 32,000-token prefill",
           "unit": "tokens/s", "n_gpus": 1, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
           "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic",
           "config": {"model": "MiniCPM4-8B shape + sparse_config, random weights", "layers": cfg.num_hidden_layers,
                      "layers_full_model": 32, "kernel_size": 32, "kernel_stride": 16, "block_size": 64, "topk": 64,
                      "window_size": 2048, "dense_len": 8192, "prompt_tokens": n_prompt, "new_tokens": new,
                      "parallelism": "1gpu", "hip_graph": bool(args.hip_graph)}, "points": {}}
    # warm-up: one whole prompt and a few decode steps (kernel libraries loaded, the weights' decode layouts made,
    # scratch grown to this context's sizes; none of that belongs to a step)
    s = eng.acquire()
    warm = [int(t) for t in torch.randint(0, cfg.vocab_size, (n_prompt + 4,), generator=g)]
    for a in range(0, n_prompt, 2048):
        eng.step([StepEntry(s, warm[a:min(a + 2048, n_prompt)], [])])
    for i in range(4):
        eng.step([StepEntry(s, [warm[n_prompt + i]], [0])])
    eng.release(s)
    for batch in (1, 4):
        slots = [eng.acquire() for _ in range(batch)]
        ids = [[int(t) for t in torch.randint(0, cfg.vocab_size, (n_prompt + new,), generator=g)] for _ in slots]
        torch.cuda.synchronize()
        t = time.perf_counter()
        for sl, tok in zip(slots, ids):
            for a in range(0, n_prompt, 2048):
                eng.step([StepEntry(sl, tok[a:min(a + 2048, n_prompt)], [])])
        torch.cuda.synchronize()
        pre = time.perf_counter() - t
        for i in range(8):
            eng.step([StepEntry(sl, [tok[n_prompt + i]], [0]) for sl, tok in zip(slots, ids)])
        torch.cuda.synchronize()
        t = time.perf_counter()
        for i in range(8, new):
            eng.step([StepEntry(sl, [tok[n_prompt + i]], [0]) for sl, tok in zip(slots, ids)])
        torch.cuda.synchronize()
        dec = time.perf_counter() - t
        for sl in slots:
            eng.release(sl)
        ms_step = dec / (new - 8) * 1e3
        step_b = sparse_decode_bytes(cfg, SPARSE_32K, esize, batch, n_prompt + new // 2)
        achieved = step_b / (ms_step * 1e-3) / 1e9
        if batch == 1:
            rec.update({"value": round((new - 8) / dec, 2), "steps": new - 8, "warmup": 8,
                        "ms_per_step": round(ms_step, 4),
                        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                     "frac": round(achieved / HBM_PEAK_GBS, 4), "bytes_per_step": step_b,
                                     "read_kernel": round(read_gbs, 1),
                                     "frac_of_read_kernel": round(achieved / read_gbs, 4)},
                        "prefill": {"value": round(n_prompt / pre, 1), "tokens": n_prompt, "ms": round(pre * 1e3, 1),
                                    "frac": round(sparse_prefill_flops(cfg, SPARSE_32K, n_prompt) / (pre / batch) / peak, 4)}})
        rec["points"][f"decode_b{batch}"] = round(batch * (new - 8) / dec, 2)
        rec["points"][f"decode_b{batch}_ms"] = round(ms_step, 4)
        rec["points"][f"decode_b{batch}_frac"] = round(achieved / HBM_PEAK_GBS, 4)
    if args.perf:
        def few_steps():
            sl = eng.acquire()
            for a in range(0, n_prompt, 2048):
                eng.step([StepEntry(sl, warm[a:min(a + 2048, n_prompt)], [])])
            for i in range(4):
                eng.step([StepEntry(sl, [warm[n_prompt + i]], [0])])
            eng.release(sl)
        rec["timers"] = timer_table(eng, few_steps, "a 32,000-token prompt in chunks of 2,048 and 4 decode steps")
    print(json.dumps(rec), flush=True)


if __name__ == "__main__":
    main()
