"""Randomly drawn tiny configurations (head sizes 16..128 in steps of 16, 1..17 query heads a kv head, widths that
are multiples of 4 or 8 only, odd vocabularies, block-sparse attention with drawn sizes) against the plain
implementation: whole, the last 20 tokens one by one, and batches of unequal lengths (GPU).

Block-sparse configurations are compared in 32-bit only: with weights drawn at random the block scores lie
within a few parts in a thousand of each other, and which block wins then turns on bfloat16's rounding."""
import random

import pytest
import torch

import plain_minicpm as plain
import schedules
import tiny

pytestmark = pytest.mark.gpu


def draw(case):
    rng = random.Random(1000 + case)
    hd = rng.choice([16, 32, 48, 64, 80, 96, 112, 128])
    nkv = rng.choice([1, 1, 2, 3])
    group = rng.choice([1, 2, 3, 4, 5, 8, 16, 17])
    hidden = rng.choice([40, 56, 72, 96, 100, 104, 136, 200, 264])
    vocab = rng.choice([97, 300, 513, 1001])
    raw = dict(architectures=["MiniCPMForCausalLM"], model_type="minicpm", hidden_act="silu",
               num_hidden_layers=rng.choice([1, 2, 3]), hidden_size=hidden, num_attention_heads=nkv * group,
               num_key_value_heads=nkv, head_dim=hd, intermediate_size=rng.choice([48, 88, 100, 160, 264]),
               vocab_size=vocab, rms_norm_eps=rng.choice([1e-5, 1e-6, 3e-4]), rope_theta=rng.choice([10000.0, 50000.0]),
               max_position_embeddings=256, scale_emb=rng.choice([1, 4, 12]), dim_model_base=rng.choice([32, hidden]),
               scale_depth=rng.choice([1.0, 1.4]), tie_word_embeddings=rng.choice([True, False]))
    if case % 2:
        st = rng.choice([4, 8, 16])
        bs = rng.choice([b for b in (16, 32, 64) if b % st == 0])
        raw["sparse_config"] = {"kernel_size": st * rng.choice([1, 2]), "kernel_stride": st, "block_size": bs,
                                "init_blocks": rng.choice([0, 1]), "topk": rng.choice([1, 2, 3]),
                                "window_size": bs * rng.choice([1, 2]), "dense_len": rng.choice([0, 40, 70])}
    return raw


@pytest.mark.parametrize("case", range(12))
def test_a_drawn_configuration(tmp_path, case):
    from cpmcu_amd import Engine, EngineOptions
    raw = draw(case)
    d = tiny.write_model(raw, str(tmp_path / "m"), seed=case + 1, norm_std=0.1)
    cfg, w = tiny.read_model(d)
    lens = {"x": 150, "y": 37, "z": 70, "u": 25, "v": 90}
    reqs = {r: tiny.random_tokens(n, raw["vocab_size"], 5 + i) for i, (r, n) in enumerate(lens.items())}
    refs = {r: plain.forward(cfg, w, t).float() for r, t in reqs.items()}
    for dtype in ("float32",) if "sparse_config" in raw else ("float32", "bfloat16"):
        eng = Engine.from_dir(d, EngineOptions(dtype=dtype, max_tokens=768, max_slots=3))
        runs = {"whole": schedules.whole(eng, reqs), "tail-20": schedules.tail(eng, reqs, 20),
                "batches": schedules.batched(eng, reqs, {"x": 120, "y": 9, "z": 40, "u": 24, "v": 3},
                                             [("x", "y", "z"), ("v", "u")])}
        for what, got in runs.items():
            for r, ref in refs.items():
                err = (got[r] - ref).abs()
                tol = 2e-5 if dtype == "float32" else 0.02 * float(ref.abs().max())
                bad = (err.max(dim=1).values > tol).nonzero().flatten()
                assert bad.numel() == 0, (f"{raw}: {dtype} {what}: request {r}: first wrong position {int(bad[0])} of "
                                          f"{ref.shape[0]} (error {float(err[bad[0]].max()):.3g} > {tol:.3g})")
        eng.cache.check()
