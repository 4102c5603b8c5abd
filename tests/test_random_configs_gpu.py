"""Randomly drawn tiny configurations (head sizes 16..128 in steps of 16, 1..17 query heads a kv head, widths that
are multiples of 4 or 8 only, odd vocabularies, block-sparse attention with drawn sizes) against the plain
implementation: whole, the last 20 tokens one by one, and batches of unequal lengths (GPU).

Block-sparse configurations are compared with the plain implementation in 32-bit only: with weights drawn at
random the block scores lie within a few parts in a thousand of each other, and which block wins then turns on
bfloat16's rounding.  Their bfloat16 engine is checked against the 32-bit engine's block lists instead: the
same lists wherever the 32-bit scores make the choice clear, and elsewhere a difference only among blocks whose
scores lie within a hundredth of the last one chosen."""
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


def record_selections(monkeypatch, eng, reqs, keep_inputs):
    """Run every request whole and note, for every call of the block selection (one a layer), the lists it
    made; with keep_inputs also the queries and the compressed keys it read, as plain tensors."""
    from cpmcu_amd import StepEntry, ops
    calls = []
    real = ops.sparse_select

    def noting(q, ckpool, nh, nkv, hd, scale, page_table, page_size, positions, tok_slot, ks, st, bs, init_blocks, topk,
               window_blocks, dense_len, max_pos, sel_blocks, sel_count, **kw):
        real(q, ckpool, nh, nkv, hd, scale, page_table, page_size, positions, tok_slot, ks, st, bs, init_blocks, topk,
             window_blocks, dense_len, max_pos, sel_blocks, sel_count, **kw)
        rec = {"blocks": sel_blocks.cpu().clone(), "count": sel_count.cpu().clone(), "pos": positions.cpu().tolist()}
        if keep_inputs:
            slot = int(tok_slot[0])
            n_ck = (max_pos + 1 - ks) // st + 1 if max_pos + 1 >= ks else 0
            rows = page_size // st
            table = page_table[slot].cpu().tolist()
            # a page of compressed keys lies [kv head][d / 8][row][d % 8]
            ck = [ckpool[table[(st * j) // page_size]].view(nkv, hd // 8, rows, 8)[:, :, ((st * j) % page_size) // st]
                  .reshape(nkv, hd) for j in range(n_ck)]
            rec["ck"] = torch.stack(ck).double().cpu() if ck else torch.zeros(0, nkv, hd, dtype=torch.float64)
            rec["q"] = q.view(q.shape[0], nh, hd).double().cpu()
        calls.append(rec)
    monkeypatch.setattr(ops, "sparse_select", noting)
    out = {}
    for r, toks in reqs.items():
        calls.clear()
        s = eng.acquire()
        eng.step([StepEntry(s, toks, [])])
        eng.release(s)
        out[r] = list(calls)
    monkeypatch.setattr(ops, "sparse_select", real)
    return out


@pytest.mark.parametrize("case", [c for c in range(12) if c % 2])
def test_bfloat16_block_lists_of_a_drawn_configuration(tmp_path, monkeypatch, case):
    from cpmcu_amd import Engine, EngineOptions
    raw = draw(case)
    sc = raw["sparse_config"]
    nkv = raw["num_key_value_heads"]
    d = tiny.write_model(raw, str(tmp_path / "m"), seed=case + 1, norm_std=0.1)
    reqs = {"x": tiny.random_tokens(250, raw["vocab_size"], 5), "y": tiny.random_tokens(131, raw["vocab_size"], 6)}
    lists = {}
    for dtype in ("float32", "bfloat16"):
        eng = Engine.from_dir(d, EngineOptions(dtype=dtype, max_tokens=768, max_slots=2))
        lists[dtype] = record_selections(monkeypatch, eng, reqs, keep_inputs=dtype == "float32")
    clear = unclear = differ = 0
    for r in reqs:
        assert len(lists["float32"][r]) == len(lists["bfloat16"][r]) == raw["num_hidden_layers"]
        for layer, (a, b) in enumerate(zip(lists["float32"][r], lists["bfloat16"][r])):
            assert torch.equal(a["count"], b["count"]), f"{raw}: request {r} layer {layer}: list lengths differ"
            for t, p in enumerate(a["pos"]):
                if int(a["count"][t, 0]) < 0:
                    continue                                  # dense
                pools = []
                want = plain.infllm_select(a["q"][t], a["ck"], p, sc, nkv, pools)
                for g in range(nkv):
                    c = int(a["count"][t, g])
                    la, lb = a["blocks"][t, g, :c].tolist(), b["blocks"][t, g, :c].tolist()
                    assert la == want[g], f"{raw}: float32 list differs from the plain selection at {r}/{layer}/{p}/{g}"
                    pool = pools[g]
                    k = min(sc["topk"], pool.numel())
                    ranked = torch.sort(pool, descending=True).values
                    # the choice is clear when the last block chosen beats the first one left out by a hundredth
                    edge = float(ranked[k - 1]) if k else 0.0
                    is_clear = k == pool.numel() or k == 0 or float(ranked[k]) < edge * 0.99
                    clear += is_clear
                    unclear += not is_clear
                    if la != lb:
                        differ += 1
                        assert not is_clear, (f"{raw}: bfloat16 chose {lb}, float32 {la} at request {r} layer {layer} "
                                              f"position {p} kv head {g}, although the scores are clear: {ranked[:k + 2]}")
                        for blk in set(la) ^ set(lb):         # only blocks about as good as the last one chosen swap
                            assert abs(float(pool[blk]) - edge) <= 0.02 * edge, (raw, r, layer, p, g, blk, la, lb)
    assert clear * 3 >= clear + unclear, f"only {clear} of {clear + unclear} choices are clear: little is compared"
