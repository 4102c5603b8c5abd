"""The engine against the plain implementation, in 32-bit and in bfloat16, under several ways of
cutting the same requests into steps (GPU)."""
import pytest
import torch

import plain_minicpm as plain
import schedules
import tiny

pytestmark = pytest.mark.gpu

# request lengths: prompt + teacher-forced continuation.  A has max_position 256, B 512 with
# dense_len 64, blocks of 16 and a window of 32, so that 90/200/300 cross into the pruned regime.
WORK = {
    "A": {"lens": {"a": 13, "b": 19, "c": 25, "d": 120, "e": 70}, "prompt": {"a": 5, "b": 11, "c": 17, "d": 90, "e": 33}},
    "B": {"lens": {"a": 106, "b": 216, "c": 40, "d": 300, "e": 65}, "prompt": {"a": 90, "b": 200, "c": 7, "d": 270, "e": 63}},
}
BATCHES = [("a", "b", "c"), ("d", "e"), ("c", "a"), ("e", "b", "d")]


def tolerance(dtype, ref):
    # float32: rounding of a few hundred float operations on logits of size ~1.
    # bfloat16: activations and weights carry 8 significant bits (2^-9 relative per rounding).
    return 2e-5 if dtype == "float32" else 0.01 * float(ref.abs().max())


@pytest.fixture(scope="module")
def references(model_dirs):
    refs = {}
    for name, d in model_dirs.items():
        cfg, w = tiny.read_model(d)
        reqs = {r: tiny.random_tokens(n, cfg["vocab_size"], 1000 + i) for i, (r, n) in enumerate(WORK[name]["lens"].items())}
        refs[name] = (cfg, w, reqs, {r: plain.forward(cfg, w, t).float() for r, t in reqs.items()})
    return refs


_engines = {}


def engine_for(model_dirs, name, dtype, **kw):
    from cpmcu_amd import Engine, EngineOptions
    key = (name, dtype, tuple(sorted(kw.items())))
    if key not in _engines:
        opts = dict(dtype=dtype, max_tokens=1024, max_slots=3)
        opts.update(kw)
        _engines[key] = Engine.from_dir(model_dirs[name], EngineOptions(**opts))
    return _engines[key]


def check(got, refs, dtype, what):
    for r, ref in refs.items():
        err = (got[r] - ref).abs()
        tol = tolerance(dtype, ref)
        bad = (err.max(dim=1).values > tol).nonzero().flatten()
        assert bad.numel() == 0, (f"{what}: request {r}: first wrong position {int(bad[0])} of {ref.shape[0]} "
                                  f"(error {float(err[bad[0]].max()):.3g} > {tol:.3g})")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_each_request_alone_and_whole(model_dirs, references, name, dtype):
    cfg, w, reqs, refs = references[name]
    eng = engine_for(model_dirs, name, dtype)
    check(schedules.whole(eng, reqs), refs, dtype, "whole")
    eng.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_last_32_tokens_one_by_one(model_dirs, references, name, dtype):
    cfg, w, reqs, refs = references[name]
    eng = engine_for(model_dirs, name, dtype)
    check(schedules.tail(eng, reqs, 32), refs, dtype, "tail-32")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_unequal_batches_one_after_another(model_dirs, references, name, dtype):
    cfg, w, reqs, refs = references[name]
    eng = engine_for(model_dirs, name, dtype)       # 3 slots: every batch takes slots that an earlier one gave back
    got = schedules.batched(eng, reqs, WORK[name]["prompt"], BATCHES[:2])
    check(got, refs, dtype, "batched")
    got = schedules.batched(eng, reqs, WORK[name]["prompt"], BATCHES[2:])
    check(got, refs, dtype, "batched, slots used again")
    eng.cache.check()
    assert not eng.cache.live


@pytest.mark.parametrize("page", [32, 128])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_other_page_sizes(model_dirs, references, name, dtype, page):
    """Pages of 32 and of 128 tokens (64 everywhere else): the same logits whole, token by token with graphs, and
    in batches whose slots are used again."""
    cfg, w, reqs, refs = references[name]
    eng = engine_for(model_dirs, name, dtype, page_size=page, hip_graph=True, max_tokens=1536)
    assert eng.cache.page_size == page
    check(schedules.whole(eng, reqs), refs, dtype, f"whole, pages of {page}")
    check(schedules.tail(eng, reqs, 32), refs, dtype, f"tail-32, pages of {page}")
    got = schedules.batched(eng, reqs, WORK[name]["prompt"], BATCHES[:2])
    check(got, refs, dtype, f"batched, pages of {page}")
    got = schedules.batched(eng, reqs, WORK[name]["prompt"], BATCHES[2:])
    check(got, refs, dtype, f"batched, slots used again, pages of {page}")
    eng.cache.check()
    assert not eng.cache.live


@pytest.mark.parametrize("name", ["A", "B"])
def test_engine_without_the_second_copy_of_the_weights(model_dirs, references, name):
    """tiled_weights=False: the bfloat16 engine keeps the checkpoint's layout only, so decode steps go through the
    split products and the norm kernels instead of the kernels that own strips of the re-laid weights."""
    cfg, w, reqs, refs = references[name]
    eng = engine_for(model_dirs, name, "bfloat16", tiled_weights=False)
    check(schedules.tail(eng, reqs, 32), refs, "bfloat16", "tail-32, checkpoint layout only")
    got = schedules.batched(eng, reqs, WORK[name]["prompt"], BATCHES[:2])
    check(got, refs, "bfloat16", "batched, checkpoint layout only")
    eng.cache.check()
    assert not eng.cache.live


@pytest.mark.parametrize("name", ["A", "B"])
def test_cutting_changes_nothing_beyond_rounding(model_dirs, references, name):
    """32-bit: whole, token by token and batched agree far below the tolerance against the plain implementation."""
    cfg, w, reqs, refs = references[name]
    eng = engine_for(model_dirs, name, "float32")
    a = schedules.whole(eng, reqs)
    b = schedules.tail(eng, reqs, 32)
    c = schedules.batched(eng, reqs, WORK[name]["prompt"], BATCHES[:2])
    for r in reqs:
        assert float((a[r] - b[r]).abs().max()) < 2e-6 and float((a[r] - c[r]).abs().max()) < 2e-6


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_small_forward_passes_equal_one_large(model_dirs, references, name, dtype):
    """A step cut into forward passes of 7 tokens (sequences split across passes) gives the same logits."""
    cfg, w, reqs, refs = references[name]
    eng = engine_for(model_dirs, name, dtype, max_step_tokens=7)
    check(schedules.whole(eng, reqs), refs, dtype, "chunks of 7")
    got = schedules.batched(eng, reqs, WORK[name]["prompt"], BATCHES[:2])
    check(got, refs, dtype, "batched in chunks of 7")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_long_decoding_and_first_tokens(model_dirs, references, name, dtype):
    cfg, w, _, _ = references[name]
    n = 250 if name == "A" else 330
    toks = tiny.random_tokens(n, cfg["vocab_size"], 77)
    ref = plain.forward(cfg, w, toks).float()
    eng = engine_for(model_dirs, name, dtype)
    got = schedules.tail(eng, {"x": toks}, n - 1)["x"]           # a one-token prompt, then everything one by one
    check({"x": got}, {"x": ref}, dtype, "long decoding")
    # the very first tokens of a sequence, each way
    for k in (1, 2, 3):
        s = eng.acquire()
        from cpmcu_amd import StepEntry
        lg = eng.step([StepEntry(s, toks[:k], list(range(k)))]).cpu()
        eng.release(s)
        check({"x": lg}, {"x": ref[:k]}, dtype, f"first {k} tokens")


@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_through_the_entry_point(model_dirs, references, name):
    from cpmcu_amd.llm import LLM
    cfg, w, reqs, _ = references[name]
    prompts = [reqs["a"][:9], reqs["b"][:70] if name == "B" else reqs["b"][:14], reqs["c"][:3]]
    want = [plain.greedy(cfg, w, p, 7) for p in prompts]
    llm = LLM(model_dirs[name], dtype="float32", max_tokens=1024, max_batch=2, apply_sparse=(name == "B"))
    llm.init_storage()
    llm.load_from_hf()
    tokens, decode_time, prefill_time = llm.generate(torch.tensor(prompts[0], dtype=torch.int32), generation_length=7)
    assert tokens == want[0] and decode_time > 0 and prefill_time > 0
    outs = llm.generate(prompts, generation_length=7)               # 3 requests, 2 slots: two batches
    assert [o.tokens for o in outs] == want
    # a stop token ends its sequence and is returned
    stop = want[1][2]
    outs = llm.generate(prompts, generation_length=7, terminators=[stop])
    for o, wnt in zip(outs, want):
        cut = wnt.index(stop) + 1 if stop in wnt else len(wnt)
        assert o.tokens == wnt[:cut] and o.finish_reason == ("stop" if stop in wnt else "length")
    # streaming yields the same tokens
    ev = list(llm.generate(prompts[2], generation_length=7, use_stream=True))
    assert [e["token"] for e in ev] == want[2] and ev[-1]["is_finished"]
    # bfloat16 through the same entry point: tokens are those of its own replayed logits
    llm16 = LLM(model_dirs[name], dtype="bfloat16", max_tokens=1024, apply_sparse=(name == "B"))
    llm16.init_storage()
    llm16.load_from_hf()
    toks16, _, _ = llm16.generate(prompts[0], generation_length=24)
    from cpmcu_amd import StepEntry
    seq = prompts[0] + toks16[:-1]
    s = llm16.engine.acquire()
    lg = llm16.engine.step([StepEntry(s, seq, list(range(len(prompts[0]) - 1, len(seq))))])
    llm16.engine.release(s)
    margin = lg.topk(2, dim=-1).values
    sure = (margin[:, 0] - margin[:, 1]) > 0.02
    assert int(sure.sum()) >= 6, f"only {int(sure.sum())} of {len(toks16)} choices are clear: too little is compared"
    assert [t for t, ok in zip(lg.argmax(-1).tolist(), sure.tolist()) if ok] == [t for t, ok in zip(toks16, sure.tolist()) if ok]


def test_steps_that_cannot_run_are_refused_and_change_nothing(model_dirs):
    from cpmcu_amd import StepEntry, StepError
    eng = engine_for(model_dirs, "A", "float32")
    s = eng.acquire()
    with pytest.raises(StepError, match="outside the vocabulary"):
        eng.step([StepEntry(s, [1, 512], [0])])
    with pytest.raises(StepError, match="at least one token"):
        eng.step([StepEntry(s, [], [])])
    with pytest.raises(StepError, match="wanted place"):
        eng.step([StepEntry(s, [1, 2], [2])])
    with pytest.raises(StepError, match="longest sequence"):
        eng.step([StepEntry(s, [1] * 257, [])])
    with pytest.raises(StepError, match="twice"):
        eng.step([StepEntry(s, [1], []), StepEntry(s, [2], [])])
    with pytest.raises(StepError, match="not held"):
        eng.step([StepEntry(2 if s != 2 else 1, [1], [])])
    with pytest.raises(StepError, match="at least one sequence"):
        eng.step([])
    assert eng.length(s) == 0
    assert eng.step([StepEntry(s, [1, 2, 3], [])]) is None and eng.length(s) == 3
    eng.release(s)
    eng.cache.check()
    with pytest.raises(ValueError, match="multiple of 32"):
        engine_for(model_dirs, "A", "float32", page_size=48)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_captured_decode_steps_equal_eager_ones(model_dirs, references, name, dtype):
    """Single-token steps replayed from a captured graph: every replay is checked, with eager work (prompts of
    other batches, larger batches that move scratch buffers) and synchronisations between the replays."""
    cfg, w, reqs, refs = references[name]
    eng = engine_for(model_dirs, name, dtype, hip_graph=True)
    for rnd_ in range(2):
        got = schedules.batched(eng, reqs, WORK[name]["prompt"], BATCHES[:2] if rnd_ == 0 else BATCHES[2:])
        check(got, refs, dtype, f"graph round {rnd_}")
        torch.cuda.synchronize()
    assert eng._graphs, "no decode step was captured"
    got = schedules.tail(eng, {"d": reqs["d"]}, 40)
    check(got, {"d": refs["d"]}, dtype, "graph tail")
    eng.cache.check()


@pytest.mark.parametrize("temperature", [0.0, 0.8])
def test_overlapped_generation_loop_equals_the_plain_loop(model_dirs, references, temperature):
    """The loop that keeps sampled tokens on the device and runs the host one step behind gives the same
    completions as the simple loop: stop tokens in the middle of a batch, unequal lengths, two batches."""
    from cpmcu_amd.engine import generate as gen
    from cpmcu_amd.sampling import Sampler
    cfg, w, reqs, _ = references["B"]
    eng = engine_for(model_dirs, "B", "float32", hip_graph=True)
    prompts = [reqs["a"][:20], reqs["b"][:75], reqs["c"][:3], reqs["d"][:40], reqs["e"][:9]]

    def run(fn, stop):
        results = [None] * len(prompts)
        for batch in ([0, 1, 2], [3, 4]):
            fn(eng, prompts, batch, 12, set(stop), Sampler(temperature, seed=5), results, None, None)
        eng.cache.check()
        assert not eng.cache.live
        return [(c.tokens, c.finish_reason) for c in results]

    free = run(gen._run_batch, [])
    assert run(gen._run_batch_overlapped, []) == free
    # stop on tokens that occur in the middle of some completions
    stops = [free[0][0][4], free[3][0][7]]
    plain_loop = run(gen._run_batch, stops)
    assert any(r == "stop" for _, r in plain_loop) and any(r == "length" for _, r in plain_loop)
    assert run(gen._run_batch_overlapped, stops) == plain_loop


ODD = {
    # head size 48 (no matrix-core attention kernel: the plain one runs), 5 query heads a kv head, sizes that are
    # multiples of 8 but of nothing more
    "hd48": dict(num_hidden_layers=2, hidden_size=200, num_attention_heads=10, num_key_value_heads=2, head_dim=48,
                 intermediate_size=344, vocab_size=777, rms_norm_eps=3e-6, rope_theta=7000.0, max_position_embeddings=192,
                 scale_emb=3, dim_model_base=100, scale_depth=2.0, tie_word_embeddings=False),
    # every query head its own kv head, head size 80, an intermediate size that is no multiple of 8 (the products
    # over it take the plain kernel), an odd vocabulary
    "mha80": dict(num_hidden_layers=1, hidden_size=72, num_attention_heads=6, num_key_value_heads=6, head_dim=80,
                  intermediate_size=100, vocab_size=1001, rms_norm_eps=1e-5, rope_theta=10000.0,
                  max_position_embeddings=192, scale_emb=1, dim_model_base=72, scale_depth=1.0, tie_word_embeddings=True),
    # a width that is a multiple of 4 only: the bfloat16 decode kernels that want 8 must step aside
    "w100": dict(num_hidden_layers=2, hidden_size=100, num_attention_heads=4, num_key_value_heads=2, head_dim=32,
                 intermediate_size=88, vocab_size=97, rms_norm_eps=1e-5, rope_theta=10000.0, max_position_embeddings=192,
                 scale_emb=4, dim_model_base=50, scale_depth=1.4, tie_word_embeddings=True),
    # block-sparse attention with 5 query heads on one kv head and blocks of 32
    "sparse5": dict(num_hidden_layers=2, hidden_size=160, num_attention_heads=5, num_key_value_heads=1, head_dim=32,
                    intermediate_size=208, vocab_size=300, rms_norm_eps=1e-6, rope_theta=20000.0,
                    max_position_embeddings=192, scale_emb=2, dim_model_base=80, scale_depth=1.0,
                    tie_word_embeddings=True,
                    sparse_config={"kernel_size": 16, "kernel_stride": 8, "block_size": 32, "init_blocks": 1, "topk": 2,
                                   "window_size": 32, "dense_len": 40}),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(ODD))
def test_sizes_that_are_no_power_of_two(tmp_path, name, dtype):
    """Whole, and the last 20 tokens one by one, against the plain implementation, at sizes the two tiny
    configurations do not have."""
    from cpmcu_amd import Engine, EngineOptions
    raw = dict(architectures=["MiniCPMForCausalLM"], model_type="minicpm", hidden_act="silu", **ODD[name])
    d = tiny.write_model(raw, str(tmp_path / name), seed=len(name), norm_std=0.1)
    cfg, w = tiny.read_model(d)
    reqs = {"x": tiny.random_tokens(150, raw["vocab_size"], 5), "y": tiny.random_tokens(37, raw["vocab_size"], 6)}
    refs = {r: plain.forward(cfg, w, t).float() for r, t in reqs.items()}
    eng = Engine.from_dir(d, EngineOptions(dtype=dtype, max_tokens=512, max_slots=2))
    check(schedules.whole(eng, reqs), refs, dtype, f"{name} whole")
    check(schedules.tail(eng, reqs, 20), refs, dtype, f"{name} tail-20")
    eng.cache.check()


def test_built_in_yarn_factors_through_the_entry_point(tmp_path):
    """``minicpm4_yarn`` (the reference's --minicpm4-yarn) installs its 64 factors for a head size of 128; with an
    engine that holds more than the original number of positions the long list and the cos/sin magnitude engage.
    The engine (both element types) against the plain implementation given the same factors."""
    from cpmcu_amd import StepEntry
    from cpmcu_amd.config.minicpm4_yarn import MINICPM4_YARN_FACTORS
    from cpmcu_amd.llm import LLM
    raw = tiny.tiny_a()
    raw.update(num_hidden_layers=1, hidden_size=256, num_attention_heads=2, num_key_value_heads=1, head_dim=128,
               intermediate_size=96, max_position_embeddings=512)
    raw["rope_scaling"] = {"rope_type": "longrope", "short_factor": [1.0] * 64, "long_factor": [1.0] * 64,
                           "original_max_position_embeddings": 64}
    d = str(tmp_path / "yarn")
    # (weights large enough for sharp attention: with scores near zero the rotation would hardly show)
    tiny.write_model(raw, d, seed=9, norm_std=0.1, std=0.1)
    cfg, w = tiny.read_model(d)
    toks = tiny.random_tokens(150, raw["vocab_size"], 4)
    want_cfg = dict(cfg)
    want_cfg["rope_scaling"] = dict(cfg["rope_scaling"], short_factor=list(MINICPM4_YARN_FACTORS),
                                    long_factor=list(MINICPM4_YARN_FACTORS))
    ref = plain.forward(want_cfg, w, toks).float()
    unchanged = plain.forward(cfg, w, toks).float()
    assert float((ref - unchanged).abs().max()) > 0.05 * float(ref.abs().max())       # the factors matter here
    for dtype in ("float32", "bfloat16"):
        llm = LLM(d, dtype=dtype, max_tokens=256, minicpm4_yarn=True)
        llm.init_storage()
        llm.load_from_hf()
        s = llm.engine.acquire()
        got = llm.engine.step([StepEntry(s, toks, list(range(len(toks))))]).cpu()
        llm.engine.release(s)
        check({"x": got}, {"x": ref}, dtype, f"yarn factors, {dtype}")
    with pytest.raises(ValueError, match="head_dim 128"):
        LLM(tiny.write_model(tiny.tiny_a(), str(tmp_path / "a"), seed=1), minicpm4_yarn=True)


def test_a_forward_pass_that_fails_is_rolled_out_of_the_cache(model_dirs, references):
    """A kernel that refuses in the middle of a step (forced here from the host) must not leave a sequence one
    pass ahead of its cache rows: lengths and pages are as before the failing pass, and the same tokens then
    give the right logits."""
    from cpmcu_amd import StepEntry
    cfg, w, reqs, refs = references["A"]
    eng = engine_for(model_dirs, "A", "float32", max_step_tokens=16)
    toks = reqs["d"]
    s, t = eng.acquire(), eng.acquire()
    eng.step([StepEntry(s, toks[:20], [])])
    free = [len(g.free_pages) for g in eng.cache.groups]
    real = eng.model.forward
    calls = {"n": 0}

    def failing(ctx):
        calls["n"] += 1
        if calls["n"] == 3:
            raise RuntimeError("kernel refused")
        return real(ctx)

    eng.model.forward = failing
    try:
        with pytest.raises(RuntimeError, match="kernel refused"):
            eng.step([StepEntry(s, toks[20:90], []), StepEntry(t, toks[:5], [])])       # 75 tokens: 5 passes of 16
    finally:
        eng.model.forward = real
    assert eng.length(s) == 20 + 32 and eng.length(t) == 0          # two passes completed, the third was rolled back
    eng.cache.check()
    # single-token steps: the failing step leaves no trace
    eng.model.forward = lambda ctx: (_ for _ in ()).throw(RuntimeError("kernel refused"))
    try:
        with pytest.raises(RuntimeError):
            eng.step([StepEntry(s, [toks[52]], [0])])
    finally:
        eng.model.forward = real
    assert eng.length(s) == 52
    got = eng.step([StepEntry(s, toks[52:], list(range(len(toks) - 52)))]).cpu()
    check({"d": got}, {"d": refs["d"][52:]}, "float32", "after a rolled-back pass")
    eng.release(s)
    eng.release(t)
    eng.cache.check()
    assert [len(g.free_pages) for g in eng.cache.groups] == [g.n_pages for g in eng.cache.groups] and free


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_a_step_that_mixes_running_sequences_with_a_fresh_prompt(model_dirs, references, name, dtype):
    """Two sequences that are under way bring one token each and a third brings its whole 40-token prompt, in one
    step: the packed batch then holds rows of both kinds, and every row must come out as if it ran alone."""
    from cpmcu_amd import StepEntry
    cfg, w, reqs, refs = references[name]
    eng = engine_for(model_dirs, name, dtype)
    # (request, tokens it already holds) of the two running sequences, and the request whose prompt is fresh;
    # B: one runs beyond dense_len with pruned blocks, the other crosses dense_len in these very steps
    (r1, n1), (r2, n2), r3 = ((("d", 100), ("c", 20), "e") if name == "A" else (("d", 280), ("e", 62), "b"))
    t1, t2, t3 = reqs[r1], reqs[r2], reqs[r3]
    s1, s2, s3 = eng.acquire(), eng.acquire(), eng.acquire()
    eng.step([StepEntry(s1, t1[:n1], []), StepEntry(s2, t2[:n2], [])])
    # the fresh prompt stands between the two single tokens; then two mixed steps more, the prompt's sequence now
    # continuing with several tokens while the others bring one
    lg = eng.step([StepEntry(s1, [t1[n1]], [0]), StepEntry(s3, t3[:40], list(range(40))), StepEntry(s2, [t2[n2]], [0])]).cpu()
    got = {r1: [lg[:1]], r3: [lg[1:41]], r2: [lg[41:]]}
    lg = eng.step([StepEntry(s3, t3[40:43], [0, 1, 2]), StepEntry(s2, [t2[n2 + 1]], [0]), StepEntry(s1, [t1[n1 + 1]], [0])]).cpu()
    got[r3].append(lg[:3]); got[r2].append(lg[3:4]); got[r1].append(lg[4:5])
    lg = eng.step([StepEntry(s1, [t1[n1 + 2]], [0]), StepEntry(s2, [t2[n2 + 2]], []), StepEntry(s3, [t3[43]], [0])]).cpu()
    got[r1].append(lg[:1]); got[r3].append(lg[1:2])
    check({r: torch.cat(v) for r, v in got.items()},
          {r1: refs[r1][n1:n1 + 3], r2: refs[r2][n2:n2 + 2], r3: refs[r3][:44]}, dtype, "mixed step")
    for s in (s1, s2, s3):
        eng.release(s)
    eng.cache.check()
