"""The engine's memory figure (GPU): weights, workspace and cache are known when the engine is built, a limit
that they exceed is refused there with the three numbers, the cache is sized from what the limit leaves, and
no later step makes the workspace grow."""
import pytest
import torch

import plain_minicpm as plain
import tiny

pytestmark = pytest.mark.gpu


def total_memory():
    return torch.cuda.get_device_properties(0).total_memory


@pytest.mark.parametrize("name", ["A", "B"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_no_step_grows_the_workspace_after_the_engine_is_built(model_dirs, name, dtype):
    from cpmcu_amd import Engine, EngineOptions, StepEntry
    eng = Engine.from_dir(model_dirs[name], EngineOptions(dtype=dtype, max_tokens=8192, max_slots=20,
                                                          max_step_tokens=128, hip_graph=True))
    ws, gen = eng.workspace.bytes(), eng.workspace.generation
    mem = eng.memory_report()
    assert mem["weight_bytes"] > 0 and mem["workspace_bytes"] == ws and mem["cache_bytes"] == eng.cache.bytes()
    vocab = eng.vocab_size
    slots = [eng.acquire() for _ in range(20)]
    # prompts of every kind of length, one pass and several; then decode steps of every batch size, up to
    # the model's longest sequence (tiny B's block selection is at work from 64 on, long LongRoPE factors and split keys later)
    limit = eng.max_seq_len
    grow = (limit // 2) // 19
    eng.step([StepEntry(s, tiny.random_tokens(3 + grow * i, vocab, i), [2 + grow * i]) for i, s in enumerate(slots)])
    for b in (20, 17, 16, 9, 3, 2, 1):
        for _ in range(2):
            eng.step([StepEntry(s, [5], [0]) for s in slots[:b]])
    more = limit - eng.length(slots[0]) - 4
    eng.step([StepEntry(slots[0], tiny.random_tokens(more, vocab, 77), [more - 1])])
    eng.step([StepEntry(slots[0], [1], [0]), StepEntry(slots[1], [2], [0])])
    assert eng.workspace.grown == [] and eng.workspace.bytes() == ws and eng.workspace.generation == gen
    for s in slots:
        eng.release(s)


def test_a_limit_that_weights_workspace_and_cache_exceed_is_refused_when_the_engine_is_built(model_dirs):
    from cpmcu_amd import Engine, EngineOptions
    from cpmcu_amd.engine.engine import EngineMemoryError
    ok = Engine.from_dir(model_dirs["B"], EngineOptions(dtype="bfloat16", max_tokens=4096, max_slots=4,
                                                        memory_limit=0.5))
    mem = ok.memory_report()
    need = mem["weight_bytes"] + mem["workspace_bytes"] + mem["cache_bytes"]
    # a limit a little below what the same engine needs: refused with the three numbers
    small = (need - 4096) / total_memory()
    with pytest.raises(EngineMemoryError, match=r"weights .* GiB \+ workspace .* GiB \+ cache .* GiB \(for 4096 tokens\)"
                                                r".*the limit is"):
        Engine.from_dir(model_dirs["B"], EngineOptions(dtype="bfloat16", max_tokens=4096, max_slots=4,
                                                       memory_limit=small))
    # the same limit sizes a cache that fits when max_tokens is left open: fewer tokens, whole pages
    sized = Engine.from_dir(model_dirs["B"], EngineOptions(dtype="bfloat16", max_tokens=None, max_slots=4,
                                                           memory_limit=small))
    m2 = sized.memory_report()
    assert 0 < sized.max_tokens < 4096 and sized.max_tokens % 64 == 0
    assert m2["weight_bytes"] + m2["workspace_bytes"] + m2["cache_bytes"] <= small * total_memory()
    # no room even for a page a slot
    with pytest.raises(EngineMemoryError, match="memory limit exceeded"):
        Engine.from_dir(model_dirs["B"], EngineOptions(dtype="bfloat16", max_tokens=None, max_slots=4,
                                                       memory_limit=(mem["weight_bytes"] + 1000) / total_memory()))
    # no limit given, but a cache that the device cannot hold: said at build too, not by the allocator later
    with pytest.raises(EngineMemoryError, match=r"device memory exceeded: weights .* \+ workspace .* \+ cache .*left for"):
        Engine.from_dir(model_dirs["B"], EngineOptions(dtype="bfloat16", max_tokens=2_000_000_000, max_slots=4))
    with pytest.raises(ValueError, match="max_tokens, or a memory_limit"):
        Engine.from_dir(model_dirs["B"], EngineOptions(dtype="bfloat16", max_tokens=None))


@pytest.mark.parametrize("name,batch,seq", [("A", None, None), ("A", 3, 100), ("B", 2, None)])
def test_llm_sizes_its_cache_from_the_memory_limit_and_generates(model_dirs, name, batch, seq):
    """The command line's default: no max_tokens; the cache takes what memory_limit leaves, capped by the
    sequences it is for (cpmcu/llm.py:115-116)."""
    from cpmcu_amd.llm import LLM
    cfg, w = tiny.read_model(model_dirs[name])
    llm = LLM(model_dirs[name], dtype="float32", memory_limit=0.02, max_batch=batch, max_seq_len=seq)
    with pytest.raises(RuntimeError, match="init_storage"):
        llm.load_from_hf()
    longest = llm.init_storage()
    llm.load_from_hf()
    limit = seq or cfg["max_position_embeddings"]
    slots = batch or 1
    assert longest == limit
    # 2 % of the device holds far more than these sequences: the cap decides, in whole pages
    assert llm.engine.max_tokens == slots * (-(-limit // 64) * 64) and llm.engine.cache.max_slots == slots
    mem = llm.engine.memory_report()
    assert mem["weight_bytes"] + mem["workspace_bytes"] + mem["cache_bytes"] <= 0.02 * total_memory()
    prompts = [tiny.random_tokens(7 + 6 * i, cfg["vocab_size"], 50 + i) for i in range(slots + 1)]   # one batch more
    outs = llm.generate(prompts, generation_length=6)
    assert [c.tokens for c in outs] == [plain.greedy(cfg, w, p, 6) for p in prompts]
    llm.engine.cache.check()
    with pytest.raises(ValueError, match="exceeds maximum supported length"):
        llm.prefill(list(range(limit + 1)))


@pytest.mark.parametrize("name", ["A", "B"])
def test_an_engine_of_short_passes_lets_the_checkpoint_layout_go(model_dirs, name):
    """With forward passes of at most 32 tokens no product reads the weights in the checkpoint's layout: the linear
    layers keep their re-laid copy only (and the fused q/k/v copy), the memory figure shows it, and prompts, cut
    into passes of 32, and decode steps give the logits of the plain implementation."""
    import plain_minicpm as plain
    import schedules
    from cpmcu_amd import Engine, EngineOptions
    from cpmcu_amd.parts.linear import Linear
    cfg, w = tiny.read_model(model_dirs[name])
    full = Engine.from_dir(model_dirs[name], EngineOptions(dtype="bfloat16", max_tokens=1024, max_slots=3))
    short = Engine.from_dir(model_dirs[name], EngineOptions(dtype="bfloat16", max_tokens=1024, max_slots=3,
                                                            max_step_tokens=32, hip_graph=True))
    linears = [p for p in short.model.all_parts() if isinstance(p, Linear)]
    assert linears and all(p.weight is None and p.tiled is not None for p in linears)
    assert all(p.weight is not None for p in full.model.all_parts() if isinstance(p, Linear))
    assert short.memory_report()["weight_bytes"] < 0.8 * full.memory_report()["weight_bytes"]
    reqs = {"x": tiny.random_tokens(150, cfg["vocab_size"], 31), "y": tiny.random_tokens(45, cfg["vocab_size"], 32)}
    refs = {r: plain.forward(cfg, w, t).float() for r, t in reqs.items()}
    for what, got in (("whole", schedules.whole(short, reqs)), ("tail", schedules.tail(short, reqs, 20)),
                      ("batched", schedules.batched(short, reqs, {"x": 100, "y": 7}, [("x", "y")]))):
        for r, ref in refs.items():
            assert float((got[r] - ref).abs().max()) < 0.01 * float(ref.abs().max()), (what, r)
    short.cache.check()
