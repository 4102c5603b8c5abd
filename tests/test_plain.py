"""What pins the plain implementation beside the reference's text (CPU).

The reference holds no numeric vectors (its only test checks that the command
line exits with 0 and prints text, tests/test_model_generation.py:186-196), so
every formula is pinned by a library routine it must reduce to, by an invariant,
or by the weight-folding identity of the reference's own converter; each check is
chosen so that a plausible mistake (a sign, a pairing, a norm in the wrong place)
fails it.
"""
import copy
import math

import pytest
import torch
import torch.nn.functional as F

import plain_minicpm as P
import tiny

D = torch.float64


def rnd(*shape, seed=0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=D)


def tensors_for(raw, seed=0, norm_std=0.1):
    """Random float64 tensors with the checkpoint's names (the plain implementation needs nothing else)."""
    H, I, V = raw["hidden_size"], raw["intermediate_size"], raw["vocab_size"]
    nh, nkv = raw["num_attention_heads"], raw.get("num_key_value_heads", raw["num_attention_heads"])
    hd = P.head_dim_of(raw)
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g, dtype=D) * 0.05
    w = {"model.embed_tokens.weight": r(V, H), "model.norm.weight": 1 + norm_std * torch.randn(H, generator=g, dtype=D)}
    if not raw.get("tie_word_embeddings", False):
        w["lm_head.weight"] = r(V, H)
    for i in range(raw["num_hidden_layers"]):
        p = f"model.layers.{i}."
        w[p + "input_layernorm.weight"] = 1 + norm_std * torch.randn(H, generator=g, dtype=D)
        w[p + "post_attention_layernorm.weight"] = 1 + norm_std * torch.randn(H, generator=g, dtype=D)
        w[p + "self_attn.q_proj.weight"] = r(nh * hd, H)
        w[p + "self_attn.k_proj.weight"] = r(nkv * hd, H)
        w[p + "self_attn.v_proj.weight"] = r(nkv * hd, H)
        w[p + "self_attn.o_proj.weight"] = r(H, nh * hd)
        w[p + "mlp.gate_proj.weight"] = r(I, H)
        w[p + "mlp.up_proj.weight"] = r(I, H)
        w[p + "mlp.down_proj.weight"] = r(H, I)
    return w


# ---------------------------------------------------------------------------- norm
def test_rms_norm_is_the_library_routine_and_eps_sits_inside_the_root():
    x, w = rnd(5, 24), rnd(24, seed=1)
    assert torch.allclose(P.rms_norm(x, w, 1e-5), F.rms_norm(x, (24,), w, 1e-5), atol=1e-12)
    c, eps = 3e-3, 1e-5                       # small enough that eps matters: c / sqrt(c^2 + eps), not c / (|c| + eps)
    y = P.rms_norm(torch.full((1, 8), c, dtype=D), torch.ones(8, dtype=D), eps)
    assert torch.allclose(y, torch.full((1, 8), c / math.sqrt(c * c + eps), dtype=D), atol=1e-14)
    assert torch.allclose(P.rms_norm(7.0 * x, w, 0.0), P.rms_norm(x, w, 0.0), atol=1e-12)      # scale invariance
    assert torch.allclose(P.rms_norm(x, 2 * w, 1e-5), 2 * P.rms_norm(x, w, 1e-5))              # weight after, no 1+w


# ---------------------------------------------------------------------------- position encoding
def rope_cfg(hd=8, **kw):
    c = {"hidden_size": hd, "num_attention_heads": 1, "rope_theta": 10000.0, "max_position_embeddings": 64}
    c.update(kw)
    return c


def test_rope_is_the_textbook_rotation_of_pairs_c_and_c_plus_half():
    cfg = rope_cfg(8)
    inv, m = P.rope_inv_freq(cfg)
    assert m == 1.0 and torch.allclose(inv, 10000.0 ** (-torch.arange(0, 8, 2, dtype=D) / 8))
    x = rnd(6, 2, 8)
    pos = torch.tensor([0, 1, 2, 5, 9, 30])
    y = P.apply_rope(x, pos, inv, m)
    assert torch.equal(y[0], x[0])                                              # position 0 is the identity
    z = torch.complex(x[..., :4], x[..., 4:]) * torch.polar(torch.ones(6, 4, dtype=D), pos.to(D)[:, None] * inv)[:, None, :]
    assert torch.allclose(y, torch.cat([z.real, z.imag], -1), atol=1e-12)       # pairing (c, c+hd/2), counter-clockwise
    # a quarter turn of (1, 0) gives (0, 1): fixes the sign of the sine
    q = torch.zeros(1, 1, 2, dtype=D)
    q[0, 0, 0] = 1.0
    out = P.apply_rope(q, torch.tensor([1]), torch.tensor([math.pi / 2], dtype=D), 1.0)
    assert torch.allclose(out.flatten(), torch.tensor([0.0, 1.0], dtype=D), atol=1e-12)


def test_rope_scores_depend_on_distance_only():
    inv, m = P.rope_inv_freq(rope_cfg(16))
    q, k = rnd(1, 1, 16), rnd(1, 1, 16, seed=1)
    def score(pq, pk):
        return (P.apply_rope(q, torch.tensor([pq]), inv, m) * P.apply_rope(k, torch.tensor([pk]), inv, m)).sum()
    assert torch.allclose(score(9, 4), score(105, 100), atol=1e-10)
    assert not torch.allclose(score(9, 4), score(4, 9), atol=1e-6)


def test_longrope_factor_choice_and_magnitude():
    raw = tiny.tiny_b()                                     # original_max 128, max_position 512
    hd = 32
    base = 50000.0 ** (torch.arange(0, hd, 2, dtype=D) / hd)
    inv_long, m = P.rope_inv_freq(raw)
    assert torch.allclose(inv_long, 1 / (torch.tensor(raw["rope_scaling"]["long_factor"], dtype=D) * base))
    assert m == pytest.approx(math.sqrt(1 + math.log(4) / math.log(128)))
    inv_short, _ = P.rope_inv_freq(raw, max_seq_len=128)    # flips exactly at max_seq_len > original_max
    inv_129, _ = P.rope_inv_freq(raw, max_seq_len=129)
    assert torch.allclose(inv_short, 1 / (torch.tensor(raw["rope_scaling"]["short_factor"], dtype=D) * base))
    assert torch.equal(inv_129, inv_long)
    a = tiny.tiny_a()                                       # not stretched: magnitude 1, short factors
    inv_a, m_a = P.rope_inv_freq(a)
    assert m_a == 1.0
    raw["rope_attention_scaling"] = False
    assert P.rope_inv_freq(raw)[1] == 1.0
    # the magnitude multiplies cos and sin: pair norms grow by m
    x = rnd(3, 1, hd)
    y = P.apply_rope(x, torch.tensor([1, 2, 3]), inv_long, m)
    assert torch.allclose((y[..., :16] ** 2 + y[..., 16:] ** 2), m * m * (x[..., :16] ** 2 + x[..., 16:] ** 2))


def test_longrope_factor_stretches_the_positions_of_its_pair():
    """What the factors are for, without restating the formula: a factor f on pair c makes that pair turn f times
    slower, so the rotation at position f * k equals the factor-free rotation (pinned to the textbook form
    above) at position k.  A factor that multiplied the frequency, or one applied to the wrong pair, fails."""
    raw = tiny.tiny_b()
    hd = 32
    fac = [1.0, 2.0, 4.0, 8.0] * 4
    raw["rope_scaling"] = dict(raw["rope_scaling"], long_factor=fac, short_factor=[3.0] * 16)
    raw["rope_attention_scaling"] = False
    inv_long, m = P.rope_inv_freq(raw)                      # max_position 512 > original 128: the long list
    plain_cfg = {k: v for k, v in raw.items() if k != "rope_scaling"}
    inv_plain, m_plain = P.rope_inv_freq(plain_cfg)
    assert m == 1.0 and m_plain == 1.0
    x = rnd(1, 2, hd)
    k = 5
    for f in (1.0, 2.0, 4.0, 8.0):
        stretched = P.apply_rope(x, torch.tensor([int(f) * k]), inv_long, m)
        unstretched = P.apply_rope(x, torch.tensor([k]), inv_plain, 1.0)
        pairs = [c for c in range(16) if fac[c] == f]
        for c in pairs:
            assert torch.allclose(stretched[..., c], unstretched[..., c], atol=1e-12)
            assert torch.allclose(stretched[..., c + 16], unstretched[..., c + 16], atol=1e-12)
        others = [c for c in range(16) if fac[c] != f]
        assert not torch.allclose(stretched[..., others], unstretched[..., others], atol=1e-3)
    # the short list below the original length: every pair three times slower
    inv_short, _ = P.rope_inv_freq(raw, max_seq_len=128)
    assert torch.allclose(P.apply_rope(x, torch.tensor([15]), inv_short, 1.0), P.apply_rope(x, torch.tensor([5]), inv_plain, 1.0),
                          atol=1e-12)


def test_longrope_magnitude_is_a_number_known_in_closed_form():
    """Tiny B stretches 128 positions to 512: ln 4 / ln 128 = 2/7 exactly, so the magnitude is sqrt(9/7).
    A natural logarithm of the wrong quantity (the factor lists, max/1, original/max) does not give this.
    Parity unpinned: the reference engine loads the frequencies only and leaves the magnitude out
    (cpmcu/llm.py:189-192), and takes both from an installed package's model code, which this repository neither
    imports nor reads; no file of the reference holds the number.  What is pinned here is the definition that
    config.json's keys describe, in closed form; `rope_attention_scaling: false` gives the reference's engine."""
    assert P.rope_inv_freq(tiny.tiny_b())[1] == pytest.approx(1.1338934190276817, abs=1e-15)
    raw = tiny.tiny_b()
    raw["max_position_embeddings"] = 128 * 128          # stretched by the original length itself: sqrt(2)
    assert P.rope_inv_freq(raw)[1] == pytest.approx(1.4142135623730951, abs=1e-15)


def test_the_engines_position_part_equals_the_plain_frequencies():
    """parts/rope.py bound for engines of different lengths against the plain implementation (which the tests
    above pin): same factor list at 128 / 129 / 512 positions, same magnitude, float32 roundings only."""
    from cpmcu_amd.config import MiniCPMConfig
    from cpmcu_amd.models.minicpm import layer_specs
    from cpmcu_amd.parts import POSITION_ENCODINGS
    from cpmcu_amd.parts.base import Runtime, Workspace
    for raw in (tiny.tiny_a(), tiny.tiny_b()):
        cfg = MiniCPMConfig.from_dict(raw)
        for max_seq_len in (128, 129, 256, 257, 512):
            part = layer_specs(cfg)[0]["position"].build(POSITION_ENCODINGS)
            part.bind({}, Runtime(torch.device("cpu"), torch.float32, Workspace("cpu"), max_seq_len))
            inv, m = part.rotary_params()
            want, want_m = P.rope_inv_freq(raw, max_seq_len)
            assert inv.dtype == torch.float32 and torch.equal(inv, want.to(torch.float32))
            assert m == pytest.approx(want_m, abs=1e-15)
    raw = tiny.tiny_b()
    raw["rope_attention_scaling"] = False               # what the reference does (cpmcu/llm.py:190-192)
    part = layer_specs(MiniCPMConfig.from_dict(raw))[0]["position"].build(POSITION_ENCODINGS)
    assert part.rotary_params()[1] == 1.0


# ---------------------------------------------------------------------------- attention
def test_dense_attention_is_the_library_routine():
    T, nh, nkv, hd = 13, 6, 2, 8
    q, k, v = rnd(T, nh, hd), rnd(T, nkv, hd, seed=1), rnd(T, nkv, hd, seed=2)
    ref = F.scaled_dot_product_attention(q.transpose(0, 1)[None], k.repeat_interleave(3, 1).transpose(0, 1)[None],
                                         v.repeat_interleave(3, 1).transpose(0, 1)[None], is_causal=True)[0].transpose(0, 1)
    assert torch.allclose(P.dense_attention(q, k, v), ref, atol=1e-12)
    # head h reads kv head h // G (not h % nkv): heads 0..2 share kv head 0
    v2 = v.clone()
    v2[:, 1] += 1.0
    out2 = P.dense_attention(q, k, v2)
    assert torch.allclose(out2[:, :3], ref[:, :3]) and torch.allclose(out2[:, 3:], ref[:, 3:] + 1.0)
    assert torch.allclose(P.dense_attention(q[:1], k[:1], v[:1])[0, 4], v[0, 1])     # one token returns its value


def test_ffn_is_silu_gate_times_up():
    x, wg, wu, wd = rnd(4, 10), rnd(14, 10, seed=1), rnd(14, 10, seed=2), rnd(10, 14, seed=3)
    assert torch.allclose(P.gated_ffn(x, wg, wu, wd), F.linear(F.silu(F.linear(x, wg)) * F.linear(x, wu), wd), atol=1e-12)


# ---------------------------------------------------------------------------- muP scalars
@pytest.mark.parametrize("raw", [tiny.tiny_a(), tiny.tiny_b()], ids=["A-tied", "B-untied"])
def test_scalars_fold_into_weights_as_the_reference_converter_does(raw):
    """scripts/model_convert/minicpm2llama.py:28-39: embed *= scale_emb, lm_head /= hidden/dim_model_base,
    o_proj and down_proj *= scale_depth/sqrt(L) give a scalar-free decoder with the same logits."""
    raw.pop("sparse_config", None)
    w = tensors_for(raw, seed=3)
    toks = tiny.random_tokens(12, raw["vocab_size"], 1)
    ref = P.forward(raw, w, toks)
    s_e, s_r, s_l = P.mup_scalars(raw)
    f = dict(w)
    head = w.get("lm_head.weight", w["model.embed_tokens.weight"])       # tied: the head reads the unscaled table
    f["lm_head.weight"] = head * s_l
    f["model.embed_tokens.weight"] = w["model.embed_tokens.weight"] * s_e
    for i in range(raw["num_hidden_layers"]):
        for n in ("self_attn.o_proj.weight", "mlp.down_proj.weight"):
            f[f"model.layers.{i}.{n}"] = w[f"model.layers.{i}.{n}"] * s_r
    plain_cfg = {k: v for k, v in raw.items() if k not in ("scale_emb", "dim_model_base", "scale_depth")}
    plain_cfg["tie_word_embeddings"] = False
    assert P.mup_scalars(plain_cfg) == (1.0, 1.0, 1.0)
    assert torch.allclose(P.forward(plain_cfg, f, toks), ref, atol=1e-10)
    # and the neutral values are a no-op
    neutral = dict(plain_cfg, scale_emb=1, scale_depth=math.sqrt(raw["num_hidden_layers"]), dim_model_base=raw["hidden_size"])
    assert torch.allclose(P.forward(neutral, f, toks), ref, atol=1e-10)


def test_only_distances_count_in_the_whole_model():
    raw = tiny.tiny_a()
    w = tensors_for(raw, seed=4)
    a = rnd(9, raw["hidden_size"])
    inv, m = P.rope_inv_freq(raw)
    o0 = P.attention_layer(raw, w, "model.layers.0.", a, torch.arange(9), inv, m)
    o7 = P.attention_layer(raw, w, "model.layers.0.", a, torch.arange(9) + 77, inv, m)
    assert torch.allclose(o0, o7, atol=1e-10)


def test_logits_of_a_prefix_do_not_change_when_tokens_follow():
    raw = tiny.tiny_b()
    w = tensors_for(raw, seed=5)
    toks = tiny.random_tokens(120, raw["vocab_size"], 2)
    full = P.forward(raw, w, toks)
    assert torch.allclose(P.forward(raw, w, toks[:97]), full[:97], atol=1e-10)


# ---------------------------------------------------------------------------- InfLLM-v2
SC = {"kernel_size": 8, "kernel_stride": 4, "block_size": 16, "init_blocks": 1, "topk": 3, "window_size": 32, "dense_len": 40}


def test_compressed_keys_are_average_pooling():
    k = rnd(50, 2, 6)
    ck = P.compressed_keys(k, 8, 4)
    ref = F.avg_pool1d(k.permute(1, 2, 0), 8, 4).permute(2, 0, 1)
    assert ck.shape == (11, 2, 6) and torch.allclose(ck, ref, atol=1e-12)
    assert P.compressed_keys(k[:7], 8, 4).shape[0] == 0


def test_block_scores_are_max_pooling_5_4_1_and_ties_go_to_the_lower_block():
    """With kernel 2*stride and block 4*stride the pooling equals max_pool1d(kernel 5, stride 4, padding 1),
    which is what the reference computes (src/model/minicpm4/minicpm4_kvcache.cuh:64-108)."""
    hd, nkv, G = 4, 1, 2
    p = 200                                            # q_block 12, candidates 0..10, window blocks 11, 12
    sc = dict(SC, topk=3, init_blocks=0)
    n_vis = (p - 8) // 4 + 1
    ck = rnd(n_vis, nkv, hd, seed=7)
    q = rnd(G, hd, seed=8)
    s = torch.softmax((q @ ck[:, 0].T) * hd ** -0.5, -1).sum(0)
    pooled = F.max_pool1d(s[None, None], 5, 4, 1)[0, 0]
    want = sorted(sorted(range(11), key=lambda b: (-pooled[b].item(), b))[:3])
    got = P.infllm_select(q, ck, p, sc, nkv)[0]
    assert got == want + [11, 12]
    # all compressed keys equal: every score ties, the lowest blocks win; init blocks count toward topk
    flat = torch.ones(n_vis, nkv, hd, dtype=D)
    assert P.infllm_select(q, flat, p, sc, nkv)[0] == [0, 1, 2, 11, 12]
    assert P.infllm_select(q, flat, p, dict(sc, init_blocks=2, topk=2), nkv)[0] == [0, 1, 11, 12]
    # a compressed key is visible only when it ends before the query: st*j + ks <= p
    assert P.infllm_select(q, ck, 40, dict(sc, dense_len=0), nkv)[0] == [0, 1, 2]       # blocks 1, 2 are the window


def test_dense_below_dense_len_and_when_topk_covers_all_candidates():
    raw = tiny.tiny_b()
    w = tensors_for(raw, seed=6)
    toks = tiny.random_tokens(150, raw["vocab_size"], 3)
    dense = P.forward(raw, w, toks, sparse=False)
    sparse = P.forward(raw, w, toks)
    dl = raw["sparse_config"]["dense_len"]
    assert torch.allclose(sparse[:dl], dense[:dl], atol=1e-12)
    assert (sparse[dl + 40:] - dense[dl + 40:]).abs().max() > 1e-6           # the top-k really prunes
    big = copy.deepcopy(raw)
    big["sparse_config"]["topk"] = 100
    assert torch.allclose(P.forward(big, w, toks), dense, atol=1e-12)


def test_far_key_is_found_by_the_block_scores():
    """One early key made to stand out is attended to through its block although it lies outside the window."""
    T, nh, nkv, hd = 160, 2, 1, 8
    sc = dict(SC, topk=2, init_blocks=1, dense_len=0)
    q, k, v = 0.1 * rnd(T, nh, hd), 0.1 * rnd(T, nkv, hd, seed=1), rnd(T, nkv, hd, seed=2)
    k[37:41] = 0
    k[37:41, 0, 0] = 30.0                      # block 2 (tokens 32..47)
    q[-1, :, :] = 0
    q[-1, :, 0] = 30.0
    allowed = P.sparse_allowed(q, k, sc)
    assert allowed[-1, 0, 37] and allowed[-1, 0, 0] and allowed[-1, 0, 159] and not allowed[-1, 0, 60]
    out = P.dense_attention(q, k, v, allowed)[-1]
    assert torch.allclose(out[0], v[37:41, 0].mean(0), atol=1e-6)
