"""Two groups of layers with different cache needs in one model: a layer of the package's attention, which
keeps every key, and a layer of a windowed attention defined here, whose group keeps a trailing window and
gives older pages back while the sequence grows.  Registered, built from a model folder and stepped without a
change to the package's files (GPU)."""
from dataclasses import dataclass
from typing import Any, Dict

import pytest
import torch

pytestmark = pytest.mark.gpu

BS = 32          # the windowed layer reads whole blocks of 32 keys: from the block of position p - window + 1 on


def _define():
    from cpmcu_amd import ops
    from cpmcu_amd.cache import CacheNeeds, StreamSpec
    from cpmcu_amd.config.base import ModelConfig, field_from
    from cpmcu_amd.models.decoder import DecoderModel
    from cpmcu_amd.parts import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS, LMHead, TokenEmbedding)
    from cpmcu_amd.parts.attention import GQAAttention
    from cpmcu_amd.registry import Architecture, register_architecture

    class WindowAttention(GQAAttention):
        """The package's attention over the blocks of BS keys that reach back `window` tokens from each query:
        its cache entry asks for a window, so its group drops pages that no query can read any more."""

        def __init__(self, window: int, **kw):
            super().__init__(**kw)
            self.window = window

        def cache_needs(self):
            w = self.nkv * self.hd
            return CacheNeeds(streams=(("k", StreamSpec(w)), ("v", StreamSpec(w))), window=self.window)

        def forward(self, h, ctx, cache, writes_cache=True, row_scale=None):
            assert cache.window == self.window
            q = self.project_and_store(h, ctx, cache, writes_cache, row_scale)
            n = q.shape[0]
            pos = ctx.positions.long()
            first = (pos - self.window + 1).clamp(min=0) // BS
            count = pos // BS - first + 1
            max_sel = self.window // BS + 1
            blocks = (first[:, None] + torch.arange(max_sel, device=q.device)[None, :]).to(torch.int32)
            sel_blocks = blocks[:, None, :].expand(n, self.nkv, max_sel).contiguous()
            sel_count = count.to(torch.int32)[:, None].expand(n, self.nkv).contiguous()
            out = ctx.ws.get("toy.window.out", tuple(q.shape), q.dtype)
            ops.attention(q, out, self.nh, self.nkv, self.hd, self.scale, cache.streams["k"], cache.streams["v"],
                          cache.page_table, cache.page_size, ctx, sel_blocks, sel_count, BS, 0)
            return self.o.forward(out, ctx, "attn.o", out_dtype=torch.float32, partials=True)

    @dataclass(frozen=True)
    class ToyConfig(ModelConfig):
        vocab_size: int = 0
        hidden_size: int = 0
        num_attention_heads: int = 0
        num_key_value_heads: int = 0
        head_dim: int = 0
        intermediate_size: int = 0
        window: int = 64
        rope_theta: float = 10000.0
        rms_norm_eps: float = 1e-5
        max_position_embeddings: int = 512

        @property
        def longest_sequence(self):
            return self.max_position_embeddings

        @classmethod
        def from_dict(cls, raw: Dict[str, Any]):
            return cls(raw["architectures"][0], *(field_from(raw, k, t) for k, t in (
                ("vocab_size", int), ("hidden_size", int), ("num_attention_heads", int), ("num_key_value_heads", int),
                ("head_dim", int), ("intermediate_size", int), ("window", int), ("rope_theta", float),
                ("rms_norm_eps", float), ("max_position_embeddings", int))))

        def to_dict(self):
            d = {k: getattr(self, k) for k in ("vocab_size", "hidden_size", "num_attention_heads",
                                               "num_key_value_heads", "head_dim", "intermediate_size", "window",
                                               "rope_theta", "rms_norm_eps", "max_position_embeddings")}
            d["architectures"] = [self.architecture]
            return d

    MIXERS.register("toy_window_attention", WindowAttention)

    def build(cfg: ToyConfig, all_windowed: bool = False):
        layers = []
        for i, kind in enumerate(("toy_window_attention" if all_windowed else "gqa_attention", "toy_window_attention")):
            p = f"layers.{i}."
            position = POSITION_ENCODINGS.build("rope", head_dim=cfg.head_dim, theta=cfg.rope_theta)
            extra = {"window": cfg.window} if kind == "toy_window_attention" else {}
            layers.append(BLOCKS.build(
                "pre_norm",
                mixer_norm=NORMS.build("rms_norm", name=p + "norm1.weight", hidden_size=cfg.hidden_size, eps=cfg.rms_norm_eps),
                mixer=MIXERS.build(kind, prefix=p + "attn.", hidden_size=cfg.hidden_size,
                                   num_heads=cfg.num_attention_heads, num_kv_heads=cfg.num_key_value_heads,
                                   head_dim=cfg.head_dim, position=position, **extra),
                ff_norm=NORMS.build("rms_norm", name=p + "norm2.weight", hidden_size=cfg.hidden_size, eps=cfg.rms_norm_eps),
                feed_forward=FEED_FORWARDS.build("gated_silu", prefix=p + "mlp.", hidden_size=cfg.hidden_size,
                                                 intermediate_size=cfg.intermediate_size),
                residual_scale=0.7))
        emb = TokenEmbedding("embed.weight", cfg.vocab_size, cfg.hidden_size, 1.0)
        head = LMHead("head.weight", cfg.vocab_size, cfg.hidden_size, 1.0, tied_to=emb)
        norm = NORMS.build("rms_norm", name="norm.weight", hidden_size=cfg.hidden_size, eps=cfg.rms_norm_eps)
        return DecoderModel(cfg, emb, layers, norm, head)

    # an option of this architecture's own, declared to the registry (EngineOptions.model_options hands it over)
    register_architecture(Architecture("ToyWindowForCausalLM", ToyConfig, build, options={"all_windowed": False}),
                          replace=True)
    return ToyConfig


def plain_toy(raw, w, toks, all_windowed=False):
    """The same model, whole sequence, in float64 on the CPU: layer 0 sees every key before it (unless
    all_windowed), layer 1 the keys from the block of position p - window + 1 on."""
    import torch.nn.functional as F
    W = {k: v.double() for k, v in w.items()}
    n = len(toks)
    nh, nkv, hd, win = raw["num_attention_heads"], raw["num_key_value_heads"], raw["head_dim"], raw["window"]
    eps = raw["rms_norm_eps"]
    x = W["embed.weight"][torch.tensor(toks)]
    pos = torch.arange(n, dtype=torch.float64)
    inv = 1.0 / raw["rope_theta"] ** (torch.arange(0, hd, 2, dtype=torch.float64) / hd)
    ang = pos[:, None] * inv.float().double()[None, :]
    cos, sin = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]

    def rot(t):                                               # [n, heads, hd], pairs (c, c + hd/2)
        a, b = t[..., :hd // 2], t[..., hd // 2:]
        return torch.cat([a * cos - b * sin, a * sin + b * cos], dim=-1)

    for i in range(2):
        p = f"layers.{i}."
        a = F.rms_norm(x, (x.shape[-1],), W[p + "norm1.weight"], eps)
        q = rot((a @ W[p + "attn.q_proj.weight"].T).view(n, nh, hd))
        k = rot((a @ W[p + "attn.k_proj.weight"].T).view(n, nkv, hd))
        v = (a @ W[p + "attn.v_proj.weight"].T).view(n, nkv, hd)
        k, v = k.repeat_interleave(nh // nkv, dim=1), v.repeat_interleave(nh // nkv, dim=1)
        s = torch.einsum("qhd,khd->hqk", q, k) * hd ** -0.5
        qi, ki = torch.arange(n)[:, None], torch.arange(n)[None, :]
        seen = ki <= qi
        if i == 1 or all_windowed:
            seen = seen & (ki >= ((qi - win + 1).clamp(min=0) // BS) * BS)
        s = s.masked_fill(~seen[None], float("-inf"))
        o = torch.einsum("hqk,khd->qhd", torch.softmax(s, dim=-1), v).reshape(n, nh * hd)
        x = x + 0.7 * (o @ W[p + "attn.o_proj.weight"].T)
        f = F.rms_norm(x, (x.shape[-1],), W[p + "norm2.weight"], eps)
        x = x + 0.7 * ((F.silu(f @ W[p + "mlp.gate_proj.weight"].T) * (f @ W[p + "mlp.up_proj.weight"].T))
                       @ W[p + "mlp.down_proj.weight"].T)
    return F.rms_norm(x, (x.shape[-1],), W["norm.weight"], eps) @ W["embed.weight"].T


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_windowed_layer_beside_a_full_one(tmp_path, dtype):
    from safetensors.torch import load_file
    from cpmcu_amd import Engine, EngineOptions, StepEntry
    from cpmcu_amd.parts import MIXERS
    from cpmcu_amd.registry import unregister_architecture
    from cpmcu_amd.weights import write_model_dir
    ToyConfig = _define()
    try:
        raw = {"architectures": ["ToyWindowForCausalLM"], "vocab_size": 120, "hidden_size": 64, "num_attention_heads": 4,
               "num_key_value_heads": 2, "head_dim": 16, "intermediate_size": 96, "window": 64, "rope_theta": 10000.0,
               "rms_norm_eps": 1e-5, "max_position_embeddings": 512}
        write_model_dir(ToyConfig.from_dict(raw), str(tmp_path), seed=6, std=0.1, norm_std=0.1)
        w = load_file(str(tmp_path / "model.safetensors"))
        eng = Engine.from_dir(str(tmp_path), EngineOptions(dtype=dtype, max_tokens=1024, max_slots=2,
                                                           max_step_tokens=128))
        cache = eng.cache
        assert len(cache.groups) == 2                        # every key / a window of them: storage of their own
        full = next(g for g in cache.groups if g.needs.window is None)
        win = next(g for g in cache.groups if g.needs.window == 64)
        n = 333
        toks = [int(t) for t in torch.randint(0, 120, (n,), generator=torch.Generator().manual_seed(2))]
        ref = plain_toy(raw, w, toks).float()
        tol = 1e-4 if dtype == "float32" else 0.03 * float(ref.abs().max())
        # the whole prompt at once (the engine cuts it into passes of 128 tokens), every logit
        s = eng.acquire()
        whole = eng.step([StepEntry(s, toks, list(range(n)))]).cpu()
        assert float((whole - ref).abs().max()) < tol
        assert full.held(s) == -(-n // 64) and win.held(s) <= 64 // 64 + 2
        eng.release(s)
        cache.check()
        # a prompt of 150 tokens, then token by token, beside a second sequence that starts later; the window
        # group never holds more than the pages a window touches, the other group all of them
        s = eng.acquire()
        outs = [eng.step([StepEntry(s, toks[:150], list(range(150)))]).cpu()]
        other = eng.acquire()
        for i in range(150, n):
            lg = eng.step([StepEntry(s, [toks[i]], [0]), StepEntry(other, [toks[i - 150]], [0])]).cpu()
            outs.append(lg[:1])
            assert float((lg[1] - ref[i - 150]).abs().max()) < tol, i
            assert win.held(s) <= 3 and full.held(s) == i // 64 + 1
        assert float((torch.cat(outs) - ref).abs().max()) < tol
        eng.release(s)
        eng.release(other)
        cache.check()
    finally:
        unregister_architecture("ToyWindowForCausalLM")
        MIXERS.unregister("toy_window_attention")


def test_a_model_of_windowed_layers_only_outgrows_the_cache_pool(tmp_path):
    """With the architecture's own option `all_windowed` both layers keep a window: the one cache group then holds
    a few pages a sequence however long it grows, so a sequence of 700 tokens runs in a cache of 256 (the prompt
    in passes of 64 tokens, then token by token), and the planner's question of how many pages a sequence needs
    is answered by the group."""
    from safetensors.torch import load_file
    from cpmcu_amd import Engine, EngineOptions, StepEntry, StepError
    from cpmcu_amd.parts import MIXERS
    from cpmcu_amd.registry import unregister_architecture
    from cpmcu_amd.weights import write_model_dir
    ToyConfig = _define()
    try:
        raw = {"architectures": ["ToyWindowForCausalLM"], "vocab_size": 120, "hidden_size": 64, "num_attention_heads": 4,
               "num_key_value_heads": 2, "head_dim": 16, "intermediate_size": 96, "window": 64, "rope_theta": 10000.0,
               "rms_norm_eps": 1e-5, "max_position_embeddings": 1024}
        write_model_dir(ToyConfig.from_dict(raw), str(tmp_path), seed=8, std=0.1, norm_std=0.1)
        w = load_file(str(tmp_path / "model.safetensors"))
        with pytest.raises(ValueError, match="no option 'windowed'"):
            Engine.from_dir(str(tmp_path), EngineOptions(dtype="float32", max_tokens=256, model_options={"windowed": True}))
        eng = Engine.from_dir(str(tmp_path), EngineOptions(dtype="float32", max_tokens=256, max_slots=2, max_step_tokens=64,
                                                           model_options={"all_windowed": True}))
        cache = eng.cache
        assert len(cache.groups) == 1 and cache.groups[0].needs.window == 64 and cache.capacity() == [4]
        assert cache.pages_to_hold(700, 64) == [3] and cache.groups[0].table.shape[1] == 16
        n = 700
        toks = [int(t) for t in torch.randint(0, 120, (n,), generator=torch.Generator().manual_seed(3))]
        ref = plain_toy(raw, w, toks, all_windowed=True).float()
        s = eng.acquire()
        outs = [eng.step([StepEntry(s, toks[:300], list(range(300)))]).cpu()]        # more tokens than the pool holds
        for i in range(300, n):
            outs.append(eng.step([StepEntry(s, [toks[i]], [0])]).cpu())
            assert cache.groups[0].held(s) <= 3
        assert eng.length(s) == n
        got = torch.cat(outs)
        err = (got - ref).abs().amax(1)
        assert float(err.max()) < 1e-4, f"first wrong position {int((err >= 1e-4).nonzero()[0])}"
        # a step that brings more tokens at once than the pool has room for is still refused, and changes nothing
        other = eng.acquire()
        eng.max_step_tokens = 512
        with pytest.raises(StepError, match="cache is full"):
            eng.step([StepEntry(other, toks[:200], [])])
        assert eng.length(other) == 0
        eng.release(s)
        eng.release(other)
        cache.check()
    finally:
        unregister_architecture("ToyWindowForCausalLM")
        MIXERS.unregister("toy_window_attention")
