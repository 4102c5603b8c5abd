"""Another arrangement of a layer's parts, and a schedule in which one layer reads another layer's cache: both
defined here, outside the package, registered, built from a model folder and stepped (GPU).

The block is a *parallel* one: mixer and feed-forward read the same normed rows and their branches are added to
the residual stream together, x += s * (Mixer(norm(x)) + FeedForward(norm(x))), with one norm a layer.  The
schedule runs layers 0, 1, 2 and lets layer 2 read the keys and values that layer 0 wrote: its mixer projects
queries only.  Neither is a model of anyone's."""
from dataclasses import dataclass
from typing import Any, Dict

import pytest
import torch

pytestmark = pytest.mark.gpu

ARCH = "ToyParallelForCausalLM"
SCALE = 0.6


def _define():
    from cpmcu_amd.config.base import ModelConfig, field_from
    from cpmcu_amd.models.decoder import DecoderModel, Run
    from cpmcu_amd.parts import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS, Block, LMHead,
                                 TokenEmbedding)
    from cpmcu_amd.parts.base import branch_tensor
    from cpmcu_amd.registry import Architecture, register_architecture

    class ParallelBlock(Block):
        def __init__(self, norm, mixer, feed_forward, residual_scale: float):
            self.norm, self.mixer, self.feed_forward = norm, mixer, feed_forward
            self.residual_scale = float(residual_scale)

        def parts(self):
            return [self.norm, self.mixer, self.feed_forward]

        def forward(self, stream, ctx, cache, writes_cache=True):
            # the norm adds what the layer before left pending, as every norm of the package does
            h = self.norm.forward(stream.x, stream.pending, stream.pending_scale, ctx, tag="toy.parallel.h")
            a = branch_tensor(self.mixer.forward(h, ctx, cache, writes_cache))
            f = branch_tensor(self.feed_forward.forward(h, ctx))
            a = a.sum(0) if a.dim() == 3 else a                       # partial sums of a split product
            f = f.sum(0) if f.dim() == 3 else f
            stream.pending = a.float() + f.float()
            stream.pending_scale = self.residual_scale

    @dataclass(frozen=True)
    class ToyConfig(ModelConfig):
        vocab_size: int = 0
        hidden_size: int = 0
        num_attention_heads: int = 0
        num_key_value_heads: int = 0
        head_dim: int = 0
        intermediate_size: int = 0
        rope_theta: float = 10000.0
        rms_norm_eps: float = 1e-5
        max_position_embeddings: int = 256

        @property
        def longest_sequence(self):
            return self.max_position_embeddings

        @classmethod
        def from_dict(cls, raw: Dict[str, Any]):
            return cls(raw["architectures"][0], *(field_from(raw, k, t) for k, t in (
                ("vocab_size", int), ("hidden_size", int), ("num_attention_heads", int), ("num_key_value_heads", int),
                ("head_dim", int), ("intermediate_size", int), ("rope_theta", float), ("rms_norm_eps", float),
                ("max_position_embeddings", int))))

        def to_dict(self):
            d = {k: getattr(self, k) for k in ("vocab_size", "hidden_size", "num_attention_heads",
                                               "num_key_value_heads", "head_dim", "intermediate_size", "rope_theta",
                                               "rms_norm_eps", "max_position_embeddings")}
            d["architectures"] = [self.architecture]
            return d

    BLOCKS.register("toy_parallel", ParallelBlock)

    def build(cfg: ToyConfig):
        layers = []
        for i in range(3):
            p = f"layers.{i}."
            position = POSITION_ENCODINGS.build("rope", head_dim=cfg.head_dim, theta=cfg.rope_theta)
            layers.append(BLOCKS.build(
                "toy_parallel",
                norm=NORMS.build("rms_norm", name=p + "norm.weight", hidden_size=cfg.hidden_size, eps=cfg.rms_norm_eps),
                mixer=MIXERS.build("gqa_attention", prefix=p + "attn.", hidden_size=cfg.hidden_size,
                                   num_heads=cfg.num_attention_heads, num_kv_heads=cfg.num_key_value_heads,
                                   head_dim=cfg.head_dim, position=position),
                feed_forward=FEED_FORWARDS.build("gated_silu", prefix=p + "mlp.", hidden_size=cfg.hidden_size,
                                                 intermediate_size=cfg.intermediate_size),
                residual_scale=SCALE))
        emb = TokenEmbedding("embed.weight", cfg.vocab_size, cfg.hidden_size, 1.0)
        head = LMHead("head.weight", cfg.vocab_size, cfg.hidden_size, 1.0, tied_to=emb)
        norm = NORMS.build("rms_norm", name="norm.weight", hidden_size=cfg.hidden_size, eps=cfg.rms_norm_eps)
        # the order of the layers is data: layer 2 reads the cache entry that layer 0 wrote and writes none
        schedule = [Run(0, 0), Run(1, 1), Run(2, 0, writes_cache=False)]
        return DecoderModel(cfg, emb, layers, norm, head, schedule)

    register_architecture(Architecture(ARCH, ToyConfig, build), replace=True)
    return ToyConfig


def plain_toy(raw, w, toks):
    """The same model, whole sequence, float64, no cache."""
    import torch.nn.functional as F
    W = {k: v.double() for k, v in w.items()}
    n = len(toks)
    nh, nkv, hd, eps = raw["num_attention_heads"], raw["num_key_value_heads"], raw["head_dim"], raw["rms_norm_eps"]
    x = W["embed.weight"][torch.tensor(toks)]
    pos = torch.arange(n, dtype=torch.float64)
    inv = (1.0 / raw["rope_theta"] ** (torch.arange(0, hd, 2, dtype=torch.float64) / hd)).float().double()
    cos, sin = torch.cos(pos[:, None] * inv)[:, None, :], torch.sin(pos[:, None] * inv)[:, None, :]

    def rot(t):
        a, b = t[..., :hd // 2], t[..., hd // 2:]
        return torch.cat([a * cos - b * sin, a * sin + b * cos], dim=-1)

    kept = {}
    for i in range(3):
        p = f"layers.{i}."
        h = F.rms_norm(x, (x.shape[-1],), W[p + "norm.weight"], eps)
        q = rot((h @ W[p + "attn.q_proj.weight"].T).view(n, nh, hd))
        if i == 2:
            k, v = kept[0]                                       # layer 0's keys and values
        else:
            k = rot((h @ W[p + "attn.k_proj.weight"].T).view(n, nkv, hd))
            v = (h @ W[p + "attn.v_proj.weight"].T).view(n, nkv, hd)
            kept[i] = (k, v)
        o = F.scaled_dot_product_attention(q.transpose(0, 1), k.repeat_interleave(nh // nkv, 1).transpose(0, 1),
                                           v.repeat_interleave(nh // nkv, 1).transpose(0, 1), is_causal=True)
        a = o.transpose(0, 1).reshape(n, nh * hd) @ W[p + "attn.o_proj.weight"].T
        f = (F.silu(h @ W[p + "mlp.gate_proj.weight"].T) * (h @ W[p + "mlp.up_proj.weight"].T)) @ W[p + "mlp.down_proj.weight"].T
        x = x + SCALE * (a + f)
    return F.rms_norm(x, (x.shape[-1],), W["norm.weight"], eps) @ W["embed.weight"].T


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_parallel_block_and_a_layer_that_reads_another_layers_cache(tmp_path, dtype):
    from safetensors.torch import load_file
    from cpmcu_amd import Engine, EngineOptions, StepEntry
    from cpmcu_amd.parts import BLOCKS
    from cpmcu_amd.registry import unregister_architecture
    from cpmcu_amd.weights import write_model_dir
    ToyConfig = _define()
    try:
        raw = {"architectures": [ARCH], "vocab_size": 120, "hidden_size": 72, "num_attention_heads": 6,
               "num_key_value_heads": 2, "head_dim": 16, "intermediate_size": 88, "rope_theta": 3000.0,
               "rms_norm_eps": 1e-5, "max_position_embeddings": 256}
        write_model_dir(ToyConfig.from_dict(raw), str(tmp_path), seed=11, std=0.1, norm_std=0.1)
        w = load_file(str(tmp_path / "model.safetensors"))
        eng = Engine.from_dir(str(tmp_path), EngineOptions(dtype=dtype, max_tokens=1024, max_slots=3, hip_graph=True))
        # two cache entries for three runs: the third run holds none
        assert eng.model.n_cache_entries == 2 and len(eng.cache.groups) == 1 and eng.uses_graph
        g = torch.Generator().manual_seed(2)
        reqs = {r: [int(t) for t in torch.randint(0, 120, (n,), generator=g)] for r, n in (("a", 150), ("b", 41), ("c", 77))}
        refs = {r: plain_toy(raw, w, t).float() for r, t in reqs.items()}
        tol = {r: (3e-5 if dtype == "float32" else 0.03 * float(ref.abs().max())) for r, ref in refs.items()}
        # whole
        for r, toks in reqs.items():
            s = eng.acquire()
            got = eng.step([StepEntry(s, toks, list(range(len(toks))))]).cpu()
            eng.release(s)
            assert float((got - refs[r]).abs().max()) < tol[r], (r, "whole")
        # unequal prompts together, then one token each from captured graphs; the shorter ones end earlier
        fed = {"a": 100, "b": 9, "c": 60}
        slots = {r: eng.acquire() for r in reqs}
        lg = eng.step([StepEntry(slots[r], reqs[r][:fed[r]], [fed[r] - 1]) for r in reqs]).cpu()
        for i, r in enumerate(reqs):
            assert float((lg[i] - refs[r][fed[r] - 1]).abs().max()) < tol[r], (r, "prompt")
        live = list(reqs)
        while live:
            lg = eng.step([StepEntry(slots[r], [reqs[r][fed[r]]], [0]) for r in live]).cpu()
            for i, r in enumerate(live):
                assert float((lg[i] - refs[r][fed[r]]).abs().max()) < tol[r], (r, fed[r])
                fed[r] += 1
            for r in list(live):
                if fed[r] >= len(reqs[r]):
                    eng.release(slots.pop(r))
                    live.remove(r)
        assert eng._graphs and not eng.cache.live
        eng.cache.check()
    finally:
        unregister_architecture(ARCH)
        BLOCKS.unregister("toy_parallel")
