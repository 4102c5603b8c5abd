"""A mixer with state of its own, defined here, is registered, built from a model folder and stepped
without a change to the package's files (GPU)."""
import json
from dataclasses import dataclass
from typing import Any, Dict, List, Mapping, Optional

import pytest
import torch

pytestmark = pytest.mark.gpu


def _define():
    from cpmcu_amd.cache import CacheNeeds, StateSpec
    from cpmcu_amd.config.base import ModelConfig, field_from
    from cpmcu_amd.models.decoder import DecoderModel, Run
    from cpmcu_amd.parts import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, LMHead, Linear, Mixer, TokenEmbedding)
    from cpmcu_amd.registry import Architecture, register_architecture

    class DecayMixer(Mixer):
        """h_t = decay * h_{t-1} + x_t per sequence (fixed-size state in the slot), out = W h_t."""

        def __init__(self, prefix: str, hidden_size: int, decay: float):
            self.hidden_size, self.decay = hidden_size, decay
            self.proj = Linear([(prefix + "proj.weight", hidden_size)], hidden_size)

        def parts(self):
            return [self.proj]

        def bind(self, tensors, rt):
            self.rt = rt

        def cache_needs(self):
            return CacheNeeds(state=(("h", StateSpec((self.hidden_size,), torch.float32)),))

        graph_capturable = False        # the scan below reads the batch on the host and loops in Python

        def forward(self, h, ctx, cache, writes_cache=True):
            state = cache.state["h"]
            out = torch.empty_like(h)
            o = 0
            for slot, q in zip(ctx.seq_slot.tolist(), ctx.q_lens):      # a scan over each sequence's tokens
                s = state[slot]
                for j in range(q):
                    s = self.decay * s + h[o + j].float()
                    out[o + j] = s.to(h.dtype)
                if writes_cache:
                    state[slot] = s
                o += q
            return self.proj.forward(out, ctx, "toy.proj", out_dtype=torch.float32)

    @dataclass(frozen=True)
    class ToyConfig(ModelConfig):
        vocab_size: int = 0
        hidden_size: int = 0
        num_hidden_layers: int = 0
        intermediate_size: int = 0
        decay: float = 0.5
        rms_norm_eps: float = 1e-5
        max_position_embeddings: int = 128

        @property
        def longest_sequence(self):
            return self.max_position_embeddings

        @classmethod
        def from_dict(cls, raw: Dict[str, Any]):
            return cls(raw["architectures"][0], field_from(raw, "vocab_size", int), field_from(raw, "hidden_size", int),
                       field_from(raw, "num_hidden_layers", int), field_from(raw, "intermediate_size", int),
                       field_from(raw, "decay", float), field_from(raw, "rms_norm_eps", float),
                       field_from(raw, "max_position_embeddings", int, 128))

        def to_dict(self):
            return {"architectures": [self.architecture], "vocab_size": self.vocab_size, "hidden_size": self.hidden_size,
                    "num_hidden_layers": self.num_hidden_layers, "intermediate_size": self.intermediate_size,
                    "decay": self.decay, "rms_norm_eps": self.rms_norm_eps,
                    "max_position_embeddings": self.max_position_embeddings}

    MIXERS.register("toy_decay", DecayMixer)

    def build(cfg: ToyConfig):
        layers = []
        for i in range(cfg.num_hidden_layers):
            p = f"layers.{i}."
            layers.append(BLOCKS.build(
                "pre_norm",
                mixer_norm=NORMS.build("rms_norm", name=p + "norm1.weight", hidden_size=cfg.hidden_size, eps=cfg.rms_norm_eps),
                mixer=MIXERS.build("toy_decay", prefix=p + "mixer.", hidden_size=cfg.hidden_size, decay=cfg.decay),
                ff_norm=NORMS.build("rms_norm", name=p + "norm2.weight", hidden_size=cfg.hidden_size, eps=cfg.rms_norm_eps),
                feed_forward=FEED_FORWARDS.build("gated_silu", prefix=p + "mlp.", hidden_size=cfg.hidden_size,
                                                 intermediate_size=cfg.intermediate_size),
                residual_scale=0.5))
        emb = TokenEmbedding("embed.weight", cfg.vocab_size, cfg.hidden_size, 1.0)
        head = LMHead("head.weight", cfg.vocab_size, cfg.hidden_size, 1.0, tied_to=emb)
        norm = NORMS.build("rms_norm", name="norm.weight", hidden_size=cfg.hidden_size, eps=cfg.rms_norm_eps)
        # layer 0 runs twice (second run with a cache entry of its own), then layer 1
        schedule = [Run(0, 0), Run(0, 1), Run(1, 2)] if cfg.num_hidden_layers == 2 else None
        return DecoderModel(cfg, emb, layers, norm, head, schedule)

    register_architecture(Architecture("ToyDecayForCausalLM", ToyConfig, build), replace=True)
    return ToyConfig


def plain_toy(raw, w, toks):
    """The same model, whole sequence, in float64 on the CPU."""
    import torch.nn.functional as F
    W = {k: v.double() for k, v in w.items()}
    x = W["embed.weight"][torch.tensor(toks)]
    eps, decay = raw["rms_norm_eps"], raw["decay"]

    def layer(x, i):
        p = f"layers.{i}."
        a = F.rms_norm(x, (x.shape[-1],), W[p + "norm1.weight"], eps)
        s = torch.zeros_like(a[0])
        hs = []
        for t in range(a.shape[0]):
            s = decay * s + a[t]
            hs.append(s)
        x = x + 0.5 * (torch.stack(hs) @ W[p + "mixer.proj.weight"].T)
        f = F.rms_norm(x, (x.shape[-1],), W[p + "norm2.weight"], eps)
        return x + 0.5 * ((F.silu(f @ W[p + "mlp.gate_proj.weight"].T) * (f @ W[p + "mlp.up_proj.weight"].T))
                          @ W[p + "mlp.down_proj.weight"].T)
    for i in (0, 0, 1):
        x = layer(x, i)
    return F.rms_norm(x, (x.shape[-1],), W["norm.weight"], eps) @ W["embed.weight"].T


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_mixer_registers_builds_and_steps(tmp_path, dtype):
    from safetensors.torch import load_file
    from cpmcu_amd import Engine, EngineOptions, StepEntry
    from cpmcu_amd.registry import unregister_architecture
    from cpmcu_amd.parts import MIXERS
    from cpmcu_amd.weights import write_model_dir
    ToyConfig = _define()
    try:
        raw = {"architectures": ["ToyDecayForCausalLM"], "vocab_size": 90, "hidden_size": 40, "num_hidden_layers": 2,
               "intermediate_size": 56, "decay": 0.6, "rms_norm_eps": 1e-5, "max_position_embeddings": 64}
        write_model_dir(ToyConfig.from_dict(raw), str(tmp_path), seed=4, std=0.1, norm_std=0.1)
        w = load_file(str(tmp_path / "model.safetensors"))
        # hip_graph is asked for (the command line's default); the mixer says that it cannot be captured, and
        # the engine then runs every step eagerly
        eng = Engine.from_dir(str(tmp_path), EngineOptions(dtype=dtype, max_tokens=256, max_slots=2, hip_graph=True))
        assert not eng.graph_capturable and not eng.uses_graph
        assert len(eng.cache.groups) == 1 and eng.model.n_cache_entries == 3
        assert eng.cache.view(1).state["h"].shape == (2, 40) and not eng.cache.view(1).streams
        toks = [int(t) for t in torch.randint(0, 90, (23,), generator=torch.Generator().manual_seed(0))]
        ref = plain_toy(raw, w, toks).float()
        tol = 2e-5 if dtype == "float32" else 0.03 * float(ref.abs().max())
        s = eng.acquire()
        whole = eng.step([StepEntry(s, toks, list(range(23)))]).cpu()
        eng.release(s)
        assert float((whole - ref).abs().max()) < tol
        # token by token in the slot just given back: the state must have been zeroed
        s2 = eng.acquire()
        assert s2 == s
        outs = [eng.step([StepEntry(s2, toks[:5], list(range(5)))]).cpu()]
        other = eng.acquire()
        for i in range(5, 23):                                 # another sequence shares the steps
            lg = eng.step([StepEntry(s2, [toks[i]], [0]), StepEntry(other, [toks[i - 5]], [0])]).cpu()
            outs.append(lg[:1])
            assert float((lg[1] - ref[i - 5]).abs().max()) < tol
        assert float((torch.cat(outs) - ref).abs().max()) < tol
        assert not eng._graphs
        eng.release(s2)
        eng.release(other)
        eng.cache.check()
        # a forward pass that fails after the mixer advanced its state: the state is put back, and the same
        # tokens then give the logits of a first try
        s3 = eng.acquire()
        eng.step([StepEntry(s3, toks[:9], [])])
        real = eng.model.final_norm.forward
        for bring in (toks[9:15], toks[9:10]):                  # a pass of several tokens, a single-token step
            eng.model.final_norm.forward = lambda *a, **k: (_ for _ in ()).throw(RuntimeError("kernel refused"))
            try:
                with pytest.raises(RuntimeError, match="kernel refused"):
                    eng.step([StepEntry(s3, bring, [0])])
            finally:
                eng.model.final_norm.forward = real
            assert eng.length(s3) == 9
        got = eng.step([StepEntry(s3, toks[9:], list(range(14)))]).cpu()
        assert float((got - ref[9:]).abs().max()) < tol
        eng.release(s3)
    finally:
        unregister_architecture("ToyDecayForCausalLM")
        MIXERS.unregister("toy_decay")
