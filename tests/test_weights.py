"""Weights: reading by name, dtype rules, the one error that lists every difference (CPU)."""
import json
import os

import pytest
import torch
from safetensors.torch import load_file, save_file

import cpmcu_amd
from cpmcu_amd.config import MiniCPMConfig
from cpmcu_amd.models import minicpm
from cpmcu_amd.weights import WeightError, load_tensors, write_model_dir

import tiny


def _specs(raw, tied=None):
    cfg = MiniCPMConfig.from_dict(raw)
    return cfg, minicpm.build(cfg, tied=tied).all_weight_specs()


def _load(d, raw, tied=None):
    cfg, specs = _specs(raw, tied)
    return load_tensors(d, specs, split_fused=lambda n, t: minicpm.split_fused(cfg, n, t),
                        ignore=lambda n: minicpm.ignore_tensor(cfg, n))


def test_random_weights_folder_round_trip(tmp_path):
    raw = tiny.tiny_b()
    cfg = MiniCPMConfig.from_dict(raw)
    write_model_dir(cfg, str(tmp_path), seed=5, norm_std=0.1)
    assert sorted(os.listdir(tmp_path)) == ["config.json", "model.safetensors"]
    with open(tmp_path / "config.json") as f:
        assert MiniCPMConfig.from_dict(json.load(f)) == cfg
    t = _load(str(tmp_path), raw)
    assert t["model.embed_tokens.weight"].shape == (1000, 96) and t["model.embed_tokens.weight"].dtype == torch.bfloat16
    assert t["lm_head.weight"].shape == (1000, 96)
    w = t["model.layers.1.mlp.gate_proj.weight"].float()
    assert abs(w.std().item() - 0.02) < 0.002 and abs(w.mean().item()) < 0.001
    n = t["model.layers.0.input_layernorm.weight"].float()
    assert abs(n.mean().item() - 1.0) < 0.05 and 0.05 < n.std().item() < 0.15
    # same seed and name -> same values; another seed -> others
    again = tmp_path / "again"
    write_model_dir(cfg, str(again), seed=5, norm_std=0.1)
    other = tmp_path / "other"
    write_model_dir(cfg, str(other), seed=6, norm_std=0.1)
    a, b = load_file(str(again / "model.safetensors")), load_file(str(other / "model.safetensors"))
    assert all(torch.equal(a[k], load_file(str(tmp_path / "model.safetensors"))[k]) for k in a)
    assert not torch.equal(a["model.norm.weight"], b["model.norm.weight"])


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    raw = tiny.tiny_a()
    write_model_dir(MiniCPMConfig.from_dict(raw), str(tmp_path), seed=1)
    path = str(tmp_path / "model.safetensors")
    t = load_file(path)
    del t["model.layers.1.self_attn.o_proj.weight"]
    del t["model.norm.weight"]
    t["model.layers.0.mlp.up_proj.weight"] = torch.zeros(161, 64, dtype=torch.bfloat16)
    t["model.layers.0.extra.weight"] = torch.zeros(3)
    save_file(t, path)
    with pytest.raises(WeightError) as ei:
        _load(str(tmp_path), raw)
    e = ei.value
    assert e.missing == ["model.layers.1.self_attn.o_proj.weight", "model.norm.weight"]
    assert e.unexpected == ["model.layers.0.extra.weight"]
    assert [w[0] for w in e.wrong_shape] == ["model.layers.0.mlp.up_proj.weight"]
    msg = str(e)
    for needle in ("missing tensors (2)", "model.norm.weight", "unexpected tensors (1)", "model.layers.0.extra.weight",
                   "wrong shapes (1)", "[161, 64]", "[160, 64]"):
        assert needle in msg


def test_stored_dtypes_are_kept(tmp_path):
    raw = tiny.tiny_a()
    write_model_dir(MiniCPMConfig.from_dict(raw), str(tmp_path), seed=1)
    path = str(tmp_path / "model.safetensors")
    t = load_file(path)
    t["model.norm.weight"] = t["model.norm.weight"].float() + 1e-4        # a 32-bit tensor stays 32-bit
    t["model.layers.0.mlp.down_proj.weight"] = t["model.layers.0.mlp.down_proj.weight"].half()
    t["model.rotary_emb.inv_freq"] = torch.ones(8)                          # computed by the engine: ignored
    save_file(t, path)
    out = _load(str(tmp_path), raw)
    assert out["model.norm.weight"].dtype == torch.float32
    assert torch.equal(out["model.norm.weight"], t["model.norm.weight"])
    assert out["model.layers.0.mlp.down_proj.weight"].dtype == torch.bfloat16
    assert out["model.embed_tokens.weight"].dtype == torch.bfloat16
    assert "model.rotary_emb.inv_freq" not in out
    from cpmcu_amd.weights import stored_dtype
    assert stored_dtype(torch.int64) == torch.int32 and stored_dtype(torch.uint8) == torch.int32


def test_fused_spellings_are_split(tmp_path):
    raw = tiny.tiny_b()
    write_model_dir(MiniCPMConfig.from_dict(raw), str(tmp_path), seed=9)
    path = str(tmp_path / "model.safetensors")
    t = load_file(path)
    ref = dict(t)
    for i in range(3):
        p = f"model.layers.{i}."
        t[p + "self_attn.qkv_proj.weight"] = torch.cat([t.pop(p + f"self_attn.{n}_proj.weight") for n in "qkv"])
        t[p + "mlp.gate_up_proj.weight"] = torch.cat([t.pop(p + "mlp.gate_proj.weight"), t.pop(p + "mlp.up_proj.weight")])
    save_file(t, path)
    out = _load(str(tmp_path), raw)
    assert set(out) == set(ref) and all(torch.equal(out[k], ref[k]) for k in ref)


def test_file_discovery(tmp_path):
    raw = tiny.tiny_a()
    with pytest.raises(WeightError, match="no \\*.safetensors"):
        _load(str(tmp_path), raw)
    write_model_dir(MiniCPMConfig.from_dict(raw), str(tmp_path), seed=1)
    t = load_file(str(tmp_path / "model.safetensors"))
    save_file(t, str(tmp_path / "second.safetensors"))
    with pytest.raises(WeightError, match="several"):
        _load(str(tmp_path), raw)
    # an index names the shards: two shards, each half of the tensors
    os.remove(tmp_path / "second.safetensors")
    os.remove(tmp_path / "model.safetensors")
    names = sorted(t)
    half = len(names) // 2
    save_file({k: t[k] for k in names[:half]}, str(tmp_path / "model-00001-of-00002.safetensors"))
    save_file({k: t[k] for k in names[half:]}, str(tmp_path / "model-00002-of-00002.safetensors"))
    wm = {k: "model-00001-of-00002.safetensors" for k in names[:half]}
    wm.update({k: "model-00002-of-00002.safetensors" for k in names[half:]})
    with open(tmp_path / "model.safetensors.index.json", "w") as f:
        json.dump({"weight_map": wm}, f)
    out = _load(str(tmp_path), raw)
    assert all(torch.equal(out[k], t[k]) for k in t)


def test_tying_follows_the_checkpoint_when_the_config_is_silent(tmp_path):
    raw = tiny.tiny_b()
    raw.pop("tie_word_embeddings")
    cfg = MiniCPMConfig.from_dict(raw)
    assert cfg.tie_word_embeddings is None
    assert minicpm.build(cfg, tied=True).head.tied_to is not None
    assert minicpm.build(cfg, tied=False).head.tied_to is None


def test_a_part_brings_its_own_init_rule():
    """Another kind of tensor (here: decay rates in (0, 1)) registers its rule; the writer needs no change."""
    from cpmcu_amd.parts.base import WeightSpec
    from cpmcu_amd.weights import INIT_RULES, draw, register_init_rule

    def decay(spec, g, device, dtype, std, norm_std):
        return torch.rand(spec.shape, generator=g, device=device).to(dtype)

    register_init_rule("test_decay", decay)
    try:
        spec = WeightSpec("layer.decay", (7,), "test_decay", "float32")
        a, b = draw(spec, 3), draw(spec, 3)
        assert torch.equal(a, b) and a.dtype == torch.float32 and bool(((a >= 0) & (a < 1)).all())
        assert not torch.equal(a, draw(spec, 4))
        with pytest.raises(ValueError, match="already registered"):
            register_init_rule("test_decay", lambda *a: None)
    finally:
        INIT_RULES.pop("test_decay", None)
    with pytest.raises(ValueError, match="unknown init rule 'test_decay'.*matrix"):
        draw(WeightSpec("layer.decay", (7,), "test_decay", "float32"), 3)
