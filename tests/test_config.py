"""Configuration and registry (CPU)."""
import copy

import pytest

import cpmcu_amd
from cpmcu_amd.config import ConfigError, MiniCPMConfig
from cpmcu_amd.registry import get_architecture

import tiny


def test_reads_every_key_of_tiny_configs():
    a = MiniCPMConfig.from_dict(tiny.tiny_a())
    assert (a.num_hidden_layers, a.hidden_size, a.num_attention_heads, a.num_key_value_heads, a.head_dim) == (2, 64, 4, 2, 16)
    assert (a.intermediate_size, a.vocab_size, a.rms_norm_eps, a.rope_theta) == (160, 512, 1e-6, 10000.0)
    assert a.tie_word_embeddings is True and a.sparse_config is None and a.eos_token_ids == (2,)
    assert a.residual_scale == pytest.approx(1.4 / 2 ** 0.5) and a.head_scale == pytest.approx(32 / 64)
    b = MiniCPMConfig.from_dict(tiny.tiny_b())
    assert b.head_dim == 32 and b.num_key_value_heads == 1 and b.eos_token_ids == (1, 7)
    assert b.sparse_config.window_blocks == 2 and b.sparse_config.dense_len == 64
    assert b.rope_scaling.original_max_position_embeddings == 128 and len(b.rope_scaling.long_factor) == 16


def test_defaults_when_keys_are_absent():
    raw = tiny.tiny_a()
    for k in ("scale_emb", "dim_model_base", "scale_depth", "num_key_value_heads", "rope_scaling", "tie_word_embeddings",
              "eos_token_id", "rope_theta"):
        raw.pop(k)
    c = MiniCPMConfig.from_dict(raw)
    assert c.scale_emb == 1.0 and c.residual_scale == 1.0 and c.head_scale == 1.0
    assert c.num_key_value_heads == c.num_attention_heads and c.head_dim == 16
    assert c.rope_scaling is None and c.tie_word_embeddings is None and c.eos_token_ids == () and c.rope_theta == 10000.0


def test_round_trip_through_to_dict():
    for raw in (tiny.tiny_a(), tiny.tiny_b()):
        c = MiniCPMConfig.from_dict(raw)
        assert MiniCPMConfig.from_dict(c.to_dict()) == c


@pytest.mark.parametrize("change,needle", [
    ({"num_key_value_heads": 3}, "multiple of num_key_value_heads"),
    ({"hidden_act": "gelu"}, "hidden_act"),
    ({"attention_bias": True}, "attention_bias"),
    ({"vocab_size": "many"}, "vocab_size"),
    ({"rms_norm_eps": None}, "rms_norm_eps"),
    ({"head_dim": 15}, "head_dim"),
    ({"eos_token_id": 99999}, "outside the vocabulary"),
])
def test_bad_values_are_refused(change, needle):
    raw = tiny.tiny_a()
    raw.update(change)
    with pytest.raises(ConfigError, match=needle):
        MiniCPMConfig.from_dict(raw)


def test_factor_list_of_wrong_length():
    raw = tiny.tiny_a()
    raw["rope_scaling"]["long_factor"] = [1.0] * 7
    with pytest.raises(ConfigError, match="long_factor.*7 entries.*8"):
        MiniCPMConfig.from_dict(raw)
    raw = tiny.tiny_a()
    raw["rope_scaling"]["rope_type"] = "yarn"
    with pytest.raises(ConfigError, match="yarn"):
        MiniCPMConfig.from_dict(raw)


@pytest.mark.parametrize("change,needle", [
    ({"block_size": 18}, "multiple of kernel_stride"),
    ({"kernel_size": 2}, "kernel_size"),
    ({"window_size": 40}, "window_size"),
    ({"init_blocks": 9}, "init_blocks"),
])
def test_sparse_config_is_validated(change, needle):
    raw = tiny.tiny_b()
    raw["sparse_config"].update(change)
    with pytest.raises(ConfigError, match=needle):
        MiniCPMConfig.from_dict(raw)


def test_registry_names_what_it_knows():
    assert "MiniCPMForCausalLM" in cpmcu_amd.architectures()
    with pytest.raises(KeyError, match="MiniCPMForCausalLM"):
        get_architecture("NoSuchModelForCausalLM")


def test_model_is_built_from_the_configuration_layer_by_layer():
    from cpmcu_amd.parts import GQAAttention, InfLLMv2Attention
    a = get_architecture("MiniCPMForCausalLM").build(MiniCPMConfig.from_dict(tiny.tiny_a()))
    b = get_architecture("MiniCPMForCausalLM").build(MiniCPMConfig.from_dict(tiny.tiny_b()))
    assert len(a.layers) == 2 and len(b.layers) == 3
    assert all(type(l.mixer) is GQAAttention for l in a.layers)
    assert all(type(l.mixer) is InfLLMv2Attention for l in b.layers)
    assert b.layers[0].mixer.bs == 16 and b.layers[0].mixer.window_blocks == 2
    assert a.head.tied_to is a.embedding and b.head.tied_to is None
    names = {s.name for s in b.all_weight_specs()}
    assert "lm_head.weight" in names and "model.layers.2.mlp.down_proj.weight" in names
    assert "lm_head.weight" not in {s.name for s in a.all_weight_specs()}
    # sparse attention can be switched off without touching the configuration
    d = get_architecture("MiniCPMForCausalLM").build(MiniCPMConfig.from_dict(tiny.tiny_b()), sparse=False)
    assert all(type(l.mixer) is GQAAttention for l in d.layers)


def test_options_are_declared_by_the_architecture():
    arch = get_architecture("MiniCPMForCausalLM")
    cfg = MiniCPMConfig.from_dict(tiny.tiny_b())
    from cpmcu_amd.parts import GQAAttention
    assert set(arch.options) == {"tied", "sparse"}
    dense = arch.build_model(cfg, {"sparse": False})
    assert all(type(l.mixer) is GQAAttention for l in dense.layers)
    with pytest.raises(ValueError, match="no option 'window'.*sparse"):
        arch.build_model(cfg, {"window": 3})
    # what the checkpoint decides (no head tensor: tied) yields to an explicit option
    raw = tiny.tiny_b()
    del raw["tie_word_embeddings"]
    cfg2 = MiniCPMConfig.from_dict(raw)
    assert arch.build_model(cfg2, None, ["model.embed_tokens.weight"]).head.tied_to is not None
    assert arch.build_model(cfg2, None, ["model.embed_tokens.weight", "lm_head.weight"]).head.tied_to is None
    assert arch.build_model(cfg2, {"tied": False}, ["model.embed_tokens.weight"]).head.tied_to is None


def test_head_sizes_the_kernels_do_not_take_are_refused_when_the_model_is_built():
    raw = tiny.tiny_a()
    raw["head_dim"] = 24
    raw["rope_scaling"]["short_factor"] = raw["rope_scaling"]["short_factor"][:4] * 3
    raw["rope_scaling"]["long_factor"] = raw["rope_scaling"]["long_factor"][:4] * 3
    cfg = MiniCPMConfig.from_dict(raw)              # a valid configuration of the architecture
    with pytest.raises(ValueError, match="head_dim 24.*steps of 16"):
        get_architecture("MiniCPMForCausalLM").build_model(cfg)


def test_front_end_flags_go_through_the_architecture():
    arch = get_architecture("MiniCPMForCausalLM")
    cfg = MiniCPMConfig.from_dict(tiny.tiny_b())
    same, opts = arch.with_flags(cfg, {"apply_sparse": False})
    assert same == cfg and opts == {"sparse": False}
    with pytest.raises(ValueError, match="sparse_topk_k.*apply_sparse is false"):
        arch.with_flags(cfg, {"apply_sparse": False, "sparse_topk_k": 9})
    with pytest.raises(ValueError, match="sparse_switch.*no sparse_config"):
        arch.with_flags(MiniCPMConfig.from_dict(tiny.tiny_a()), {"sparse_switch": 9})
    new, opts = arch.with_flags(cfg, {"apply_sparse": True, "sparse_topk_k": 9, "block_window_size": 3, "sink_window_size": 2,
                                      "sparse_switch": 100})
    sc = new.sparse_config
    assert opts == {"sparse": True} and (sc.topk, sc.window_size, sc.init_blocks, sc.dense_len) == (9, 48, 2, 100)
    # the command line's model type 'auto' gives no apply_sparse at all: the configuration decides, and the
    # overrides still arrive
    new, opts = arch.with_flags(cfg, {"apply_sparse": None, "sparse_topk_k": 3, "sparse_switch": 5})
    assert opts == {} and (new.sparse_config.topk, new.sparse_config.dense_len) == (3, 5)
    assert new.sparse_config.window_size == cfg.sparse_config.window_size
    with pytest.raises(ValueError, match="use_compress_lse"):
        arch.with_flags(cfg, {"use_compress_lse": True})
    with pytest.raises(ValueError, match="no sparse_config"):
        arch.with_flags(MiniCPMConfig.from_dict(tiny.tiny_a()), {"apply_sparse": True})
    with pytest.raises(ValueError, match="does not know the flags"):
        arch.with_flags(cfg, {"draft_model": "x"})


def test_minicpm4_yarn_installs_the_built_in_factors_for_head_size_128_only():
    """--minicpm4-yarn overwrites both factor lists with the reference's 64 numbers
    (cpmcu/common/utils.py:181-207): only a head size of 128 has 64 rotation pairs."""
    from cpmcu_amd.config.minicpm4_yarn import MINICPM4_YARN_FACTORS
    arch = get_architecture("MiniCPMForCausalLM")
    assert len(MINICPM4_YARN_FACTORS) == 64 and MINICPM4_YARN_FACTORS[0] < 1.0 < MINICPM4_YARN_FACTORS[-1]
    with pytest.raises(ValueError, match="head_dim 128"):
        arch.with_flags(MiniCPMConfig.from_dict(tiny.tiny_b()), {"minicpm4_yarn": True})
    raw = tiny.tiny_b()
    raw.update(hidden_size=384, num_attention_heads=3, head_dim=128)
    raw["rope_scaling"].update(short_factor=[1.5] * 64, long_factor=[2.5] * 64)
    cfg = MiniCPMConfig.from_dict(raw)
    new, opts = arch.with_flags(cfg, {"minicpm4_yarn": True})
    assert opts == {}
    rs = new.rope_scaling
    assert rs.short_factor == tuple(MINICPM4_YARN_FACTORS) == rs.long_factor
    assert rs.original_max_position_embeddings == cfg.rope_scaling.original_max_position_embeddings
    # and they reach the position encoding of every layer, whichever list the engine's length selects
    model = arch.build_model(new)
    for layer in model.layers:
        for max_len in (64, 4096):
            assert tuple(layer.mixer.position.factors(max_len)) == tuple(MINICPM4_YARN_FACTORS)


def test_neutral_properties_of_a_configuration():
    cfg = MiniCPMConfig.from_dict(tiny.tiny_b())
    assert cfg.vocabulary_size == 1000 and cfg.longest_sequence == 512 and tuple(cfg.stop_token_ids) == (1, 7)


def test_share_and_slice_heuristics_stay_within_what_the_kernels_take():
    """The host-side choices of split-KV shares and K slices: at most 32 shares of at least 128 keys, about one
    workgroup a CU; slices of whole 128-column blocks that cover K."""
    from cpmcu_amd import ops
    for n in (1, 2, 3, 8, 16, 24, 64, 200, 257):
        for nkv, group in ((1, 4), (2, 16), (8, 5), (2, 40)):
            for keys in (1, 100, 128, 700, 4096, 8192, 33000, 140000):
                s = ops.attention_splits(n, nkv, group, keys)
                assert 1 <= s <= 32
                assert s == 1 or keys // s >= 128
                groups = n * nkv * -(-group // 16)
                assert s == 1 or s * groups <= 256 or (groups >= 128 and s == 2)
    for M in (1, 16, 17, 32, 33, 64):
        for N, K in ((4096, 4096), (4608, 4096), (4096, 16384), (100, 104), (73448, 4096), (1024, 896)):
            S = ops.skinny_split(M, N, K)
            assert S >= 1
            if S > 1:
                ks = -(-(-(-K // S)) // 128) * 128
                assert -(-K // ks) == S and ks >= 512
                assert M <= 16 or -(-N // 64) * S <= 256


def test_model_type_auto_keeps_the_sparse_overrides(model_dirs):
    """The command line's default model type gives no apply_sparse; the sparse options it does give must still
    reach the configuration of a model whose config.json describes the block-sparse attention."""
    from cpmcu_amd.args import parse_cli_args
    from cpmcu_amd.llm import LLM
    args = parse_cli_args(["--model-path", model_dirs["B"], "--sparse-topk-k", "3", "--sparse_switch", "5"])
    assert args.model_type == "auto" and args.apply_sparse is None and args.sparse_topk_k == 3
    arch = get_architecture("MiniCPMForCausalLM")
    flags = {f.name: getattr(args, f.name) for f in arch.flags}
    llm = LLM(model_dirs["B"], **flags)
    assert (llm.config.sparse_config.topk, llm.config.sparse_config.dense_len) == (3, 5)
    assert llm.model_options == {}
    assert type(arch.build_model(llm.config, llm.model_options).layers[0].mixer).__name__ == "InfLLMv2Attention"
    # a model without sparse_config refuses them instead of dropping them
    with pytest.raises(ValueError, match="no sparse_config"):
        LLM(model_dirs["A"], sparse_topk_k=3)
    # a float16 checkpoint is served in bfloat16 unless a dtype is asked for; float16 itself is refused
    assert LLM(model_dirs["A"]).dtype == "bfloat16"
    with pytest.raises(ValueError, match="float16"):
        LLM(model_dirs["A"], dtype="float16")


def test_an_architecture_brings_its_own_front_end_flags(tmp_path):
    """Nothing in args.py, cli.py or llm.py spells a model flag: an architecture registered here declares one and
    a model type, and the parser, the command line's flag hand-over and ``LLM`` know them."""
    import json
    from dataclasses import dataclass, replace

    from cpmcu_amd.args import create_cli_parser
    from cpmcu_amd.config.base import ModelConfig
    from cpmcu_amd.llm import LLM
    from cpmcu_amd.registry import Architecture, Flag, register_architecture, unregister_architecture

    @dataclass(frozen=True)
    class FlagToyConfig(ModelConfig):
        depth: int = 1

        @classmethod
        def from_dict(cls, raw):
            return cls("FlagToyForTests", depth=int(raw.get("depth", 1)))

        def to_dict(self):
            return {"architectures": [self.architecture], "depth": self.depth}

        vocabulary_size = 10

    def apply_flags(cfg, flags):
        assert set(flags) <= {"toy_depth", "toy_fast"}
        if "toy_depth" in flags:
            cfg = replace(cfg, depth=flags["toy_depth"])
        return cfg, ({"fast": flags["toy_fast"]} if "toy_fast" in flags else {})

    arch = Architecture("FlagToyForTests", FlagToyConfig, build=lambda cfg, fast=False: None, options={"fast": False},
                        apply_flags=apply_flags,
                        flags=(Flag("toy_depth", int, "layers to run", "Toy"), Flag("toy_fast", bool, "fast path", "Toy")),
                        model_types={"toyfast": {"toy_fast": True}})
    register_architecture(arch)
    try:
        p = create_cli_parser()
        a = p.parse_args(["--toy-depth", "3", "--model-type", "toyfast", "--toy_fast", "false"])
        assert a.toy_depth == 3 and a.toy_fast is False and a.model_type == "toyfast"
        assert a.sparse_topk_k is None                     # MiniCPM4's own are still there
        d = tmp_path / "m"
        d.mkdir()
        (d / "config.json").write_text(json.dumps({"architectures": ["FlagToyForTests"], "depth": 2}))
        llm = LLM(str(d), toy_depth=5, toy_fast=True)
        assert llm.config.depth == 5 and llm.model_options == {"fast": True}
        with pytest.raises(AssertionError):
            LLM(str(d), sparse_topk_k=2)                   # not this architecture's flag
    finally:
        unregister_architecture("FlagToyForTests")
    with pytest.raises(SystemExit):
        create_cli_parser().parse_args(["--toy-depth", "3"])


def test_the_package_description_names_every_subpackage_and_the_kernel_sources():
    """pyproject.toml installs the folder `cpm.cu_amd` as `cpmcu_amd`: every folder with an __init__.py is
    listed, the HIP sources are package data, and the scripts point at functions that exist."""
    import importlib
    import os
    import tomli
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    with open(os.path.join(root, "pyproject.toml"), "rb") as f:
        meta = tomli.load(f)
    tool = meta["tool"]["setuptools"]
    src = os.path.join(root, tool["package-dir"]["cpmcu_amd"])
    found = {"cpmcu_amd"} | {"cpmcu_amd." + d for d in os.listdir(src)
                             if os.path.isfile(os.path.join(src, d, "__init__.py"))}
    assert set(tool["packages"]) == found
    assert any(f.endswith(".hip") for f in os.listdir(os.path.join(src, "csrc")))
    assert tool["package-data"]["cpmcu_amd.csrc"] == ["*.hip", "*.h"]
    for target in meta["project"]["scripts"].values():
        module, func = target.split(":")
        assert callable(getattr(importlib.import_module(module), func))


def test_the_command_lines_model_type_and_flags_resolve_through_the_architecture(model_dirs):
    """--model-type names set what their architecture says unless an option says otherwise; names and options of
    another architecture are refused (cpmcu/common/utils.py:123: 'minicpm4' means block-sparse attention)."""
    from cpmcu_amd.args import parse_cli_args
    from cpmcu_amd.cli import resolve_model_flags
    from cpmcu_amd.llm import LLM
    arch = get_architecture("MiniCPMForCausalLM")
    flags = resolve_model_flags(parse_cli_args(["--model-type", "minicpm4", "--sparse-topk-k", "2"]), arch)
    assert flags["apply_sparse"] is True and flags["sparse_topk_k"] == 2 and flags["sink_window_size"] is None
    assert LLM(model_dirs["B"], **flags).config.sparse_config.topk == 2
    with pytest.raises(ValueError, match="no sparse_config"):
        LLM(model_dirs["A"], **flags)                            # 'minicpm4' on a model that describes no sparse attention
    flags = resolve_model_flags(parse_cli_args(["--model-type", "minicpm"]), arch)
    assert flags["apply_sparse"] is False
    llm = LLM(model_dirs["B"], **flags)
    assert llm.model_options == {"sparse": False}
    assert type(arch.build_model(llm.config, llm.model_options).layers[0].mixer).__name__ == "GQAAttention"
    # an explicit option wins over the model type's setting
    flags = resolve_model_flags(parse_cli_args(["--model-type", "minicpm", "--apply-sparse", "true"]), arch)
    assert flags["apply_sparse"] is True
    # an architecture without model types refuses a name, and options that are not its own
    from cpmcu_amd.registry import Architecture
    bare = Architecture("BareForTests", MiniCPMConfig, build=lambda cfg: None)
    with pytest.raises(ValueError, match="knows no model types"):
        resolve_model_flags(parse_cli_args(["--model-type", "minicpm4"]), bare)
    with pytest.raises(ValueError, match="has no flags \\['sparse_topk_k'\\]"):
        resolve_model_flags(parse_cli_args(["--sparse-topk-k", "2"]), bare)
    assert resolve_model_flags(parse_cli_args([]), bare) == {}
