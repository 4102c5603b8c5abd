"""MiniCPM4 (``MiniCPMForCausalLM``): which parts, with which numbers.

Pre-norm decoder with muP scaling (cpmcu/llm.py:67-69): embeddings times
scale_emb, residual branches times scale_depth/sqrt(L), final hidden times
dim_model_base/hidden before the head; GQA attention with LongRoPE, InfLLM-v2
block-sparse attention when sparse_config is given; SiLU-gated feed-forward;
RMSNorm.  Checkpoint names are the HF ones (src/model/model.cuh:122-143,
src/model/minicpm4/minicpm4_attn.cuh:79-95, src/model/ffn.cuh:61-75); fused
``qkv_proj`` / ``gate_up_proj`` tensors are split as cpmcu/llm.py:125-131 does.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Tuple

import torch

from ..config.minicpm import MiniCPMConfig
from ..parts import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS, LMHead, PartSpec, TokenEmbedding)
from ..registry import Architecture, Flag, register_architecture
from .decoder import DecoderModel

ARCHITECTURE = "MiniCPMForCausalLM"


def layer_specs(cfg: MiniCPMConfig, sparse: bool = True) -> List[Dict[str, PartSpec]]:
    """The parts of every layer, chosen layer by layer from the configuration."""
    if cfg.rope_scaling is not None:
        rs = cfg.rope_scaling
        position = PartSpec.of("longrope", head_dim=cfg.head_dim, theta=cfg.rope_theta,
                               short_factor=rs.short_factor, long_factor=rs.long_factor,
                               original_max_position=rs.original_max_position_embeddings,
                               max_position=cfg.max_position_embeddings,
                               attention_scaling=cfg.rope_attention_scaling)
    else:
        position = PartSpec.of("rope", head_dim=cfg.head_dim, theta=cfg.rope_theta)
    specs = []
    for i in range(cfg.num_hidden_layers):
        p = f"model.layers.{i}."
        attn = dict(prefix=p + "self_attn.", hidden_size=cfg.hidden_size, num_heads=cfg.num_attention_heads,
                    num_kv_heads=cfg.num_key_value_heads, head_dim=cfg.head_dim)
        if cfg.sparse_config is not None and sparse:
            mixer = PartSpec.of("infllm_v2_attention", **attn, **cfg.sparse_config.to_dict())
        else:
            mixer = PartSpec.of("gqa_attention", **attn)
        specs.append({
            "position": position,
            "mixer_norm": PartSpec.of("rms_norm", name=p + "input_layernorm.weight", hidden_size=cfg.hidden_size,
                                      eps=cfg.rms_norm_eps),
            "mixer": mixer,
            "ff_norm": PartSpec.of("rms_norm", name=p + "post_attention_layernorm.weight",
                                   hidden_size=cfg.hidden_size, eps=cfg.rms_norm_eps),
            "feed_forward": PartSpec.of("gated_silu", prefix=p + "mlp.", hidden_size=cfg.hidden_size,
                                        intermediate_size=cfg.intermediate_size),
            "block": PartSpec.of("pre_norm", residual_scale=cfg.residual_scale),
        })
    return specs


def build(cfg: MiniCPMConfig, tied: Optional[bool] = None, sparse: bool = True) -> DecoderModel:
    tie = cfg.tie_word_embeddings if cfg.tie_word_embeddings is not None else bool(tied)
    layers = []
    for s in layer_specs(cfg, sparse):
        position = s["position"].build(POSITION_ENCODINGS)
        layers.append(s["block"].build(
            BLOCKS,
            mixer_norm=s["mixer_norm"].build(NORMS),
            mixer=s["mixer"].build(MIXERS, position=position),
            ff_norm=s["ff_norm"].build(NORMS),
            feed_forward=s["feed_forward"].build(FEED_FORWARDS)))
    embedding = TokenEmbedding("model.embed_tokens.weight", cfg.vocab_size, cfg.hidden_size, cfg.scale_emb)
    head = LMHead("lm_head.weight", cfg.vocab_size, cfg.hidden_size, cfg.head_scale, tied_to=embedding if tie else None)
    final_norm = NORMS.build("rms_norm", name="model.norm.weight", hidden_size=cfg.hidden_size, eps=cfg.rms_norm_eps)
    return DecoderModel(cfg, embedding, layers, final_norm, head)


def split_fused(cfg: MiniCPMConfig, name: str, tensor: torch.Tensor) -> Optional[List[Tuple[str, torch.Tensor]]]:
    """Checkpoints may hold q,k,v or gate,up as one tensor stacked on the output axis (cpmcu/llm.py:125-131)."""
    if "gate_up_proj" in name:
        half = tensor.shape[0] // 2
        return [(name.replace("gate_up_proj", "gate_proj"), tensor[:half]),
                (name.replace("gate_up_proj", "up_proj"), tensor[half:])]
    if "qkv_proj" in name:
        q = cfg.num_attention_heads * cfg.head_dim
        kv = cfg.num_key_value_heads * cfg.head_dim
        return [(name.replace("qkv_proj", "q_proj"), tensor[:q]),
                (name.replace("qkv_proj", "k_proj"), tensor[q:q + kv]),
                (name.replace("qkv_proj", "v_proj"), tensor[q + kv:])]
    return None


def ignore_tensor(cfg: MiniCPMConfig, name: str) -> bool:
    """Tensors a checkpoint may carry that the engine computes itself."""
    return "rotary_emb.inv_freq" in name


def checkpoint_options(cfg: MiniCPMConfig, names) -> Dict[str, object]:
    """Embeddings are tied when config.json is silent and the checkpoint holds no head (cpmcu/llm.py:136-137)."""
    return {"tied": "lm_head.weight" not in names}


def apply_flags(cfg: MiniCPMConfig, flags: Dict[str, object]) -> Tuple[MiniCPMConfig, Dict[str, object]]:
    """The reference's front-end flags for this architecture (cpmcu/common/args.py:38-40, 72-83,
    cpmcu/llm.py:31-36): ``apply_sparse`` switches InfLLM-v2 on, the sparse flags override single values of
    config.json's sparse_config, ``minicpm4_yarn`` installs the built-in LongRoPE factors
    (cpmcu/common/utils.py:181-207)."""
    import dataclasses

    from ..config.minicpm import RopeScaling, SparseConfig
    known = {"apply_sparse", "sink_window_size", "block_window_size", "sparse_topk_k", "sparse_switch",
             "use_compress_lse", "minicpm4_yarn"}
    unknown = sorted(set(flags) - known)
    if unknown:
        raise ValueError(f"{ARCHITECTURE} does not know the flags {unknown} (it knows: {sorted(known)})")
    if flags.get("use_compress_lse"):
        raise ValueError("use_compress_lse is not supported: block scores are normalised over the compressed "
                         "keys they are computed from")
    options: Dict[str, object] = {}
    if "apply_sparse" in flags:
        options["sparse"] = bool(flags["apply_sparse"])
    sc = cfg.sparse_config
    # absent (the command line's model type 'auto'): block-sparse attention is on iff config.json describes it
    sparse_on = bool(flags["apply_sparse"]) if "apply_sparse" in flags else sc is not None
    if flags.get("apply_sparse") and sc is None:
        raise ValueError("apply_sparse: config.json has no sparse_config (kernel_size, kernel_stride, block_size ...)")
    over_flags = [k for k in ("sink_window_size", "block_window_size", "sparse_topk_k", "sparse_switch") if k in flags]
    if over_flags and not sparse_on:
        raise ValueError(f"{over_flags} change the block-sparse attention, which is off: "
                         + ("apply_sparse is false" if sc is not None else "config.json has no sparse_config"))
    if over_flags:
        over = {}
        if "sink_window_size" in flags:
            over["init_blocks"] = flags["sink_window_size"]
        if "block_window_size" in flags:
            over["window_size"] = flags["block_window_size"] * sc.block_size
        if "sparse_topk_k" in flags:
            over["topk"] = flags["sparse_topk_k"]
        if "sparse_switch" in flags:
            over["dense_len"] = flags["sparse_switch"]
        cfg = dataclasses.replace(cfg, sparse_config=SparseConfig.from_dict({**sc.to_dict(), **over}))
    if flags.get("minicpm4_yarn"):
        from ..config.minicpm4_yarn import MINICPM4_YARN_FACTORS
        if cfg.head_dim != 2 * len(MINICPM4_YARN_FACTORS):
            raise ValueError(f"minicpm4_yarn holds factors for head_dim {2 * len(MINICPM4_YARN_FACTORS)}, "
                             f"the model has {cfg.head_dim}")
        rs = cfg.rope_scaling
        orig = rs.original_max_position_embeddings if rs else cfg.max_position_embeddings
        cfg = dataclasses.replace(cfg, rope_scaling=RopeScaling("longrope", MINICPM4_YARN_FACTORS,
                                                                MINICPM4_YARN_FACTORS, orig))
    return cfg, options


register_architecture(Architecture(
    name=ARCHITECTURE, config_class=MiniCPMConfig, build=build, options={"tied": None, "sparse": True},
    split_fused=split_fused, ignore_tensor=ignore_tensor, checkpoint_options=checkpoint_options,
    apply_flags=apply_flags,
    flags=(
        Flag("minicpm4_yarn", bool, "Replace the LongRoPE factors by the built-in long-context list (default: False)"),
        Flag("apply_sparse", bool, "Block-sparse attention on or off (default: on iff config.json has sparse_config)",
             "Sparse Attention"),
        Flag("sink_window_size", int, "Initial blocks always attended to (default: sparse_config.init_blocks)",
             "Sparse Attention"),
        Flag("block_window_size", int, "Trailing window in blocks (default: sparse_config.window_size / block_size)",
             "Sparse Attention"),
        Flag("sparse_topk_k", int, "Blocks chosen by score (default: sparse_config.topk)", "Sparse Attention"),
        Flag("sparse_switch", int, "Context up to which attention stays dense (default: sparse_config.dense_len)",
             "Sparse Attention"),
        Flag("use_compress_lse", bool, "Not supported (scores are normalised over the keys they come from); must "
             "stay False", "Sparse Attention")),
    # 'minicpm4' switches the block-sparse attention on, 'minicpm' off (cpmcu/common/utils.py:123)
    model_types={"minicpm4": {"apply_sparse": True}, "minicpm": {"apply_sparse": False}}))
