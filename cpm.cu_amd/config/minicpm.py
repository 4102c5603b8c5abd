"""Typed configuration of MiniCPM4 (config.json of ``MiniCPMForCausalLM``).

The keys are those that OpenBMB/CPM.cu reads from the HF config
(cpmcu/llm.py:62-81, 136, 182-187), plus ``sparse_config`` (InfLLM-v2, which the
reference takes from command-line flags, cpmcu/common/args.py:72-83) and the
token ids that end a sequence.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Any, Dict, Optional, Tuple

from .base import ConfigError, ModelConfig, field_from, require


@dataclass(frozen=True)
class RopeScaling:
    """``rope_scaling`` of config.json: LongRoPE factor lists."""
    rope_type: str
    short_factor: Tuple[float, ...]
    long_factor: Tuple[float, ...]
    original_max_position_embeddings: int

    @classmethod
    def from_dict(cls, raw: Dict[str, Any], half_dim: int, max_position: int, top: Dict[str, Any]):
        where = "config.json rope_scaling"
        # the reference accepts both spellings of the kind (cpmcu/llm.py:183)
        kind = raw.get("rope_type", raw.get("type"))
        require(isinstance(kind, str), f"{where}: 'rope_type' (or 'type') must name the scaling")
        if kind != "longrope":
            raise ConfigError(f"{where}: rope_type '{kind}' is not supported (supported: longrope, or no rope_scaling)")

        def factors(key):
            v = raw.get(key)
            require(isinstance(v, list) and all(isinstance(f, (int, float)) and not isinstance(f, bool) for f in v),
                    f"{where}: '{key}' must be a list of numbers")
            require(len(v) == half_dim,
                    f"{where}: '{key}' has {len(v)} entries, head_dim/2 = {half_dim} are needed")
            require(all(f > 0 for f in v), f"{where}: '{key}' entries must be positive")
            return tuple(float(f) for f in v)

        orig = raw.get("original_max_position_embeddings", top.get("original_max_position_embeddings"))
        if orig is None:
            orig = max_position
        require(isinstance(orig, int) and not isinstance(orig, bool) and orig > 1,
                f"{where}: 'original_max_position_embeddings' must be an integer > 1")
        return cls(kind, factors("short_factor"), factors("long_factor"), int(orig))

    def to_dict(self):
        return {"rope_type": self.rope_type, "short_factor": list(self.short_factor),
                "long_factor": list(self.long_factor),
                "original_max_position_embeddings": self.original_max_position_embeddings}


@dataclass(frozen=True)
class SparseConfig:
    """``sparse_config`` of config.json: InfLLM-v2 block-sparse attention.

    The reference fixes kernel 32 / stride 16 / block 64 in code
    (src/model/minicpm4/minicpm4_kvcache.cuh:6-62, 156-178) and takes the rest
    from flags; here all of them are configuration."""
    kernel_size: int
    kernel_stride: int
    block_size: int
    init_blocks: int
    topk: int
    window_size: int
    dense_len: int

    @classmethod
    def from_dict(cls, raw: Dict[str, Any]):
        where = "config.json sparse_config"
        vals = {k: field_from(raw, k, int, where=where) for k in
                ("kernel_size", "kernel_stride", "block_size", "init_blocks", "topk", "window_size", "dense_len")}
        sc = cls(**vals)
        require(sc.kernel_stride > 0 and sc.kernel_size >= sc.kernel_stride,
                f"{where}: kernel_size ({sc.kernel_size}) must be >= kernel_stride ({sc.kernel_stride}) > 0")
        require(sc.block_size > 0 and sc.block_size % sc.kernel_stride == 0,
                f"{where}: block_size ({sc.block_size}) must be a multiple of kernel_stride ({sc.kernel_stride})")
        require(sc.window_size % sc.block_size == 0 and sc.window_size >= sc.block_size,
                f"{where}: window_size ({sc.window_size}) must be a positive multiple of block_size ({sc.block_size})")
        require(0 <= sc.init_blocks <= sc.topk, f"{where}: need 0 <= init_blocks ({sc.init_blocks}) <= topk ({sc.topk})")
        require(sc.dense_len >= 0, f"{where}: dense_len must be >= 0")
        return sc

    @property
    def window_blocks(self) -> int:
        return self.window_size // self.block_size

    def to_dict(self):
        return {k: getattr(self, k) for k in
                ("kernel_size", "kernel_stride", "block_size", "init_blocks", "topk", "window_size", "dense_len")}


@dataclass(frozen=True)
class MiniCPMConfig(ModelConfig):
    vocab_size: int
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    rms_norm_eps: float
    rope_theta: float
    max_position_embeddings: int
    rope_scaling: Optional[RopeScaling]
    rope_attention_scaling: bool
    scale_emb: float
    dim_model_base: Optional[float]
    scale_depth: Optional[float]
    tie_word_embeddings: Optional[bool]      # None: decided by the checkpoint (lm_head.weight present or not)
    sparse_config: Optional[SparseConfig]
    eos_token_ids: Tuple[int, ...] = ()
    bos_token_id: Optional[int] = None
    torch_dtype: Optional[str] = None

    # ---- derived scalars (the three muP factors, cpmcu/llm.py:67-69) ----
    @property
    def residual_scale(self) -> float:
        return 1.0 if self.scale_depth is None else self.scale_depth / math.sqrt(self.num_hidden_layers)

    @property
    def head_scale(self) -> float:
        return 1.0 if self.dim_model_base is None else self.dim_model_base / self.hidden_size

    @property
    def stop_token_ids(self):
        return self.eos_token_ids

    @property
    def vocabulary_size(self) -> int:
        return self.vocab_size

    @property
    def longest_sequence(self) -> Optional[int]:
        return self.max_position_embeddings

    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "MiniCPMConfig":
        arch = raw.get("architectures") or ["MiniCPMForCausalLM"]
        H = field_from(raw, "hidden_size", int)
        nh = field_from(raw, "num_attention_heads", int)
        require(H > 0 and nh > 0, "config.json: hidden_size and num_attention_heads must be positive")
        nkv = field_from(raw, "num_key_value_heads", int, nh)
        require(nkv > 0 and nh % nkv == 0,
                f"config.json: num_attention_heads ({nh}) must be a multiple of num_key_value_heads ({nkv})")
        if raw.get("head_dim") is None:
            require(H % nh == 0, f"config.json: hidden_size ({H}) is not a multiple of num_attention_heads ({nh}) "
                                 f"and no head_dim is given")
        hd = field_from(raw, "head_dim", int, H // nh)
        require(hd > 0 and hd % 2 == 0, f"config.json: head_dim ({hd}) must be even (rotate-half position encoding)")
        act = raw.get("hidden_act", "silu")
        require(act == "silu", f"config.json: hidden_act '{act}' is not supported (this architecture's feed-forward is SiLU-gated)")
        require(not raw.get("attention_bias", False), "config.json: attention_bias=true is not supported")
        max_pos = field_from(raw, "max_position_embeddings", int)
        require(max_pos > 0, "config.json: max_position_embeddings must be positive")
        rs_raw = raw.get("rope_scaling")
        rs = None
        if rs_raw is not None:
            require(isinstance(rs_raw, dict), "config.json: rope_scaling must be an object or null")
            kind = rs_raw.get("rope_type", rs_raw.get("type"))
            if kind not in (None, "default"):
                rs = RopeScaling.from_dict(rs_raw, hd // 2, max_pos, raw)
        sc_raw = raw.get("sparse_config")
        sc = None
        if sc_raw is not None:
            require(isinstance(sc_raw, dict), "config.json: sparse_config must be an object or null")
            sc = SparseConfig.from_dict(sc_raw)
        eos = raw.get("eos_token_id")
        if eos is None:
            eos_ids: Tuple[int, ...] = ()
        elif isinstance(eos, int) and not isinstance(eos, bool):
            eos_ids = (eos,)
        elif isinstance(eos, list) and all(isinstance(e, int) and not isinstance(e, bool) for e in eos):
            eos_ids = tuple(eos)
        else:
            raise ConfigError(f"config.json: eos_token_id must be an integer or a list of integers, got {eos!r}")
        V = field_from(raw, "vocab_size", int)
        L = field_from(raw, "num_hidden_layers", int)
        I = field_from(raw, "intermediate_size", int)
        require(V > 0 and L > 0 and I > 0, "config.json: vocab_size, num_hidden_layers, intermediate_size must be positive")
        require(all(0 <= e < V for e in eos_ids), f"config.json: eos_token_id {eos_ids} outside the vocabulary of {V}")
        eps = field_from(raw, "rms_norm_eps", float)
        require(eps >= 0, "config.json: rms_norm_eps must be >= 0")
        dmb = raw.get("dim_model_base")
        sd = raw.get("scale_depth")
        tie = raw.get("tie_word_embeddings")
        return cls(
            architecture=arch[0],
            vocab_size=V, hidden_size=H, num_hidden_layers=L,
            num_attention_heads=nh, num_key_value_heads=nkv, head_dim=hd,
            intermediate_size=I, rms_norm_eps=eps,
            rope_theta=field_from(raw, "rope_theta", float, 10000.0),
            max_position_embeddings=max_pos, rope_scaling=rs,
            rope_attention_scaling=field_from(raw, "rope_attention_scaling", bool, True),
            scale_emb=field_from(raw, "scale_emb", float, 1.0),
            dim_model_base=None if dmb is None else field_from(raw, "dim_model_base", float),
            scale_depth=None if sd is None else field_from(raw, "scale_depth", float),
            tie_word_embeddings=None if tie is None else field_from(raw, "tie_word_embeddings", bool),
            sparse_config=sc, eos_token_ids=eos_ids,
            bos_token_id=raw.get("bos_token_id") if isinstance(raw.get("bos_token_id"), int) else None,
            torch_dtype=raw.get("torch_dtype") if isinstance(raw.get("torch_dtype"), str) else None,
        )

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {
            "architectures": [self.architecture], "model_type": "minicpm",
            "vocab_size": self.vocab_size, "hidden_size": self.hidden_size,
            "num_hidden_layers": self.num_hidden_layers, "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads, "head_dim": self.head_dim,
            "intermediate_size": self.intermediate_size, "hidden_act": "silu",
            "rms_norm_eps": self.rms_norm_eps, "rope_theta": self.rope_theta,
            "max_position_embeddings": self.max_position_embeddings,
            "rope_scaling": None if self.rope_scaling is None else self.rope_scaling.to_dict(),
            "scale_emb": self.scale_emb,
            "sparse_config": None if self.sparse_config is None else self.sparse_config.to_dict(),
            "torch_dtype": self.torch_dtype or "bfloat16",
        }
        if not self.rope_attention_scaling:
            d["rope_attention_scaling"] = False
        if self.dim_model_base is not None:
            d["dim_model_base"] = self.dim_model_base
        if self.scale_depth is not None:
            d["scale_depth"] = self.scale_depth
        if self.tie_word_embeddings is not None:
            d["tie_word_embeddings"] = self.tie_word_embeddings
        if self.eos_token_ids:
            d["eos_token_id"] = list(self.eos_token_ids) if len(self.eos_token_ids) > 1 else self.eos_token_ids[0]
        if self.bos_token_id is not None:
            d["bos_token_id"] = self.bos_token_id
        return d
