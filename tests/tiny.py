"""Tiny MiniCPM4 configurations for the tests, and helpers around them.

Two configurations that differ in every size and option: A (tied embeddings,
short LongRoPE factors, dense attention, 2 kv heads of 2 query heads each) and
B (untied, long factors and a cos/sin magnitude > 1, one kv head for 3 query
heads, InfLLM-v2 block-sparse attention whose top-k really prunes).
"""
import json
import os

import torch


def _factors(n, lo, hi, seed):
    g = torch.Generator().manual_seed(seed)
    return [float(x) for x in (torch.rand(n, generator=g, dtype=torch.float64) * (hi - lo) + lo)]


def tiny_a():
    return {
        "architectures": ["MiniCPMForCausalLM"], "model_type": "minicpm",
        "num_hidden_layers": 2, "hidden_size": 64, "num_attention_heads": 4, "num_key_value_heads": 2,
        "intermediate_size": 160, "vocab_size": 512, "rms_norm_eps": 1e-6, "rope_theta": 10000.0,
        "max_position_embeddings": 256,
        "rope_scaling": {"rope_type": "longrope", "short_factor": _factors(8, 1.0, 2.0, 11),
                         "long_factor": _factors(8, 1.0, 2.0, 12), "original_max_position_embeddings": 256},
        "scale_emb": 12, "dim_model_base": 32, "scale_depth": 1.4, "tie_word_embeddings": True,
        "hidden_act": "silu", "eos_token_id": 2, "torch_dtype": "bfloat16",
    }


def tiny_b():
    return {
        "architectures": ["MiniCPMForCausalLM"], "model_type": "minicpm",
        "num_hidden_layers": 3, "hidden_size": 96, "num_attention_heads": 3, "num_key_value_heads": 1,
        "head_dim": 32, "intermediate_size": 256, "vocab_size": 1000, "rms_norm_eps": 1e-5, "rope_theta": 50000.0,
        "max_position_embeddings": 512,
        "rope_scaling": {"rope_type": "longrope", "short_factor": _factors(16, 1.0, 4.0, 21),
                         "long_factor": _factors(16, 1.0, 4.0, 22), "original_max_position_embeddings": 128},
        "scale_emb": 10, "dim_model_base": 48, "scale_depth": 1.0, "tie_word_embeddings": False,
        "hidden_act": "silu", "eos_token_id": [1, 7], "torch_dtype": "bfloat16",
        "sparse_config": {"kernel_size": 8, "kernel_stride": 4, "block_size": 16, "init_blocks": 1, "topk": 4,
                          "window_size": 32, "dense_len": 64},
    }


def write_model(raw, out_dir, seed, norm_std=0.0, std=0.02):
    """A model folder for ``raw`` with random weights, through the package's own writer."""
    import cpmcu_amd
    from cpmcu_amd.weights import write_model_dir
    arch = cpmcu_amd.get_architecture(raw["architectures"][0])
    cfg = arch.config_class.from_dict(raw)
    write_model_dir(cfg, out_dir, seed, std=std, norm_std=norm_std)
    # keep the raw dict as the folder's config.json so that the plain implementation reads the test's own keys
    with open(os.path.join(out_dir, "config.json"), "w") as f:
        json.dump(raw, f, indent=1)
    return out_dir


def read_model(model_dir):
    """(raw config, {name: tensor}) read with nothing but json and safetensors."""
    from safetensors.torch import load_file
    with open(os.path.join(model_dir, "config.json")) as f:
        raw = json.load(f)
    return raw, load_file(os.path.join(model_dir, "model.safetensors"))


def random_tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return [int(t) for t in torch.randint(0, vocab, (n,), generator=g)]
