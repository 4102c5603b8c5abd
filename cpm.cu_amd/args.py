"""Command-line options, with the reference's names and meanings where it has them
(cpmcu/common/args.py:22-131): every option has a --kebab and a --snake spelling and
booleans accept true/false values.  Options of speculative decoding and servers are absent.

The options that belong to an architecture (the reference's sparse-attention group, --minicpm4-yarn, the
names --model-type accepts) are not spelled here: every registered architecture declares its own
(registry.Flag), and the parser offers what is declared.
"""
from __future__ import annotations

import argparse

from .registry import declared_flags, declared_model_types


def str2bool(v):
    if isinstance(v, bool):
        return v
    if v.lower() in ("yes", "true", "t", "y", "1"):
        return True
    if v.lower() in ("no", "false", "f", "n", "0"):
        return False
    raise argparse.ArgumentTypeError("Boolean value expected.")


def _flag(group, *names, default, help):
    group.add_argument(*names, default=default, type=str2bool, nargs="?", const=True, help=help)


def add_model_config_args(parser: argparse.ArgumentParser):
    g = parser.add_argument_group("Model Configuration")
    g.add_argument("--model-path", "--model_path", "--model", type=str, default=None,
                   help="Folder with config.json and safetensors weights (or, with --random-weights, where to write them)")
    g.add_argument("--model-type", "--model_type", type=str, default="auto",
                   choices=["auto"] + declared_model_types(),
                   help="Model type (default: auto: config.json decides); a name sets the flags its architecture "
                        "gives it")
    g.add_argument("--dtype", type=str, default="bfloat16", choices=["bfloat16", "float32"],
                   help="Model dtype (default: bfloat16; float32 runs everything in true 32-bit)")
    g.add_argument("--random-weights", "--random_weights", action="store_true",
                   help="Write a model folder with random weights from --config and --seed, then run on it")
    g.add_argument("--config", type=str, default=None, help="config.json to draw random weights for")
    g.add_argument("--seed", type=int, default=0, help="Seed of the random weights (default: 0)")

    s = parser.add_argument_group("System Configuration")
    _flag(s, "--hip-graph", "--hip_graph", "--cuda-graph", "--cuda_graph", default=True,
          help="Replay decode steps from a captured graph (default: True)")
    s.add_argument("--memory-limit", "--memory_limit", type=float, default=0.9, help="Memory limit (default: 0.9)")
    s.add_argument("--chunk-length", "--chunk_length", type=int, default=2048,
                   help="Chunked prefill size (default: 2048)")
    _flag(s, "--plain-output", "--plain_output", default=False,
          help="Use plain text output (no colors/formatting) (default: False)")
    s.add_argument("--max-tokens", "--max_tokens", type=int, default=None,
                   help="Tokens the cache holds (default: from --memory-limit)")
    s.add_argument("--max-seq-len", "--max_seq_len", type=int, default=None,
                   help="Longest sequence (default: the model's max_position_embeddings)")
    _flag(s, "--perf", default=False, help="Print the timer summary at the end (default: False)")

    # what the registered architectures declare; not given = None = the architecture's own default
    groups = {"Model Configuration": g, "System Configuration": s}
    for f in declared_flags():
        grp = groups.get(f.group)
        if grp is None:
            grp = groups[f.group] = parser.add_argument_group(f.group)
        names = sorted({"--" + f.name.replace("_", "-"), "--" + f.name})
        if f.kind is bool:
            _flag(grp, *names, default=None, help=f.help)
        else:
            grp.add_argument(*names, dest=f.name, type=f.kind, default=None, help=f.help)


def create_cli_parser() -> argparse.ArgumentParser:
    parser = argparse.ArgumentParser(prog="cpmcu_amd.cli", description="cpm.cu_amd CLI")
    p = parser.add_argument_group("Prompt Configuration")
    p.add_argument("--prompt-file", "--prompt_file", type=str, default=None, help="Path to prompt file")
    p.add_argument("--prompt-text", "--prompt_text", type=str, default=None, help="Direct prompt text")
    _flag(p, "--use-chat-template", "--use_chat_template", default=True,
          help="Use chat template for prompt formatting (default: True)")
    p.add_argument("--prompt-ids", "--prompt_ids", type=str, default=None,
                   help="File of token ids: one prompt a line, ids separated by blanks or commas (no tokenizer needed)")
    p.add_argument("--prompt-lens", "--prompt_lens", type=str, default=None,
                   help="Comma-separated lengths of random prompts, e.g. 5,11,17 (ids uniform from --seed)")
    p.add_argument("--batch", "--max-slots", "--max_slots", dest="batch", type=int, default=None, help="Most sequences that run together (default: all that fit)")

    g = parser.add_argument_group("Generation Configuration")
    _flag(g, "--use-stream", "--use_stream", default=True, help="Use stream generation (default: True)")
    g.add_argument("--num-generate", "--num_generate", type=int, default=1024,
                   help="Number of tokens to generate (default: 1024)")
    g.add_argument("--temperature", "--temp", type=float, default=0.0, help="Temperature (default: 0.0)")
    g.add_argument("--random-seed", "--random_seed", type=int, default=None, help="Random seed")
    _flag(g, "--ignore-eos", "--ignore_eos", default=False,
          help="Ignore EOS tokens during generation (default: False)")
    add_model_config_args(parser)
    return parser


def parse_cli_args(argv=None) -> argparse.Namespace:
    return create_cli_parser().parse_args(argv)
