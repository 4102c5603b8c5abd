"""Command line: ``python -m cpmcu_amd.cli --model-path DIR --prompt-text ...``.

The flow is the reference's (cpmcu/cli.py:211-301): resolve the model, build the
``LLM``, make the input ids (chat template when a tokenizer is there), size the
storage, load the weights, generate (streaming by default), print the speeds.
Without a tokenizer the prompt comes as token ids (--prompt-ids / --prompt-lens)
and the output is printed as ids; --random-weights first writes a model folder
from --config and --seed.
"""
from __future__ import annotations

import json
import os
import sys
import tempfile
from typing import List, Optional

from .args import parse_cli_args


def log(msg: str):
    print(f"[cpmcu_amd] {msg}", file=sys.stderr, flush=True)


# what the configuration summary shows (cpmcu/common/display.py:62-90 groups the same facts)
SUMMARY_SECTIONS = (
    ("Model", (("model_path", "Model Path"), ("model_type", "Model Type"), ("dtype", "Data Type"),
               ("minicpm4_yarn", "MiniCPM4 YARN"))),
    ("Generation", (("num_generate", "Num Generate"), ("temperature", "Temperature"), ("random_seed", "Random Seed"),
                    ("use_stream", "Use Stream"), ("ignore_eos", "Ignore EOS"), ("use_chat_template", "Chat Template"))),
    ("System", (("hip_graph", "HIP Graph"), ("memory_limit", "Memory Limit"), ("chunk_length", "Chunk Length"),
                ("max_tokens", "Max Tokens"), ("max_seq_len", "Max Seq Len"), ("batch", "Batch"))),
)


class TextTokenizer:
    """tokenizer.json (and the chat template of tokenizer_config.json) if the model folder has them."""

    def __init__(self, model_dir: str):
        from tokenizers import Tokenizer
        self.tok = Tokenizer.from_file(os.path.join(model_dir, "tokenizer.json"))
        self.chat_template = None
        self.eos_token_id = None
        cfg_path = os.path.join(model_dir, "tokenizer_config.json")
        if os.path.isfile(cfg_path):
            with open(cfg_path, "r", encoding="utf-8") as f:
                cfg = json.load(f)
            self.chat_template = cfg.get("chat_template")
            eos = cfg.get("eos_token")
            if isinstance(eos, dict):
                eos = eos.get("content")
            if isinstance(eos, str):
                self.eos_token_id = self.tok.token_to_id(eos)

    def encode(self, text: str) -> List[int]:
        return self.tok.encode(text).ids

    def decode(self, ids: List[int]) -> str:
        return self.tok.decode(ids, skip_special_tokens=True)

    def apply_chat_template(self, content: str) -> str:
        if not self.chat_template:
            raise ValueError("the tokenizer has no chat template")
        import jinja2
        env = jinja2.Environment()
        return env.from_string(self.chat_template).render(
            messages=[{"role": "user", "content": content}], add_generation_prompt=True, bos_token="", eos_token="")


def load_tokenizer(model_dir: str) -> Optional[TextTokenizer]:
    if os.path.isfile(os.path.join(model_dir, "tokenizer.json")):
        try:
            return TextTokenizer(model_dir)
        except Exception as e:  # a broken tokenizer must not stop id-based runs
            log(f"tokenizer not usable ({e}); working with token ids")
    return None


def make_prompts(args, tokenizer, vocab_size: int) -> List[List[int]]:
    """Input ids as the reference makes them (cpmcu/cli.py:47-79), or from ids / random lengths."""
    if args.prompt_ids:
        prompts = []
        with open(args.prompt_ids, "r", encoding="utf-8") as f:
            for line in f:
                ids = [int(t) for t in line.replace(",", " ").split()]
                if ids:
                    prompts.append(ids)
        if not prompts:
            raise ValueError(f"no token ids in {args.prompt_ids}")
        return prompts
    if args.prompt_lens:
        import torch
        g = torch.Generator().manual_seed(args.seed)
        return [[int(t) for t in torch.randint(0, vocab_size, (int(n),), generator=g)]
                for n in args.prompt_lens.split(",")]
    if tokenizer is None:
        raise ValueError("the model folder has no tokenizer.json: give the prompt as token ids "
                         "(--prompt-ids FILE) or ask for random prompts (--prompt-lens 5,11,17)")
    if args.prompt_file:
        if not os.path.exists(args.prompt_file):
            raise FileNotFoundError(f"Prompt file not found: {args.prompt_file}")
        with open(args.prompt_file, "r", encoding="utf-8") as f:
            content = f.read().strip()
    elif args.prompt_text:
        content = args.prompt_text
    else:
        content = "Who are you"
    prompt = content
    if args.use_chat_template:
        try:
            prompt = tokenizer.apply_chat_template(content)
        except Exception as e:
            log(f"Failed to apply chat template: {e}, using raw prompt")
    log(f"Input prompt: {prompt[:100]!r}{'...' if len(prompt) > 100 else ''}")
    return [tokenizer.encode(prompt)]


def resolve_model_flags(args, arch) -> dict:
    """The flags of the architecture that config.json names, as the command line gave them: the options the
    architecture declares, then what the --model-type name sets where no option said otherwise ('minicpm4' turns
    block-sparse attention on, cpmcu/common/utils.py:123).  A model type or an option that belongs to another
    architecture is refused by name."""
    from .registry import declared_flags
    flags = {f.name: getattr(args, f.name, None) for f in arch.flags}
    if args.model_type != "auto":
        if args.model_type not in arch.model_types:
            raise ValueError(f"--model-type {args.model_type}: architecture '{arch.name}' knows "
                             f"{sorted(arch.model_types) or 'no model types'} (and 'auto')")
        for k, v in arch.model_types[args.model_type].items():
            if flags.get(k) is None:
                flags[k] = v
    foreign = [f.name for f in declared_flags() if f.name not in flags and getattr(args, f.name, None) is not None]
    if foreign:
        raise ValueError(f"architecture '{arch.name}' has no flags {foreign}")
    return flags


def run_generation(args):
    from . import get_architecture
    from .config.base import architecture_name, read_config_json
    from .llm import LLM
    from .utils.display import Display

    display = Display(plain=args.plain_output)

    model_path = args.model_path
    if args.random_weights:
        if not args.config:
            raise ValueError("--random-weights needs --config <config.json>")
        from .weights import write_model_dir
        with open(args.config, "r", encoding="utf-8") as f:
            raw = json.load(f)
        cfg = get_architecture(architecture_name(raw)).config_class.from_dict(raw)
        model_path = model_path or tempfile.mkdtemp(prefix="cpmcu_amd_random_")
        log(f"writing random weights (seed {args.seed}) to {model_path}")
        write_model_dir(cfg, model_path, args.seed)
    if not model_path:
        raise ValueError("model_path is required")
    if not os.path.isdir(model_path):
        raise FileNotFoundError(f"model folder not found: {model_path} (there is no download: give a local folder)")

    arch = get_architecture(architecture_name(read_config_json(model_path)))
    flags = resolve_model_flags(args, arch)
    sections = list(SUMMARY_SECTIONS)
    if arch.flags:
        sections.append((arch.name, tuple((f.name, f.name.replace("_", " ").title()) for f in arch.flags)))
    display.configuration(args, sections)
    tokenizer = load_tokenizer(model_path)
    llm = LLM(model_path, memory_limit=args.memory_limit, chunk_length=args.chunk_length, dtype=args.dtype,
              cuda_graph=args.hip_graph, temperature=args.temperature, random_seed=args.random_seed,
              max_tokens=args.max_tokens, max_seq_len=args.max_seq_len, max_batch=args.batch, **flags)
    llm.tokenizer = tokenizer
    llm.perf.enabled = bool(args.perf)
    prompts = make_prompts(args, tokenizer, llm.config.vocabulary_size)
    log(f"Input tokens: {[len(p) for p in prompts]}")
    terminators = []
    if not args.ignore_eos:
        terminators = list(llm.config.stop_token_ids)
        if tokenizer is not None and tokenizer.eos_token_id is not None and tokenizer.eos_token_id not in terminators:
            terminators.append(tokenizer.eos_token_id)

    log("Loading model weights and sizing the cache...")
    if args.max_tokens is None and args.batch is None:
        llm.max_batch = len(prompts)
    max_len = llm.init_storage()
    llm.load_from_hf()
    mem = llm.engine.memory_report()
    log(f"Maximum context length under current memory limit: {max_len} tokens "
        f"(weights {mem['weight_bytes'] / 2**30:.2f} GiB, workspace {mem['workspace_bytes'] / 2**30:.2f} GiB, cache "
        f"{mem['cache_bytes'] / 2**30:.2f} GiB for {mem['max_tokens']} tokens in {mem['slots']} slots)")
    log("Model loading completed!")

    if len(prompts) == 1 and args.use_stream:
        tokens = []
        prefill_time = decode_time = 0.0
        for ev in llm.generate(prompts[0], args.num_generate, terminators, use_stream=True,
                               progress_callback=display.progress_callback()):
            tokens.append(ev["token"])
            prefill_time = max(prefill_time, ev["prefill_time"])
            decode_time = max(decode_time, ev["decode_time"])
            sys.stdout.write(ev["text"] if tokenizer is not None else f"{ev['token']} ")
            sys.stdout.flush()
        sys.stdout.write("\n")
        stats = [(len(prompts[0]), prefill_time, len(tokens), decode_time)]
    else:
        outs = llm.generate(prompts, args.num_generate, terminators, progress_callback=display.progress_callback())
        stats = []
        for i, c in enumerate(outs):
            text = tokenizer.decode(c.tokens) if tokenizer is not None else " ".join(str(t) for t in c.tokens)
            print(f"[{i}] ({c.finish_reason}) {text}")
            stats.append((len(prompts[i]), c.prefill_time, len(c.tokens), c.decode_time))
    # the figures the reference prints (cpmcu/common/display.py:95-115)
    n_prompt = sum(s[0] for s in stats)
    t_prefill = max(s[1] for s in stats)
    n_dec = sum(max(s[2] - 1, 0) for s in stats)
    t_dec = max(s[3] for s in stats)
    display.performance(n_prompt, t_prefill, n_dec, t_dec)
    if args.perf:
        llm.print_perf_summary()


def main(argv=None):
    # a fatal signal prints the Python stack of every thread (the reference installs handlers that print a
    # native backtrace, src/signal_handler.cu:7-124)
    import faulthandler
    faulthandler.enable()
    try:
        run_generation(parse_cli_args(argv))
    except (ValueError, FileNotFoundError) as e:
        log(f"Configuration error: {e}")
        sys.exit(1)
    except RuntimeError as e:
        log(f"Runtime error: {e}")
        sys.exit(1)
    except KeyboardInterrupt:
        log("Generation interrupted by user.")
        sys.exit(0)


if __name__ == "__main__":
    main()
