"""``LLM``: the Python entry point, in the manner of cpmcu's (cpmcu/llm.py:24-379).

Constructor arguments, ``init_storage()``, ``load_from_hf()``, ``prefill()``,
``decode()``, ``generate()`` and ``print_perf_summary()`` keep the reference's
names and meanings.  Differences: ``generate`` also takes a list of prompts (a
batch); ``dtype`` may be float32; the sparse-attention arguments override what
config.json's ``sparse_config`` gives instead of being the only source; the
tokenizer is optional (token ids are first-class).
"""
from __future__ import annotations

import time
from typing import Iterable, List, Optional, Sequence, Union

import torch

from .config.base import architecture_name, read_config_json
from .engine.engine import Engine, EngineOptions, StepEntry
from .engine.generate import Completion, generate as _generate
from .registry import get_architecture
from .utils.perf import PerfTimers

_DTYPE_NAMES = {torch.float32: "float32", torch.bfloat16: "bfloat16", "float32": "float32", "bfloat16": "bfloat16"}


class LLM:
    def __init__(self,
                 path: str,
                 memory_limit: float = 0.8,
                 chunk_length: int = 1024,
                 dtype=None,
                 cuda_graph: bool = False,
                 temperature: float = 0.0,
                 random_seed: Optional[int] = None,
                 max_tokens: Optional[int] = None,
                 max_seq_len: Optional[int] = None,
                 max_batch: Optional[int] = None,
                 device: str = "cuda:0",
                 **model_flags):
        self.path = path
        raw = read_config_json(path)
        self.arch = get_architecture(architecture_name(raw))
        self.config = self.arch.config_class.from_dict(raw)
        if dtype is None:
            dtype = raw.get("torch_dtype", "bfloat16")
            if dtype == "float16":
                dtype = "bfloat16"     # a float16 checkpoint is served in bfloat16 (the loader converts it)
        if dtype in (torch.float16, "float16"):
            raise ValueError("float16 is not built into this engine: use bfloat16 (serving) or float32 (exact)")
        if dtype not in _DTYPE_NAMES:
            raise ValueError(f"Unsupported dtype: {dtype}")
        self.dtype = _DTYPE_NAMES[dtype]
        # The reference's model flags (apply_sparse, sink_window_size, block_window_size, sparse_topk_k,
        # sparse_switch, use_compress_lse, minicpm4_yarn: cpmcu/llm.py:31-36, cpmcu/common/args.py:38-40, 72-83)
        # are keywords that this class does not spell: they go to the architecture that config.json names, which
        # declares the flags it knows, says what they mean for its configuration and which options of its model
        # they switch, and refuses the others.  A flag that is None or not given leaves the architecture's default.
        self.model_flags = dict(model_flags)
        self.config, self.model_options = self.arch.with_flags(self.config, self.model_flags)
        self.memory_limit = memory_limit
        self.chunk_length = chunk_length
        self.cuda_graph = cuda_graph
        self.temperature = temperature
        self.random_seed = random_seed
        self.max_tokens = max_tokens
        self.max_seq_len = max_seq_len
        self.max_batch = max_batch
        self.device = device
        self.engine: Optional[Engine] = None
        self.max_total_length: Optional[int] = None
        self.perf = PerfTimers()
        self._slot: Optional[int] = None
        self.tokenizer = None

    # ------------------------------------------------------------------
    def init_storage(self) -> int:
        """Build the engine and return the longest sequence it can hold (cpmcu/llm.py:115-116 returns the same
        number).  The reference takes ``memory_limit`` of the device's memory in one allocation and gives the
        cache what the weights leave (src/model/memory.cuh:22-43, src/model/kvcache.cuh:50); here the weights
        are read and the workspace is sized first, since their measured bytes, not an estimate, decide what is
        left: the cache gets ``max_tokens`` tokens if that was given, else all that fits under the limit for
        ``max_batch`` sequences (default one) of at most ``max_seq_len`` tokens.  Weights, workspace and cache
        beyond the limit are refused here, with the three numbers, before any step runs."""
        if self.engine is None:
            slots = self.max_batch if (self.max_batch or self.max_tokens is not None) else 1
            opts = EngineOptions(dtype=self.dtype, max_tokens=self.max_tokens, memory_limit=self.memory_limit,
                                 max_seq_len=self.max_seq_len, max_slots=slots, max_step_tokens=self.chunk_length,
                                 device=self.device, hip_graph=self.cuda_graph, model_options=dict(self.model_options))
            # the engine reads config.json itself; what the flags changed is handed over through the typed config
            self.engine = Engine.from_dir(self.path, opts, config=self.config)
            self.engine.perf = self.perf
            self.max_tokens = self.engine.max_tokens
        self.max_total_length = min(self.max_tokens, self.engine.max_seq_len)
        return self.max_total_length

    def load_from_hf(self):
        """The reference's second call (cpmcu/cli.py:257, 285).  The weights were read when init_storage built
        the engine, so nothing is left to do but to say so when the order is wrong."""
        if self.engine is None:
            raise RuntimeError("call init_storage() before load_from_hf()")
        return self

    def _need_engine(self) -> Engine:
        if self.engine is None:
            raise RuntimeError("the model is not loaded: call init_storage() and load_from_hf() first")
        return self.engine

    # ------------------------------------------------------------------
    def prefill(self, input_ids, position_ids=None, progress_callback=None, logits_buffer=None):
        """Run a prompt from position 0 (a new sequence) and return the logits of its last token, [1, vocab]."""
        eng = self._need_engine()
        ids = [int(t) for t in (input_ids.view(-1).tolist() if isinstance(input_ids, torch.Tensor) else input_ids)]
        if len(ids) > self.max_total_length:
            raise ValueError(f"Input token count ({len(ids)}) exceeds maximum supported length "
                             f"({self.max_total_length}) under current memory limit")
        if self._slot is not None:
            eng.release(self._slot)
        self._slot = eng.acquire()
        if progress_callback:
            progress_callback("begin", {"total_tokens": len(ids)})
        t0 = time.time()
        logits = None
        for a in range(0, len(ids), self.chunk_length):
            b = min(a + self.chunk_length, len(ids))
            with self.perf.gpu("prefill_chunk"):
                logits = eng.step([StepEntry(self._slot, ids[a:b], [b - a - 1] if b == len(ids) else [])])
            if progress_callback:
                progress_callback("advance", {"current_tokens": b})
        self._last_prefill_time = time.time() - t0
        if progress_callback:
            progress_callback("finish", {"total_time": self._last_prefill_time})
        return logits

    def decode(self, input_ids, position_ids=None, cache_length=None, mask_2d=None, logits_buffer=None):
        """Run the next token(s) of the sequence that prefill started; logits [n, vocab]."""
        eng = self._need_engine()
        if mask_2d is not None:
            raise ValueError("tree masks belong to speculative decoding, which this engine does not have")
        if self._slot is None:
            raise RuntimeError("decode() before prefill()")
        ids = [int(t) for t in (input_ids.view(-1).tolist() if isinstance(input_ids, torch.Tensor) else input_ids)]
        if cache_length is not None:
            have = int(cache_length.view(-1)[0]) if isinstance(cache_length, torch.Tensor) else int(cache_length)
            if have != eng.length(self._slot):
                raise ValueError(f"cache_length {have} does not match the {eng.length(self._slot)} tokens cached")
        with self.perf.gpu("decode_step"):
            return eng.step([StepEntry(self._slot, ids, list(range(len(ids))))])

    # ------------------------------------------------------------------
    def generate(self, input_ids, generation_length: int = 100, terminators: Iterable[int] = (),
                 use_stream: bool = False, progress_callback=None, temperature: Optional[float] = None):
        """One prompt (1-D tensor or list of ids): ``(tokens, decode_time, prefill_time)`` as the reference
        returns, or with use_stream a generator of {'token','text','is_finished','prefill_time','decode_time'}.
        A list of prompts: a list of Completion, one per prompt."""
        eng = self._need_engine()
        temp = self.temperature if temperature is None else temperature
        if self._slot is not None:
            eng.release(self._slot)
            self._slot = None
        batch = not isinstance(input_ids, torch.Tensor) and len(input_ids) > 0 and not isinstance(input_ids[0], int)
        if batch:
            prompts = [[int(t) for t in (p.view(-1).tolist() if isinstance(p, torch.Tensor) else p)] for p in input_ids]
            return _generate(eng, prompts, generation_length, terminators, temp, self.random_seed,
                             max_batch=self.max_batch, on_prefill=progress_callback)
        prompt = [int(t) for t in (input_ids.view(-1).tolist() if isinstance(input_ids, torch.Tensor) else input_ids)]
        if not use_stream:
            c = _generate(eng, [prompt], generation_length, terminators, temp, self.random_seed,
                          on_prefill=progress_callback)[0]
            return c.tokens, c.decode_time, c.prefill_time
        return self._stream(prompt, generation_length, set(terminators), temp, progress_callback)

    def _stream(self, prompt, generation_length, terminators, temp, progress_callback):
        import queue
        import threading
        q: "queue.Queue" = queue.Queue()
        eng = self._need_engine()
        state = {"prefill": 0.0, "t1": None}

        def on_prefill(ev, data):
            if ev == "finish":
                state["prefill"] = data["total_time"]
                state["t1"] = time.time()
            if progress_callback:
                progress_callback(ev, data)

        def work():
            try:
                _generate(eng, [prompt], generation_length, terminators, temp, self.random_seed,
                          on_token=lambda i, t: q.put(t), on_prefill=on_prefill)
                q.put(None)
            except BaseException as e:  # handed to the consumer
                q.put(e)

        threading.Thread(target=work, daemon=True).start()
        n, prev = 0, None
        while True:
            t = q.get()
            if t is None:
                return
            if isinstance(t, BaseException):
                raise t
            n += 1
            text = self._piece(prev, t)
            prev = t
            yield {"token": t, "text": text, "is_finished": t in terminators or n >= generation_length,
                   "prefill_time": state["prefill"] if n == 1 else 0.0,
                   "decode_time": 0.0 if n == 1 else time.time() - state["t1"]}

    def _piece(self, prev, token) -> str:
        """Text of one token; decoded together with the previous token for correct spacing
        (cpmcu/llm.py:327-334)."""
        if self.tokenizer is None:
            return ""
        if prev is None:
            return self.tokenizer.decode([token])
        return self.tokenizer.decode([prev, token])[len(self.tokenizer.decode([prev])):]

    def print_perf_summary(self):
        self.perf.print_summary()
