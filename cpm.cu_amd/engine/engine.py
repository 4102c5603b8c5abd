"""The engine: a model bound to a GPU, its cache, and the one step function.

``step`` takes a batch of sequences, each with the next tokens it brings
(a whole prompt, a chunk of one, or a single token) and the places among them
whose logits are wanted.  It runs only those tokens, as one packed batch without
padding, against what earlier steps left in the cache, and returns float32
logits.  The reference has two entry points for one sequence, ``prefill(n,
history, ...)`` and ``decode(...)`` (src/entry.cu:558-584,
src/model/minicpm4/minicpm4_model.cuh:125-153); batches, slots and the single
step function are this engine's own.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..cache.paged import CacheError, SequenceCache
from ..config.base import ModelConfig, architecture_name, read_config_json
from ..parts.base import Runtime, StepContext, Workspace
from ..registry import get_architecture
from ..weights.loader import checkpoint_names, load_tensors

_DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16, "fp32": torch.float32, "bf16": torch.bfloat16}


def _bytes_on(tensors, device) -> int:
    """Bytes of the distinct storages of those tensors that lie on ``device``."""
    seen = {}
    for t in tensors:
        if t.device == device:
            st = t.untyped_storage()
            seen[st.data_ptr()] = st.nbytes()
    return sum(seen.values())


class StepError(ValueError):
    """A step was refused; nothing was run and the cache is unchanged."""


class EngineMemoryError(ValueError):
    """Weights, workspace and cache together exceed the engine's memory limit; said when the engine is built."""


@dataclass
class EngineOptions:
    dtype: str = "bfloat16"                 # 'bfloat16' (serving kernels) or 'float32' (everything in true 32-bit)
    # tokens all live sequences hold together (each rounded up to a page); None: what memory_limit leaves
    max_tokens: Optional[int] = 8192
    # fraction of the device's memory that weights, workspace and cache may take together (the reference's
    # memory_limit, src/model/memory.cuh:22-43); checked when the engine is built.  None: not checked
    memory_limit: Optional[float] = None
    max_seq_len: Optional[int] = None       # longest sequence; default: what the configuration says the model is for
    max_slots: Optional[int] = None         # live sequences; default: one per page, at most 1024
    max_step_tokens: int = 2048             # tokens one forward pass carries (the reference's chunk_length)
    page_size: int = 64
    device: str = "cuda:0"
    hip_graph: bool = False                 # replay single-token steps from a captured graph
    tiled_weights: bool = True              # second copy of the linear weights laid out for decode steps (bf16)
    # options of the architecture's own (those its registry entry declares, e.g. 'sparse' for MiniCPM4)
    model_options: Dict[str, Any] = field(default_factory=dict)
    max_graphs: int = 32                    # captured decode steps kept (one per batch size and position bound)
    # run a prompt pass of max_step_tokens tokens and decode passes on a scratch cache while the engine is built,
    # so that the workspace has its full size before the memory figure is made and no later step allocates
    rehearse: bool = True


@dataclass
class StepEntry:
    slot: int
    tokens: Sequence[int]
    want: Sequence[int] = ()                # indices into ``tokens`` whose logits are returned


class Engine:
    def __init__(self, config: ModelConfig, model, tensors: Dict[str, torch.Tensor], options: EngineOptions,
                 allocated_before: Optional[int] = None):
        """``tensors``: the checkpoint's tensors on the device; the dictionary is emptied once the parts have
        taken what they keep.  ``allocated_before``: the device allocator's count before those tensors were
        loaded (from_dir and from_tensors pass it), from which the weights' share of memory is measured."""
        if options.dtype not in _DTYPES:
            raise ValueError(f"dtype '{options.dtype}' is not supported (float32, bfloat16)")
        self.options = options
        self.config = config
        self.model = model
        self.device = torch.device(options.device)
        if self.device.type != "cuda":
            raise RuntimeError("the engine runs on a GPU only (device 'cuda:N'); there is no CPU path")
        if not torch.cuda.is_available():
            raise RuntimeError("no GPU is visible: the engine's kernels cannot run")
        if self.device.index is None:
            self.device = torch.device("cuda", torch.cuda.current_device())
        self.dtype = _DTYPES[options.dtype]
        page = options.page_size
        if page <= 0 or page % 32:
            raise ValueError(f"page_size {page}: the cache kernels lay a page out in chunks of 32 tokens; "
                             f"give a positive multiple of 32")
        if options.max_tokens is None and options.memory_limit is None:
            raise ValueError("give max_tokens, or a memory_limit from which the cache is sized")
        if options.memory_limit is not None and not 0 < options.memory_limit <= 1:
            raise ValueError(f"memory_limit {options.memory_limit} must be a fraction of the device's memory in (0, 1]")
        max_seq_len = options.max_seq_len or config.longest_sequence or options.max_tokens
        if not max_seq_len:
            raise ValueError("max_seq_len is needed: the configuration names no longest sequence and max_tokens is open")
        self.max_seq_len = int(max_seq_len)
        self.max_step_tokens = max(int(options.max_step_tokens), 1)
        if options.max_tokens is not None:
            max_slots = options.max_slots or min(-(-options.max_tokens // page), 1024)
        else:
            max_slots = options.max_slots or 1
        if allocated_before is None:
            allocated_before = torch.cuda.memory_allocated(self.device) - _bytes_on(tensors.values(), self.device)
        self.workspace = Workspace(self.device)
        # parts check here, at bind time, what their kernels take of these sizes: an engine that was built runs
        self.runtime = Runtime(self.device, self.dtype, self.workspace, self.max_seq_len, options.tiled_weights, page)
        with torch.cuda.device(self.device):
            model.bind_all(tensors, self.runtime)
            parts = model.all_parts()
            for part in parts:
                part.reserve_workspace(self.workspace, self.runtime, self.max_step_tokens, max_slots)
        tensors.clear()
        # a part that cannot be recorded and replayed keeps the whole model's steps eager
        self.graph_capturable = all(part.graph_capturable for part in parts)
        self.vocab_size = model.vocab_size
        self.steps_run = 0
        self.perf = None                       # utils.perf.PerfTimers; while enabled, steps run eagerly (no graph)
        self.on_pass = None                    # called (tokens done, tokens of the step) after every forward pass
        self._graphs: Dict[Tuple[int, int], tuple] = {}
        cap = 3 * self.max_step_tokens + 3 * max_slots + 1 + self.max_step_tokens
        self._meta = torch.zeros(cap, dtype=torch.int32, device=self.device)
        self._stage = [torch.empty(cap, dtype=torch.int32).pin_memory() for _ in range(4)]
        self._stage_ev: List[Optional[torch.cuda.Event]] = [None] * 4
        self._stage_i = 0
        needs = model.cache_needs()
        self._rehearsing = False
        self.max_tokens = options.max_tokens or 0
        if options.rehearse:
            self._rehearse(needs, max_slots)
        # the memory figure: everything this engine holds beside the cache is allocated by now
        torch.cuda.synchronize(self.device)
        held = torch.cuda.memory_allocated(self.device) - allocated_before
        ws_bytes = self.workspace.bytes()
        self.weight_bytes = max(held - ws_bytes, 0)        # every copy of the weights, and the product library's scratch
        total = torch.cuda.get_device_properties(self.device).total_memory
        limit = int(options.memory_limit * total) if options.memory_limit is not None else None
        plan = lambda tokens: SequenceCache.plan_bytes(needs, tokens, max_slots, self.max_seq_len, page, self.dtype,
                                                        self.max_step_tokens)
        # what the device can still give: free memory, and what torch's allocator holds without using it
        free_now = torch.cuda.mem_get_info(self.device)[0] + (torch.cuda.memory_reserved(self.device)
                                                              - torch.cuda.memory_allocated(self.device))
        if options.max_tokens is None:
            budget = min(limit - held, free_now - (256 << 20))
            tokens = SequenceCache.tokens_for(needs, budget, max_slots, self.max_seq_len, page, self.dtype,
                                              self.max_step_tokens)
            if tokens == 0:
                raise EngineMemoryError(self._memory_message(limit, total, plan(max_slots * page), max_slots * page,
                                                             free_now))
            self.max_tokens = tokens
        else:
            self.max_tokens = int(options.max_tokens)
            over_limit = limit is not None and held + plan(self.max_tokens) > limit
            if over_limit or plan(self.max_tokens) > free_now:
                raise EngineMemoryError(self._memory_message(limit if over_limit else None, total,
                                                             plan(self.max_tokens), self.max_tokens, free_now))
        self.cache = SequenceCache(needs, self.max_tokens, max_slots, self.max_seq_len, page, self.device, self.dtype,
                                   self.max_step_tokens)
        self.workspace.sealed = True

    def _memory_message(self, limit: Optional[int], total: int, cache_bytes: int, tokens: int, free_now: int) -> str:
        gib = lambda b: f"{b / 2**30:.2f} GiB"
        figure = (f"weights {gib(self.weight_bytes)} + workspace {gib(self.workspace.bytes())} + cache {gib(cache_bytes)} "
                  f"(for {tokens} tokens) = {gib(self.weight_bytes + self.workspace.bytes() + cache_bytes)}")
        if limit is None:
            return (f"device memory exceeded: {figure}; weights and workspace are in place and the device has "
                    f"{gib(free_now)} left for the cache")
        return (f"memory limit exceeded: {figure}, the limit is {gib(limit)} "
                f"({self.options.memory_limit:.0%} of the device's {gib(total)}; {gib(free_now)} of it are free for the cache)")

    def _rehearse(self, needs, max_slots: int):
        """One prompt pass of max_step_tokens tokens and decode passes of the largest and of small batches, on a
        scratch cache that is freed afterwards: every part asks the workspace for what its largest steps need,
        and the product library sets itself up, before the memory figure is made."""
        page = self.options.page_size
        n_prompt = min(self.max_step_tokens, self.max_seq_len)
        B = max(min(max_slots, self.max_step_tokens), 1)
        tokens = -(-n_prompt // page) * page + B * page
        self.cache = SequenceCache(needs, tokens, B + 1, self.max_seq_len, page, self.device, self.dtype,
                                   self.max_step_tokens)
        self._rehearsing = True
        try:
            s = self.acquire()
            # token ids spread over the vocabulary (the product library sets itself up on ordinary rows)
            self.step([StepEntry(s, [(7919 * i) % self.vocab_size for i in range(n_prompt)], [n_prompt - 1])])
            self.release(s)
            # kernels change with the number of rows at powers of two at most: those sizes and their successors
            sizes = {1}
            b = 2
            while b < max(B, n_prompt):
                sizes.update((b, b + 1))
                b *= 2
            for b in sorted(sizes | {B}, reverse=True):
                if b <= B:
                    slots = [self.acquire() for _ in range(b)]
                    self.step([StepEntry(x, [0], [0]) for x in slots])         # a decode step of b sequences
                    for x in slots:
                        self.release(x)
                if 2 <= b < n_prompt:
                    s = self.acquire()
                    self.step([StepEntry(s, [0] * b, [b - 1])])                  # a short prompt of b tokens
                    self.release(s)
        finally:
            self._rehearsing = False
            self.cache = None
            self.steps_run = 0
        torch.cuda.synchronize(self.device)
        torch.cuda.empty_cache()

    @property
    def uses_graph(self) -> bool:
        """Whether single-token steps replay a captured graph."""
        return bool(self.options.hip_graph) and self.graph_capturable and not self._rehearsing

    # ------------------------------------------------------------------
    @classmethod
    def from_dir(cls, model_dir: str, options: Optional[EngineOptions] = None,
                 config: Optional[ModelConfig] = None) -> "Engine":
        """Build the model that config.json names and load its weights from the folder.
        ``config`` replaces the typed configuration read from config.json (same architecture)."""
        options = options or EngineOptions()
        raw = read_config_json(model_dir)
        arch = get_architecture(architecture_name(raw))
        if config is None:
            config = arch.config_class.from_dict(raw)
        model = arch.build_model(config, options.model_options, checkpoint_names(model_dir))
        dev = torch.device(options.device)
        before = torch.cuda.memory_allocated(dev) if dev.type == "cuda" and torch.cuda.is_available() else None
        tensors = load_tensors(
            model_dir, model.all_weight_specs(), device=options.device,
            split_fused=(lambda n, t: arch.split_fused(config, n, t)) if arch.split_fused else None,
            ignore=(lambda n: arch.ignore_tensor(config, n)) if arch.ignore_tensor else None)
        return cls(config, model, tensors, options, before)

    @classmethod
    def from_tensors(cls, config: ModelConfig, tensors: Dict[str, torch.Tensor],
                     options: Optional[EngineOptions] = None) -> "Engine":
        options = options or EngineOptions()
        arch = get_architecture(config.architecture)
        model = arch.build_model(config, options.model_options, tensors.keys())
        from ..weights.loader import _compare
        _compare(model.all_weight_specs(), {k: tuple(v.shape) for k, v in tensors.items()}, "the given tensors")
        dev = torch.device(options.device)
        before = None
        if dev.type == "cuda" and torch.cuda.is_available():
            dev = torch.device("cuda", dev.index if dev.index is not None else torch.cuda.current_device())
            before = torch.cuda.memory_allocated(dev) - _bytes_on(tensors.values(), dev)
        return cls(config, model, {k: v.to(dev) for k, v in tensors.items()}, options, before)

    # ------------------------------------------------------------------
    def acquire(self) -> int:
        return self.cache.acquire()

    def release(self, slot: int):
        self.cache.release(slot)

    def length(self, slot: int) -> int:
        return self.cache.length(slot)

    # ------------------------------------------------------------------
    def _validate(self, entries: Sequence[StepEntry]):
        if not entries:
            raise StepError("a step needs at least one sequence")
        seen = set()
        V = self.vocab_size
        for e in entries:
            if e.slot in seen:
                raise StepError(f"slot {e.slot} occurs twice in one step")
            seen.add(e.slot)
            try:
                have = self.cache.length(e.slot)
            except CacheError as err:
                raise StepError(str(err)) from None
            n = len(e.tokens)
            if n == 0:
                raise StepError(f"slot {e.slot}: a step must bring at least one token")
            if have + n > self.max_seq_len:
                raise StepError(f"slot {e.slot}: {have} cached + {n} new tokens exceed the longest sequence "
                                f"this engine holds ({self.max_seq_len})")
            bad = [t for t in e.tokens if not 0 <= int(t) < V]
            if bad:
                raise StepError(f"slot {e.slot}: token id {bad[0]} is outside the vocabulary [0, {V})")
            for w in e.want:
                if not 0 <= int(w) < n:
                    raise StepError(f"slot {e.slot}: wanted place {w} is outside the {n} tokens of this step")
        full = self.cache.room_for([[(entries[i].slot, b - a) for i, a, b in chunk] for chunk in self._chunks(entries)])
        if full is not None:
            raise StepError(f"{full} (max_tokens={self.max_tokens})")

    def _chunks(self, entries: Sequence[StepEntry]):
        """Cut a step into forward passes of at most max_step_tokens tokens.  Yields lists of
        (entry index, first token, last token + 1)."""
        cur: List[Tuple[int, int, int]] = []
        room = self.max_step_tokens
        for i, e in enumerate(entries):
            a, n = 0, len(e.tokens)
            while a < n:
                take = min(n - a, room)
                cur.append((i, a, a + take))
                a += take
                room -= take
                if room == 0:
                    yield cur
                    cur, room = [], self.max_step_tokens
        if cur:
            yield cur

    accepts_device_tokens = True

    def step(self, entries: Sequence[StepEntry], device_tokens: Optional[torch.Tensor] = None
             ) -> Optional[torch.Tensor]:
        """Run the entries' tokens; float32 logits [wanted, vocab] in the order of entries and of ``want``
        (None if nothing is wanted).  ``device_tokens`` (int32 [entries], on the GPU; single-token steps only)
        replaces the entries' token ids: a decode loop can feed what it sampled without reading it back."""
        entries = [e if isinstance(e, StepEntry) else StepEntry(*e) for e in entries]
        if entries and len(entries) <= self.max_step_tokens and all(len(e.tokens) == 1 for e in entries):
            if device_tokens is not None and (device_tokens.dtype != torch.int32 or device_tokens.device != self.device
                                              or tuple(device_tokens.shape) != (len(entries),)):
                raise StepError(f"device_tokens must be int32 [{len(entries)}] on {self.device}")
            with torch.cuda.device(self.device):
                out = self._step_single_tokens(entries, device_tokens)
            self.steps_run += 1
            return out
        if device_tokens is not None:
            raise StepError("device_tokens serve steps in which every sequence brings exactly one token")
        self._validate(entries)
        row_of: Dict[Tuple[int, int], List[int]] = {}
        n_rows = 0
        for i, e in enumerate(entries):
            for w in e.want:
                row_of.setdefault((i, int(w)), []).append(n_rows)
                n_rows += 1
        result = torch.empty((n_rows, self.vocab_size), dtype=torch.float32, device=self.device) if n_rows else None
        done, total = 0, sum(len(e.tokens) for e in entries)
        with torch.cuda.device(self.device):
            for chunk in self._chunks(entries):
                self._forward(entries, chunk, row_of, result)
                done += sum(b - a for _, a, b in chunk)
                if self.on_pass is not None:
                    self.on_pass(done, total)
        self.steps_run += 1
        return result

    def _step_single_tokens(self, entries, device_tokens=None) -> Optional[torch.Tensor]:
        """The step of a decode loop: every sequence brings one token.  The same checks and the same forward
        pass as the general path, with the bookkeeping done on whole arrays."""
        cache = self.cache
        B = len(entries)
        slots = [e.slot for e in entries]
        tok = np.fromiter((e.tokens[0] for e in entries), dtype=np.int64, count=B)
        if len(set(slots)) != B:
            dup = next(s for s in slots if slots.count(s) > 1)
            raise StepError(f"slot {dup} occurs twice in one step")
        live = cache.live
        for s in slots:
            if s not in live:
                raise StepError(f"slot {s} is not held by a live sequence")
        if device_tokens is None and (tok.min() < 0 or tok.max() >= self.vocab_size):
            bad = int(tok[(tok < 0) | (tok >= self.vocab_size)][0])
            raise StepError(f"slot {slots[int(np.where(tok == bad)[0][0])]}: token id {bad} is outside the vocabulary "
                            f"[0, {self.vocab_size})")
        want_rows: List[int] = []
        for i, e in enumerate(entries):
            for w in e.want:
                if int(w) != 0:
                    raise StepError(f"slot {e.slot}: wanted place {w} is outside the 1 tokens of this step")
                want_rows.append(i)
        pages = 0
        for s in slots:
            have = live[s]
            if have + 1 > self.max_seq_len:
                raise StepError(f"slot {s}: {have} cached + 1 new tokens exceed the longest sequence this engine "
                                f"holds ({self.max_seq_len})")
            pages += have % cache.page_size == 0
        if pages:
            # a token that opens a page: ask the groups (one that keeps a window gives a page back for it)
            full = cache.room_for([[(s, 1) for s in slots]])
            if full is not None:
                raise StepError(f"{full} (max_tokens={self.max_tokens})")
        before = [live[s] for s in slots]
        pos = np.fromiter((cache.extend_one(s) for s in slots), dtype=np.int32, count=B)
        cache.sync()
        sl = np.asarray(slots, dtype=np.int32)
        graph = self.uses_graph
        rows = np.arange(B, dtype=np.int32) if graph else np.asarray(want_rows, dtype=np.int32)
        host = np.concatenate([tok.astype(np.int32), pos, sl, np.arange(B + 1, dtype=np.int32), sl, pos + 1, rows])
        state = cache.snapshot_state(slots)
        try:
            logits = self._run(host, B, B, [1] * B, int(pos.max()), True, graph, int(rows.size), device_tokens)
        except BaseException:
            self._roll_back(slots, before, state)
            raise
        if not want_rows:
            return None
        if graph and want_rows != list(range(B)):
            return logits.index_select(0, torch.tensor(want_rows, dtype=torch.long).to(self.device, non_blocking=True))
        return logits.clone()

    def _run(self, host: np.ndarray, n: int, B: int, q_lens: List[int], max_pos: int, single: bool, graph: bool,
             R: int, device_tokens: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
        """Upload one forward pass's metadata (tokens, positions, token slots, sequence starts, sequence slots,
        sequence lengths, wanted rows) and run it, eagerly or from a captured graph.  Returns the logits of the
        wanted rows (a view of engine scratch)."""
        perf_on = self.perf is not None and self.perf.enabled
        graph = graph and not perf_on
        if graph:
            # a captured step sizes its launches for the largest position of a whole range of steps, so that
            # one capture serves all of them
            bound = 256
            while bound < max_pos + 1:
                bound *= 2
            max_pos = min(bound, self.max_seq_len) - 1
        key = (B, max_pos)
        entry = self._graphs.get(key) if graph else None
        if entry is not None and entry[3] != self.workspace.generation:
            self._graphs.clear()            # scratch buffers moved: what was captured points at freed memory
            entry = None
        if graph:
            meta = entry[1] if entry is not None else torch.zeros(host.size, dtype=torch.int32, device=self.device)
        else:
            if host.size > self._meta.numel():
                self._meta = torch.zeros(host.size * 2, dtype=torch.int32, device=self.device)
            meta = self._meta
        self._upload(host, meta)
        if device_tokens is not None:
            meta[:n].copy_(device_tokens)
        if entry is not None:
            entry[0].replay()
            return entry[2]
        o1, o2, o3 = n, 2 * n, 3 * n
        o4 = o3 + B + 1
        o5 = o4 + B
        o6 = o5 + B
        ctx = StepContext(
            n_tokens=n, n_seqs=B, token_ids=meta[0:o1], positions=meta[o1:o2], tok_slot=meta[o2:o3],
            cu_q=meta[o3:o4], seq_slot=meta[o4:o5], seq_len=meta[o5:o6], q_lens=q_lens,
            kv_lens=[int(x) for x in host[o5:o6]], max_pos=max_pos, single_token=single,
            ws=self.workspace, cache=self.cache, logit_rows=meta[o6:o6 + R] if R else None,
            perf=self.perf if perf_on else None)
        logits = self.model.forward(ctx)
        if graph:
            # the eager run above did this step's work and sized the scratch buffers; recording the same
            # launches executes nothing and serves the following steps of this batch size
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                captured = self.model.forward(ctx)
            while len(self._graphs) >= max(int(self.options.max_graphs), 1):
                self._graphs.pop(next(iter(self._graphs)))      # the oldest capture goes
            self._graphs[key] = (g, meta, captured, self.workspace.generation)
        return logits

    def _forward(self, entries, chunk, row_of, result):
        cache = self.cache
        B = len(chunk)
        q_lens = [b - a for _, a, b in chunk]
        n = sum(q_lens)
        single = n == B
        graph = self.uses_graph and single
        tok = np.empty(n, dtype=np.int32)
        pos = np.empty(n, dtype=np.int32)
        tslot = np.empty(n, dtype=np.int32)
        cu = np.zeros(B + 1, dtype=np.int32)
        sslot = np.empty(B, dtype=np.int32)
        slen = np.empty(B, dtype=np.int32)
        rows: List[int] = []
        dest: List[int] = []
        o = 0
        before = [cache.length(entries[i].slot) for i, _, _ in chunk]
        state = cache.snapshot_state([entries[i].slot for i, _, _ in chunk])
        for bi, (i, a, b) in enumerate(chunk):
            e = entries[i]
            first = cache.extend(e.slot, b - a)
            q = b - a
            tok[o:o + q] = np.asarray(e.tokens[a:b], dtype=np.int64)
            pos[o:o + q] = np.arange(first, first + q, dtype=np.int32)
            tslot[o:o + q] = e.slot
            cu[bi + 1] = o + q
            sslot[bi] = e.slot
            slen[bi] = first + q
            for w in e.want:
                w = int(w)
                if a <= w < b and (i, w) in row_of:
                    for r in row_of.pop((i, w)):
                        rows.append(o + (w - a))
                        dest.append(r)
            o += q
        cache.sync()
        want_rows = np.arange(B, dtype=np.int32) if graph else np.asarray(rows, dtype=np.int32)
        host = np.concatenate([tok, pos, tslot, cu, sslot, slen, want_rows])
        try:
            logits = self._run(host, n, B, q_lens, int(pos.max()), single, graph, int(want_rows.size))
        except BaseException:
            self._roll_back([entries[i].slot for i, _, _ in chunk], before, state)
            raise
        if rows:
            dest_t = torch.tensor([dest, rows], dtype=torch.long).to(self.device, non_blocking=True)
            if graph:
                result.index_copy_(0, dest_t[0], logits.index_select(0, dest_t[1]))
            else:
                result.index_copy_(0, dest_t[0], logits)

    def _roll_back(self, slots: Sequence[int], lengths: Sequence[int], state=None):
        """A forward pass failed after the cache had made room for its tokens (a kernel refused a size, the
        device ran out of memory): the slots forget that pass's tokens, so that lengths and cache rows agree
        again, and fixed-size state that the pass may have advanced is put back as it was before the pass
        (``state``: SequenceCache.snapshot_state, None for a model without such state).  Passes of the same
        step that had completed before stay (a step that validation refuses, by contrast, changes nothing at all)."""
        for s, n in zip(slots, lengths):
            if s in self.cache.live and self.cache.length(s) > n:
                self.cache.truncate(s, n)
        self.cache.restore_state(state)

    def _upload(self, host: np.ndarray, dst: torch.Tensor):
        """Step metadata to the device through pinned memory, without waiting for the GPU."""
        if host.size > self._stage[0].numel():
            self._stage = [torch.empty(host.size * 2, dtype=torch.int32).pin_memory() for _ in self._stage]
            self._stage_ev = [None] * len(self._stage)
        i = self._stage_i
        self._stage_i = (i + 1) % len(self._stage)
        if self._stage_ev[i] is not None:
            self._stage_ev[i].synchronize()      # the copy that last used this staging buffer has finished
        st = self._stage[i][:host.size]
        st.numpy()[:] = host
        dst[:host.size].copy_(st, non_blocking=True)
        ev = torch.cuda.Event()
        ev.record()
        self._stage_ev[i] = ev

    # ------------------------------------------------------------------
    def memory_report(self) -> Dict[str, int]:
        """Bytes the engine holds on the device: weights (every copy, with the product library's scratch), the
        workspace, the cache; and what the cache holds in tokens."""
        return {"weight_bytes": self.weight_bytes, "workspace_bytes": self.workspace.bytes(),
                "cache_bytes": self.cache.bytes(), "pages": self.cache.n_pages, "slots": self.cache.max_slots,
                "max_tokens": self.max_tokens}
