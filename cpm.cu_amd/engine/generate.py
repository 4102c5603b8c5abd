"""The generation loop above the step function.

For one prompt the reference loops ``prefill -> sample -> (decode -> sample)*``,
returns the stop token and ends the sequence on it, and counts the token sampled
from the prompt's logits toward the length (cpmcu/llm.py:261-376).  Here the
same loop runs over batches: prompts of unequal length start together in one
step, every later step carries one token of each sequence still running, a
sequence that ends gives its slot back at once, and when there are more
requests than one batch holds, batches run one after another.
"""
from __future__ import annotations

import time
from dataclasses import dataclass, field
from typing import Callable, Dict, Iterable, List, Optional, Sequence

import torch

from ..sampling.sampler import Sampler
from .engine import Engine, StepEntry


@dataclass
class Completion:
    tokens: List[int]
    finish_reason: str                      # 'stop' (a stop token, which is returned) or 'length'
    prefill_time: float = 0.0
    decode_time: float = 0.0


def plan_batches(prompt_lens: Sequence[int], max_new_tokens: int, max_batch: int,
                 pages_to_hold: Callable[[int], Sequence[int]], capacity: Sequence[int],
                 max_seq_len: int) -> List[List[int]]:
    """Split request indices into batches that run one after another.

    Requests keep their order.  A batch takes requests while it has a slot for each and every group of the
    cache can hold every one of them at its full length (prompt + max_new_tokens).  How many pages of each
    group a sequence of a given length holds is the cache's to say (``pages_to_hold(length)``, one number a
    group: a group that keeps a window needs fewer than one that keeps everything); ``capacity`` is the
    groups' pools."""
    if max_new_tokens < 1:
        raise ValueError("max_new_tokens must be at least 1")
    if max_batch < 1:
        raise ValueError("max_batch must be at least 1")
    batches: List[List[int]] = []
    cur: List[int] = []
    cur_pages = [0] * len(capacity)
    for i, n in enumerate(prompt_lens):
        if n < 1:
            raise ValueError(f"request {i}: the prompt is empty")
        total = n + max_new_tokens - 1      # the last sampled token is never fed back
        if total > max_seq_len:
            raise ValueError(f"request {i}: prompt of {n} + {max_new_tokens} new tokens exceeds the longest sequence "
                             f"the engine holds ({max_seq_len})")
        pages = list(pages_to_hold(total))
        if any(p > c for p, c in zip(pages, capacity)):
            raise ValueError(f"request {i}: {total} tokens do not fit the cache ({pages} pages needed, "
                             f"{list(capacity)} in all)")
        if cur and (len(cur) >= max_batch or any(a + p > c for a, p, c in zip(cur_pages, pages, capacity))):
            batches.append(cur)
            cur, cur_pages = [], [0] * len(capacity)
        cur.append(i)
        cur_pages = [a + p for a, p in zip(cur_pages, pages)]
    if cur:
        batches.append(cur)
    return batches


def generate(engine: Engine, prompts: Sequence[Sequence[int]], max_new_tokens: int,
             stop_token_ids: Iterable[int] = (), temperature: float = 0.0, seed: Optional[int] = None,
             max_batch: Optional[int] = None, on_token: Optional[Callable[[int, int], None]] = None,
             on_prefill: Optional[Callable[[str, dict], None]] = None, sampler=None) -> List[Completion]:
    """Generate up to max_new_tokens for every prompt (lists of token ids).

    ``on_token(request index, token)`` is called for each token as it is chosen."""
    stop = set(int(t) for t in stop_token_ids)
    sampler = sampler or Sampler(temperature, seed)
    max_batch = max_batch or engine.cache.max_slots
    max_batch = min(max_batch, engine.cache.max_slots)
    step = int(getattr(engine, "max_step_tokens", 0)) or engine.max_seq_len
    batches = plan_batches([len(p) for p in prompts], max_new_tokens, max_batch,
                           lambda length: engine.cache.pages_to_hold(length, step), engine.cache.capacity(),
                           engine.max_seq_len)
    results: List[Optional[Completion]] = [None] * len(prompts)
    run = _run_batch_overlapped if getattr(engine, "accepts_device_tokens", False) else _run_batch
    for batch in batches:
        run(engine, prompts, batch, max_new_tokens, stop, sampler, results, on_token, on_prefill)
    return results  # type: ignore[return-value]


def _sync(engine):
    if getattr(engine, "device", None) is not None and engine.device.type == "cuda":
        torch.cuda.synchronize(engine.device)


def _prompt_step(engine, prompts, batch, slots, on_prefill):
    """The batch's prompts in one step; an engine that cuts a step into forward passes reports each of them
    ('advance': tokens done so far)."""
    entries = [StepEntry(slots[i], list(prompts[i]), [len(prompts[i]) - 1]) for i in batch]
    if on_prefill is None or not hasattr(engine, "on_pass"):
        return engine.step(entries)
    before = engine.on_pass
    engine.on_pass = lambda done, total: on_prefill("advance", {"current_tokens": done})
    try:
        return engine.step(entries)
    finally:
        engine.on_pass = before


def _run_batch(engine, prompts, batch, max_new_tokens, stop, sampler, results, on_token, on_prefill):
    slots = {i: engine.acquire() for i in batch}
    out: Dict[int, List[int]] = {i: [] for i in batch}
    try:
        _sync(engine)
        t0 = time.time()
        if on_prefill:
            on_prefill("begin", {"total_tokens": sum(len(prompts[i]) for i in batch)})
        logits = _prompt_step(engine, prompts, batch, slots, on_prefill)
        tokens = sampler.sample(logits, batch, [0] * len(batch)).tolist()
        _sync(engine)
        prefill_time = time.time() - t0
        if on_prefill:
            on_prefill("finish", {"total_time": prefill_time})
        active = list(batch)
        t1 = time.time()
        while True:
            nxt = []
            for i, t in zip(active, tokens):
                out[i].append(t)
                if on_token:
                    on_token(i, t)
                if t in stop:
                    reason = "stop"
                elif len(out[i]) >= max_new_tokens:
                    reason = "length"
                else:
                    nxt.append((i, t))
                    continue
                results[i] = Completion(out[i], reason, prefill_time, time.time() - t1)
                engine.release(slots.pop(i))
            if not nxt:
                break
            active = [i for i, _ in nxt]
            logits = engine.step([StepEntry(slots[i], [t], [0]) for i, t in nxt])
            tokens = sampler.sample(logits, active, [len(out[i]) for i in active]).tolist()
    finally:
        for s in slots.values():
            engine.release(s)


def _run_batch_overlapped(engine, prompts, batch, max_new_tokens, stop, sampler, results, on_token, on_prefill):
    """The same loop with the host one step behind the GPU: the tokens a step samples stay on the device and
    feed the next step directly, while the host reads the previous step's tokens and decides who has ended.
    A sequence that ends on a stop token has then already been fed once more; that step's token is dropped
    (its cache rows die with the slot).  Sequences that end by length are known beforehand and are not fed."""
    slots = {i: engine.acquire() for i in batch}
    out: Dict[int, List[int]] = {i: [] for i in batch}
    n_gen: Dict[int, int] = {}
    finished = set()
    on_gpu = getattr(engine, "device", None) is not None and engine.device.type == "cuda"
    staging = [torch.empty(len(batch), dtype=torch.int32) for _ in range(2)]
    if on_gpu:
        staging = [t.pin_memory() for t in staging]
    try:
        _sync(engine)
        t0 = time.time()
        if on_prefill:
            on_prefill("begin", {"total_tokens": sum(len(prompts[i]) for i in batch)})
        logits = _prompt_step(engine, prompts, batch, slots, on_prefill)
        first = sampler.sample(logits, batch, [0] * len(batch))
        tokens = first.tolist()
        prefill_time = time.time() - t0
        if on_prefill:
            on_prefill("finish", {"total_time": prefill_time})
        t1 = time.time()

        def resolve(ids, toks):
            for i, t in zip(ids, toks):
                if i in finished:
                    continue
                out[i].append(t)
                if on_token:
                    on_token(i, t)
                reason = "stop" if t in stop else ("length" if len(out[i]) >= max_new_tokens else None)
                if reason:
                    finished.add(i)
                    results[i] = Completion(out[i], reason, prefill_time, time.time() - t1)
                    engine.release(slots.pop(i))

        for i in batch:
            n_gen[i] = 1
        resolve(batch, tokens)
        active = [i for i in batch if i not in finished]
        feed_host: Optional[List[int]] = [out[i][-1] for i in active]
        feed_dev = None
        inflight = None
        turn = 0
        while active or inflight is not None:
            launched = None
            if active:
                entries = [StepEntry(slots[i], [feed_host[k] if feed_host is not None else 0], [0])
                           for k, i in enumerate(active)]
                logits = engine.step(entries, device_tokens=feed_dev)
                sampled = sampler.sample(logits, active, [n_gen[i] for i in active])
                for i in active:
                    n_gen[i] += 1
                host = staging[turn][:len(active)]
                turn ^= 1
                host.copy_(sampled, non_blocking=True)
                ev = None
                if on_gpu:
                    ev = torch.cuda.Event()
                    ev.record()
                launched = (list(active), sampled, host, ev)
            if inflight is not None:
                ids, _, host, ev = inflight
                if ev is not None:
                    ev.synchronize()
                resolve(ids, host.tolist())
            inflight = launched
            active, feed_host, feed_dev = [], None, None
            if inflight is not None:
                ids, sampled = inflight[0], inflight[1]
                keep = [k for k, i in enumerate(ids) if i not in finished and n_gen[i] < max_new_tokens]
                active = [ids[k] for k in keep]
                if active:
                    feed_dev = sampled if len(keep) == len(ids) else sampled.index_select(
                        0, torch.tensor(keep, dtype=torch.long).to(sampled.device, non_blocking=True))
    finally:
        for s in slots.values():
            engine.release(s)
