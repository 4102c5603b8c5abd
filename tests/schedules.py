"""Ways of cutting the same requests into steps, driven through the engine's step function.

Every function returns, per request, the logits at all of its positions [len, vocab] (float32, CPU).
"""
from typing import Dict, List, Sequence

import torch

from cpmcu_amd import StepEntry


def whole(engine, requests: Dict[str, List[int]]):
    out = {}
    for rid, toks in requests.items():
        s = engine.acquire()
        out[rid] = engine.step([StepEntry(s, toks, list(range(len(toks))))]).cpu()
        engine.release(s)
    return out


def tail(engine, requests: Dict[str, List[int]], n_tail: int = 32):
    out = {}
    for rid, toks in requests.items():
        s = engine.acquire()
        k = max(len(toks) - n_tail, 1)
        parts = [engine.step([StepEntry(s, toks[:k], list(range(k)))]).cpu()]
        for i in range(k, len(toks)):
            parts.append(engine.step([StepEntry(s, toks[i:i + 1], [0])]).cpu())
        engine.release(s)
        out[rid] = torch.cat(parts)
    return out


def batched(engine, requests: Dict[str, List[int]], prompt_lens: Dict[str, int], batches: Sequence[Sequence[str]]):
    """Batches one after another; in a batch all prompts start together, then one token each;
    a request whose tokens are used up ends and gives its slot back while the others go on."""
    out = {rid: [] for rid in requests}
    for batch in batches:
        slots = {rid: engine.acquire() for rid in batch}
        fed = {rid: prompt_lens[rid] for rid in batch}
        lg = engine.step([StepEntry(slots[r], requests[r][:fed[r]], list(range(fed[r]))) for r in batch])
        o = 0
        for r in batch:
            out[r].append(lg[o:o + fed[r]].cpu())
            o += fed[r]
        live = list(batch)
        while True:
            for r in list(live):
                if fed[r] >= len(requests[r]):
                    engine.release(slots.pop(r))
                    live.remove(r)
            if not live:
                break
            lg = engine.step([StepEntry(slots[r], [requests[r][fed[r]]], [0]) for r in live]).cpu()
            for i, r in enumerate(live):
                out[r].append(lg[i:i + 1])
                fed[r] += 1
    return {r: torch.cat(v) for r, v in out.items()}
