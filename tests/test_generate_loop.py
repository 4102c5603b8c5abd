"""The generation loop's decisions, with a stand-in engine and sampler (CPU).  Every scenario runs through both
forms of the loop: the plain one, and the one that the GPU engine gets, in which the host is one step behind
(a stand-in engine that takes ``device_tokens`` is given that one)."""
import pytest
import torch

from cpmcu_amd.engine.generate import generate, plan_batches


class FakeCache:
    page_size = 16

    def __init__(self, slots, max_tokens):
        self.max_slots = slots
        self.max_tokens = max_tokens

    def pages_to_hold(self, length, step):
        return [-(-length // self.page_size)]

    def capacity(self):
        return [self.max_tokens // self.page_size]


class FakeEngine:
    """Logits that make greedy emit (last token + 1) % vocab; records every step."""

    def __init__(self, vocab=50, slots=4, max_tokens=4096, max_seq_len=512, overlapped=False):
        self.accepts_device_tokens = overlapped
        class O:
            pass
        self.options = O()
        self.options.max_tokens = max_tokens
        self.cache = FakeCache(slots, max_tokens)
        self.max_seq_len = max_seq_len
        self.device = torch.device("cpu")
        self.vocab = vocab
        self.free = list(range(slots))
        self.held = {}
        self.log = []

    def acquire(self):
        s = self.free.pop(0)
        self.held[s] = 0
        return s

    def release(self, s):
        assert s in self.held, "slot released twice"
        del self.held[s]
        self.free.append(s)

    def step(self, entries, device_tokens=None):
        if device_tokens is not None:
            assert self.accepts_device_tokens and all(len(e.tokens) == 1 for e in entries)
            assert device_tokens.dtype == torch.int32 and tuple(device_tokens.shape) == (len(entries),)
            entries = [type(e)(e.slot, [int(t)], e.want) for e, t in zip(entries, device_tokens)]
        self.log.append([(e.slot, list(e.tokens)) for e in entries])
        rows = []
        for e in entries:
            assert e.slot in self.held
            self.held[e.slot] += len(e.tokens)
            for w in e.want:
                row = torch.zeros(self.vocab)
                row[(e.tokens[w] + 1) % self.vocab] = 1.0
                rows.append(row)
        return torch.stack(rows)


class ArgmaxSampler:
    def sample(self, logits, request_ids, steps):
        self.last = (list(request_ids), list(steps))
        return logits.argmax(-1).to(torch.int32)


BOTH = pytest.mark.parametrize("overlapped", [False, True], ids=["plain loop", "host one step behind"])


@BOTH
def test_unequal_prompts_stop_tokens_and_early_leavers(overlapped):
    eng = FakeEngine(overlapped=overlapped)
    prompts = [[1, 2, 3], [10], [20, 21, 22, 23, 24]]
    outs = generate(eng, prompts, max_new_tokens=6, stop_token_ids=[13, 27], sampler=ArgmaxSampler())
    assert outs[0].tokens == [4, 5, 6, 7, 8, 9] and outs[0].finish_reason == "length"
    assert outs[1].tokens == [11, 12, 13] and outs[1].finish_reason == "stop"       # the stop token is returned
    assert outs[2].tokens == [25, 26, 27] and outs[2].finish_reason == "stop"
    # step 0 carries the whole prompts; then one token each; finished sequences leave the batch
    assert [len(t) for _, t in eng.log[0]] == [3, 1, 5]
    assert all(len(t) == 1 for step in eng.log[1:] for _, t in step)
    # with the host one step behind, the two sequences that stop at their third token have been fed once more
    # before the host saw the stop token; what that step chose for them is dropped
    assert [len(step) for step in eng.log] == ([3, 3, 3, 3, 1, 1] if overlapped else [3, 3, 3, 1, 1, 1])
    assert not eng.held and sorted(eng.free) == [0, 1, 2, 3]
    # the first sampled token counts toward the length: 6 tokens need 5 single-token steps; a sequence that ends
    # by length is never fed its last token, in either loop
    assert len(eng.log) == 6 and eng.log[-1] == [(0, [8])]


@BOTH
def test_first_token_can_already_stop(overlapped):
    eng = FakeEngine(overlapped=overlapped)
    outs = generate(eng, [[4], [8]], max_new_tokens=5, stop_token_ids=[5], sampler=ArgmaxSampler())
    assert outs[0].tokens == [5] and outs[0].finish_reason == "stop"
    assert outs[1].tokens == [9, 10, 11, 12, 13]
    assert [len(s) for s in eng.log] == [2, 1, 1, 1, 1]


@BOTH
def test_more_requests_than_slots_run_as_batches_one_after_another(overlapped):
    eng = FakeEngine(slots=2, overlapped=overlapped)
    prompts = [[i] for i in range(5)]
    s = ArgmaxSampler()
    outs = generate(eng, prompts, max_new_tokens=2, sampler=s)
    assert [o.tokens for o in outs] == [[i + 1, i + 2] for i in range(5)]
    assert [len(step) for step in eng.log] == [2, 2, 2, 2, 1, 1]                      # prompt step, then one decode step
    assert [t for _, t in eng.log[2]] == [[2], [3]] and [t for _, t in eng.log[4]] == [[4]]
    assert {slot for step in eng.log for slot, _ in step} == {0, 1}                   # slots are used again
    assert not eng.held
    assert s.last == ([4], [1])                                                       # request id and its step


def full_history(page):
    return lambda length: [-(-length // page)]


def test_plan_batches_respects_slots_cache_and_order():
    assert plan_batches([5, 11, 17], 8, 8, full_history(64), [64], 256) == [[0, 1, 2]]
    assert plan_batches([5, 11, 17, 3], 8, 2, full_history(64), [64], 256) == [[0, 1], [2, 3]]
    # 100+29 tokens = 3 pages of 64 each; a cache of 320 tokens (5 pages) holds one such request at a time
    assert plan_batches([100, 100, 10], 30, 8, full_history(64), [5], 256) == [[0], [1, 2]]
    with pytest.raises(ValueError, match="longest sequence"):
        plan_batches([250], 10, 8, full_history(64), [64], 256)
    with pytest.raises(ValueError, match="do not fit the cache"):
        plan_batches([200], 10, 8, full_history(64), [2], 256)
    with pytest.raises(ValueError, match="empty"):
        plan_batches([3, 0], 10, 8, full_history(64), [64], 256)


def test_plan_batches_asks_every_cache_group():
    """Two groups: one keeps every token, one a window of at most 2 pages a sequence; the fuller group decides."""
    def two_groups(length):
        return [-(-length // 64), min(-(-length // 64), 2)]
    # 5 pages each in the first group: a pool of 10 holds two requests, the windowed pool of 4 as well
    assert plan_batches([300, 300, 300], 10, 8, two_groups, [10, 4], 1000) == [[0, 1], [2]]
    # with a windowed pool of 3 only one request fits at a time although the first group has room for two
    assert plan_batches([300, 300, 300], 10, 8, two_groups, [10, 3], 1000) == [[0], [1], [2]]
    # a sequence longer than the windowed group's whole pool is fine as long as its window fits
    assert plan_batches([900], 10, 8, two_groups, [20, 2], 1000) == [[0]]


@BOTH
@pytest.mark.parametrize("fail_at", [0, 1, 2])
def test_a_failing_step_gives_the_slots_back(overlapped, fail_at):
    eng = FakeEngine(overlapped=overlapped)
    real = eng.step

    def boom(entries, device_tokens=None):
        if len(eng.log) == fail_at:
            raise RuntimeError("kernel refused")
        return real(entries, device_tokens) if overlapped else real(entries)
    eng.step = boom
    with pytest.raises(RuntimeError):
        generate(eng, [[1], [2]], 4, sampler=ArgmaxSampler())
    assert not eng.held and sorted(eng.free) == [0, 1, 2, 3]


@BOTH
def test_the_sampler_sees_request_and_step_of_every_row(overlapped):
    """Request index and the count of tokens already generated key the random numbers: they must be the same in
    both loops, also for the sequences that are still running after others have left."""
    calls = []

    class Recording(ArgmaxSampler):
        def sample(self, logits, request_ids, steps):
            calls.append((list(request_ids), list(steps)))
            return super().sample(logits, request_ids, steps)
    eng = FakeEngine(overlapped=overlapped)
    outs = generate(eng, [[1, 2], [10], [30]], max_new_tokens=4, stop_token_ids=[12], sampler=Recording())
    assert [o.tokens for o in outs] == [[3, 4, 5, 6], [11, 12], [31, 32, 33, 34]]
    used = {(r, st) for ids, steps in calls for r, st in zip(ids, steps)}
    assert {(0, k) for k in range(4)} | {(1, 0), (1, 1)} | {(2, k) for k in range(4)} <= used
    # nothing is drawn for a sequence beyond the step after its stop token (overlapped) or its stop token (plain)
    assert used - {(1, 2)} == {(0, k) for k in range(4)} | {(1, 0), (1, 1)} | {(2, k) for k in range(4)}
    assert ((1, 2) in used) == overlapped


def test_display_plain_and_formatted():
    """What the command line prints beside the text (cpmcu/common/display.py:95-115, 182-260): plain mode has one
    fact a line and nothing that moves; formatted mode draws a bar in place."""
    import io
    from cpmcu_amd.utils.display import Display
    out = io.StringIO()
    d = Display(plain=True, stream=out)
    cb = d.progress_callback()
    cb("begin", {"total_tokens": 100})
    cb("advance", {"current_tokens": 40})
    cb("finish", {"total_time": 0.5})
    d.performance(100, 0.5, 20, 2.0)
    text = out.getvalue()
    assert "\r" not in text and "\033" not in text
    assert text.splitlines()[:2] == ["Prefilling: 0/100 tokens", "Prefill done: 100/100 tokens in 0.50 s"]
    assert "  Prefill Speed: 200.0 tokens/s" in text and "  Decode Speed: 10.0 tokens/s" in text
    out = io.StringIO()
    d = Display(plain=False, stream=out)
    cb = d.progress_callback()
    cb("begin", {"total_tokens": 100})
    for n in (10, 50, 100):
        cb("advance", {"current_tokens": n})
    cb("finish", {"total_time": 0.25})
    text = out.getvalue()
    assert text.count("\r") >= 3 and "[" + "#" * 15 + "." * 15 + "] 50/100 tokens" in text and "0.25 s" in text
    assert "\033" not in text                                     # colours only on a terminal

    class Args:
        model_path, dtype, nothing = "/m", "bfloat16", None
    out = io.StringIO()
    Display(plain=False, stream=out).configuration(Args, [("Model", (("model_path", "Model Path"), ("dtype", "Data Type"),
                                                                      ("nothing", "Unset"), ("absent", "Absent")))])
    text = out.getvalue()
    assert "--- Model ---" in text and "Model Path  /m" in text and "Unset" not in text and "Absent" not in text


def test_prompt_passes_are_reported_as_progress():
    """An engine that cuts the prompt step into forward passes reports each one: begin, advance ..., finish."""
    class PassingEngine(FakeEngine):
        on_pass = None

        def step(self, entries, device_tokens=None):
            out = super().step(entries)
            if self.on_pass is not None and any(len(e.tokens) > 1 for e in entries):
                total = sum(len(e.tokens) for e in entries)
                for done in range(4, total + 4, 4):
                    self.on_pass(min(done, total), total)
            return out
    events = []
    eng = PassingEngine()
    generate(eng, [[1, 2, 3, 4, 5, 6], [7, 8, 9]], 2, sampler=ArgmaxSampler(), on_prefill=lambda e, d: events.append((e, dict(d))))
    assert [e for e, _ in events] == ["begin", "advance", "advance", "advance", "finish"]
    assert events[0][1] == {"total_tokens": 9} and [d["current_tokens"] for e, d in events if e == "advance"] == [4, 8, 9]
    assert eng.on_pass is None
