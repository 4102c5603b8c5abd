"""The sequence cache's bookkeeping (CPU): no slot or page lost, held twice or freed twice."""
import random

import pytest
import torch

from cpmcu_amd.cache import CacheError, CacheNeeds, SequenceCache, StateSpec, StreamSpec

FULL = CacheNeeds(streams=(("k", StreamSpec(8)), ("v", StreamSpec(8))))
CK = CacheNeeds(streams=(("k", StreamSpec(8)), ("v", StreamSpec(8)), ("ck", StreamSpec(8, every=4))))
WIN = CacheNeeds(streams=(("k", StreamSpec(4)),), window=20)
STATE = CacheNeeds(state=(("h", StateSpec((3, 5), torch.float32)),))


def make(needs, max_tokens=256, max_slots=4, max_seq_len=128, page=16):
    return SequenceCache(needs, max_tokens, max_slots, max_seq_len, page, "cpu", torch.float32)


def test_groups_share_storage_shape_and_tables():
    c = make([FULL, FULL, CK, WIN, STATE])
    assert len(c.groups) == 4
    assert c.entry_group[0] == c.entry_group[1] != c.entry_group[2]
    v0, v2, v3, v4 = c.view(0), c.view(2), c.view(3), c.view(4)
    assert v0.streams["k"].shape == (16, 16, 8) and v2.streams["ck"].shape == (16, 4, 8)
    assert v0.page_table is c.view(1).page_table and v0.page_table is not v2.page_table
    assert v0.streams["k"] is not c.view(1).streams["k"]
    assert v3.window == 20 and v4.state["h"].shape == (4, 3, 5) and not v4.streams


def test_positions_pages_and_release():
    c = make([FULL])
    s = c.acquire()
    assert c.extend(s, 5) == 0 and c.length(s) == 5
    assert c.extend(s, 30) == 5 and c.length(s) == 35
    c.sync()
    g = c.groups[0]
    assert g.held(s) == 3 and len(g.free_pages) == 13
    assert len(set(g.table[s, :3].tolist())) == 3
    c.check()
    c.release(s)
    assert len(g.free_pages) == 16
    c.check()
    with pytest.raises(CacheError, match="not held"):
        c.release(s)
    with pytest.raises(CacheError, match="not held"):
        c.length(s)


def test_limits_are_refused_without_side_effects():
    c = make([FULL], max_tokens=64, max_slots=2, max_seq_len=40)
    a, b = c.acquire(), c.acquire()
    with pytest.raises(CacheError, match="no free slot"):
        c.acquire()
    c.extend(a, 33)                       # 3 pages of 4
    with pytest.raises(CacheError, match="longest sequence"):
        c.extend(a, 8)
    with pytest.raises(CacheError, match="cache is full"):
        c.extend(b, 17)                   # needs 2 pages, 1 is free
    assert c.length(b) == 0 and c.groups[0].held(b) == 0
    c.extend(b, 16)
    c.check()


def test_a_window_group_gives_old_pages_back():
    c = make([FULL, WIN], max_tokens=128, max_seq_len=128)
    s = c.acquire()
    c.extend(s, 100)
    for _ in range(20):
        c.extend(s, 1)
    full, win = c.groups[c.entry_group[0]], c.groups[c.entry_group[1]]
    assert full.held(s) == 8
    # position 119's window reaches back to 100 -> page 6; pages 0..5 are free again
    assert win.held(s) == 2 and win.pages[s][:6] == [-1] * 6
    c.check()
    c.release(s)
    c.check()


def test_state_is_zeroed_when_a_slot_is_taken_again():
    c = make([STATE])
    s = c.acquire()
    c.view(0).state["h"][s] = 7.0
    c.release(s)
    t = c.acquire()
    assert t == s and float(c.view(0).state["h"][t].abs().sum()) == 0.0


def test_random_walk_never_loses_anything():
    rng = random.Random(0)
    c = make([FULL, CK, WIN], max_tokens=512, max_slots=6, max_seq_len=200)
    live = []
    for _ in range(600):
        op = rng.random()
        try:
            if op < 0.25 and len(live) < 6:
                live.append(c.acquire())
            elif op < 0.8 and live:
                c.extend(rng.choice(live), rng.randint(1, 40))
            elif live:
                c.release(live.pop(rng.randrange(len(live))))
        except CacheError:
            pass
        c.check()
        for g in c.groups:
            held = [p for s in live for p in g.pages[s] if p >= 0]
            assert len(held) == len(set(held))
    for s in live:
        c.release(s)
    c.check()
    assert all(len(g.free_pages) == g.n_pages for g in c.groups) and len(c.free_slots) == 6


def test_a_windowed_sequence_may_outgrow_the_pool():
    """A group that keeps a window holds only its window's pages: a sequence longer than the whole pool fits,
    and its page table has an entry for every page number it reaches."""
    c = make([WIN], max_tokens=64, max_slots=2, max_seq_len=400, page=16)        # 4 pages in all
    s = c.acquire()
    g = c.groups[0]
    assert g.table.shape[1] == 25                                               # ceil(400 / 16)
    c.extend(s, 30)
    for _ in range(370):
        assert c.room_for([[(s, 1)]]) is None
        c.extend(s, 1)
        assert g.held(s) <= 3
        c.check()
    assert c.length(s) == 400 and g.pages[s][-1] >= 0 and g.pages[s][-3] == -1
    c.sync()
    assert int(g.table[s, 24]) == g.pages[s][24]
    c.release(s)
    c.check()


def test_room_is_asked_of_every_group_and_counts_what_a_window_gives_back():
    c = make([FULL, WIN], max_tokens=64, max_slots=2, max_seq_len=400, page=16)
    a, b = c.acquire(), c.acquire()
    c.extend(a, 40)                                   # 3 of 4 pages in both groups
    assert c.room_for([[(b, 16)]]) is None
    msg = c.room_for([[(b, 17)]])                     # 2 pages: neither group has them
    assert msg is not None and "cache is full" in msg
    assert c.room_for([[(a, 24)]]) is None            # a's 4th page
    msg = c.room_for([[(a, 25)]])                     # a 5th page: the full-history group cannot, the window could
    assert msg is not None and "group 0" in msg
    assert c.room_for([[(a, 8), (b, 16)]]) is None and c.room_for([[(a, 8)], [(b, 17)]]) is not None
    assert c.pages_to_hold(400, 1) == [25, 3] and c.pages_to_hold(400, 64) == [25, 7]
    assert c.pages_to_hold(20, 64) == [2, 2] and c.capacity() == [4, 4]
    with pytest.raises(CacheError):
        c.extend(a, 25)
    assert c.length(a) == 40
    c.check()


def test_a_long_prompt_in_passes_fits_a_windowed_pool():
    """What room_for plays through is what extend then does: a windowed group takes 300 tokens in passes of 32
    (2 new pages beside the 2 a window of 20 still touches) through a pool of 4 pages, but not in one pass."""
    c = make([WIN], max_tokens=64, max_slots=2, max_seq_len=400, page=16)
    s = c.acquire()
    passes = [[(s, 32)] for _ in range(9)] + [[(s, 12)]]
    assert c.room_for(passes) is None
    assert c.room_for([[(s, 64)], [(s, 64)]]) is not None          # the second pass would need 6 pages
    assert c.room_for([[(s, 300)]]) is not None
    for (slot, n), in passes:
        c.extend(slot, n)
        c.check()
    assert c.length(s) == 300 and c.groups[0].held(s) <= 4
    # a second sequence beside it: one page is left for it, not two
    t = c.acquire()
    assert c.room_for([[(t, 16)]]) is None or c.groups[0].held(s) == 4
    c.release(s)
    c.release(t)
    c.check()


def test_truncate_gives_the_tail_back():
    c = make([FULL, CK], max_tokens=128, max_slots=2, max_seq_len=128, page=16)
    s = c.acquire()
    c.extend(s, 20)
    free = [len(g.free_pages) for g in c.groups]
    c.extend(s, 50)
    c.truncate(s, 20)
    assert c.length(s) == 20 and [len(g.free_pages) for g in c.groups] == free
    c.check()
    assert c.extend(s, 3) == 20
    with pytest.raises(CacheError):
        c.truncate(s, 24)
    c.truncate(s, 0)
    assert all(len(g.free_pages) == g.n_pages for g in c.groups)
    c.check()


def test_truncate_below_what_a_window_gave_back_is_refused():
    """Going back is only safe to a length whose next query reads no page that the group already gave back
    (the start of the last extend always is one)."""
    c = make([FULL, WIN], max_tokens=256, max_slots=2, max_seq_len=128)
    s = c.acquire()
    c.extend(s, 40)
    c.extend(s, 50)                      # the windowed group keeps from position 40 - 20 + 1 = 21 on: page 0 goes
    win = c.groups[1]
    assert win.pages[s][0] == -1 and win.pages[s][1] >= 0
    free = [len(g.free_pages) for g in c.groups]
    with pytest.raises(CacheError, match="has already given back page 0"):
        c.truncate(s, 30)                # the query at 30 reads back to 11, which lay in page 0
    assert c.length(s) == 90 and [len(g.free_pages) for g in c.groups] == free
    c.truncate(s, 40)                    # the engine's roll-back: the start of the last extend
    assert c.length(s) == 40
    c.check()
    c.extend(s, 50)
    c.check()


def test_planned_bytes_equal_built_bytes_and_window_pools_are_small():
    needs = [FULL, FULL, CK, WIN, STATE]
    for max_tokens, slots, seq, step in ((256, 4, 128, None), (1024, 3, 512, 32), (64, 2, 40, 7)):
        c = SequenceCache(needs, max_tokens, slots, seq, 16, "cpu", torch.float32, step)
        tables = sum(g.table.numel() * 4 for g in c.groups)
        plan = SequenceCache.plan_bytes(needs, max_tokens, slots, seq, 16, torch.float32, step)
        assert plan == c.bytes() + tables
    # the windowed group's pool holds its window for every slot, not a page for every token of the cache
    c = SequenceCache([FULL, WIN], 4096, 3, 2048, 16, "cpu", torch.float32, 32)
    assert c.groups[0].n_pages == 256 and c.groups[1].n_pages == 3 * ((32 + 20 - 2) // 16 + 2)
    assert c.pages_to_hold(2048, 32) == [128, (32 + 20 - 2) // 16 + 2]
    # and a walk at that step never finds the small pool empty
    slots = [c.acquire() for _ in range(3)]
    for _ in range(40):
        for s in slots:
            c.extend(s, 32)
    c.check()
    # the most tokens for a budget: the plan of the answer fits, one page more does not
    for budget in (10_000, 100_000, 1_000_000):
        t = SequenceCache.tokens_for(needs, budget, 4, 512, 16, torch.float32, 32)
        if t:
            assert SequenceCache.plan_bytes(needs, t, 4, 512, 16, torch.float32, 32) <= budget
            assert t == 4 * 512 or SequenceCache.plan_bytes(needs, t + 16, 4, 512, 16, torch.float32, 32) > budget
    assert SequenceCache.tokens_for(needs, 100, 4, 512, 16, torch.float32, 32) == 0


def test_state_snapshot_and_restore():
    c = make([FULL, STATE])
    assert c.has_state and not make([FULL]).has_state and make([FULL]).snapshot_state([0]) is None
    a, b = c.acquire(), c.acquire()
    h = c.view(1).state["h"]
    h[a] = 1.5
    h[b] = -2.0
    snap = c.snapshot_state([b])
    h[a] = 7.0
    h[b] = 9.0
    c.restore_state(snap)
    assert float(h[b].min()) == float(h[b].max()) == -2.0 and float(h[a].min()) == 7.0
