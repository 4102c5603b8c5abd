"""The attention and block-selection kernels at the context lengths they serve: thousands to tens of thousands
of keys, many shares, lookups of more than one batch of chunks a wavefront, long block lists (GPU).

Random scores over thousands of keys are diffuse: a skipped chunk of 32 keys would move the output by less than
its rounding.  So besides the comparison with a float64 reference, single keys are made to stand out (a query
and one key scaled so that this key takes nearly all the weight) at the places where an index could go wrong:
the first and last chunk of every batch of 64 chunk lookups of a wavefront, the first and last key of a share,
the first and last page."""
import pytest
import torch

from test_kernels_gpu import DEV, key_elements, key_tiles, rnd, value_tiles

pytestmark = pytest.mark.gpu
PAGE = 64


def long_paged(L, nkv, hd, seed, spare_pages=5):
    """One sequence of L random bf16 keys and values in a paged cache with scrambled pages, built on the GPU.
    Returns K, V as float64 [L, nkv, hd] and the pools / page table as the kernels take them."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    n_pages = -(-L // PAGE)
    Lp = n_pages * PAGE
    k = torch.randn(Lp, nkv, hd, generator=g).to(torch.bfloat16).to(DEV)
    v = torch.randn(Lp, nkv, hd, generator=g).to(torch.bfloat16).to(DEV)
    k[L:] = 0
    v[L:] = 0
    total = n_pages + spare_pages
    perm = torch.randperm(total, generator=g)[:n_pages].to(DEV)
    kpool = torch.zeros(total, PAGE, nkv * hd, dtype=torch.bfloat16, device=DEV)
    vpool = torch.zeros_like(kpool)
    kpool[perm] = key_tiles(k).reshape(n_pages, PAGE, nkv * hd)
    vpool[perm] = value_tiles(v).reshape(n_pages, PAGE, nkv * hd)
    table = perm.to(torch.int32).view(1, n_pages).contiguous()
    return k[:L].double(), v[:L].double(), kpool, vpool, table


def reference(q, K, V, positions, nh, scale, allowed=None):
    """float64 attention on the GPU: q [n, nh, hd]; query t sees keys 0..positions[t] (of `allowed[t][kv head]`)."""
    nkv = K.shape[1]
    G = nh // nkv
    out = torch.empty(q.shape, dtype=torch.float64, device=DEV)
    for t, p in enumerate(positions):
        for h in range(nkv):
            s = torch.einsum("ld,gd->gl", K[:p + 1, h], q[t, h * G:(h + 1) * G].double()) * scale
            if allowed is not None:
                s = s.masked_fill(~allowed[t][h][:p + 1], float("-inf"))
            out[t, h * G:(h + 1) * G] = torch.softmax(s, 1) @ V[:p + 1, h]
    return out


def close(out, ref, what):
    """bf16 output (8 significant bits) against the reference, relative to each token's largest value."""
    n = ref.shape[0]
    err = (out.double().view(ref.shape) - ref).abs().reshape(n, -1).amax(1)
    lim = 2 ** -7 * ref.abs().reshape(n, -1).amax(1) + 1e-4
    bad = (err > lim).nonzero().flatten()
    assert bad.numel() == 0, f"{what}: first wrong token {int(bad[0])}: error {float(err[bad[0]]):.3g} > {float(lim[bad[0]]):.3g}"


def run_mfma(ops, q, nh, nkv, hd, kpool, vpool, table, positions, splits, nw, sel=None, first=0):
    n = q.shape[0]
    pos_t = torch.tensor(positions, dtype=torch.int32, device=DEV)
    slot_t = torch.zeros(n, dtype=torch.int32, device=DEV)
    out = torch.full((n, nh * hd), float("nan"), dtype=torch.bfloat16, device=DEV)
    po = torch.full((n, nh, splits, hd), float("nan"), device=DEV) if splits > 1 else None
    pm = torch.full((n, nh, splits, 2), float("nan"), device=DEV) if splits > 1 else None
    sb, sc, bs = sel if sel is not None else (None, None, 0)
    ops.attention_mfma(q.view(n, -1), out, nh, nkv, hd, hd ** -0.5, kpool, vpool, table, PAGE, pos_t, slot_t, splits, po, pm,
                       sb, sc, bs, waves_per_group=nw, last_blocks_first=first)
    return out


def edge_keys(L, splits, nw):
    """Keys at which an index of the kernel's chunk walk could slip: for the first and the last share, for each
    wavefront, the first and last key of its chunks number 0, 63, 64, 127, 128 (the edges of the batches of 64
    lookups) and of its last chunk; the sequence's first and last key."""
    total = (L - 1) // 32 + 1
    per = -(-total // splits)
    keys = {0, L - 1}
    for split in {0, splits - 1, splits // 2}:
        c0, c1 = split * per, min(split * per + per, total)
        for wave in range(nw):
            mine = list(range(c0 + wave, c1, nw))
            for kj in (0, 63, 64, 127, 128, len(mine) - 1):
                if 0 <= kj < len(mine):
                    keys.update((mine[kj] * 32, min(mine[kj] * 32 + 31, L - 1)))
    return sorted(k for k in keys if k < L)


@pytest.mark.parametrize("L,nh,nkv,hd,shapes", [
    (9000, 8, 2, 32, ((1, 1), (1, 4), (16, 4), (32, 4), (16, 1))),
    (20000, 4, 1, 32, ((1, 1), (1, 4), (16, 4), (32, 4), (32, 1))),
    (4100, 32, 2, 128, ((8, 4), (16, 4))),
    (16400, 32, 2, 128, ((1, 4), (8, 4), (16, 4), (32, 4), (48, 4))),
    (33000, 32, 2, 128, ((16, 4), (32, 4), (8, 1), (64, 4))),
])
def test_decode_attention_over_long_contexts(L, nh, nkv, hd, shapes):
    """One and two tokens over thousands of keys: 1 to 64 shares (every form of the merge kernel), 1 and 4 wavefronts a workgroup, wavefronts
    with more than 64 and more than 128 chunks; random queries against the float64 reference, then one
    outstanding key at a time at the edges of the walk."""
    from cpmcu_amd import ops
    K, V, kpool, vpool, table = long_paged(L, nkv, hd, seed=L)
    positions = [L - 1, L - 34]
    q = rnd(2, nh, hd, seed=7, dtype=torch.bfloat16)
    ref = reference(q, K, V, positions, nh, hd ** -0.5)
    for splits, nw in shapes:
        close(run_mfma(ops, q, nh, nkv, hd, kpool, vpool, table, positions, splits, nw), ref, f"{splits} shares, {nw} waves")
    # one outstanding key: every head's output must be that key's value
    qf = torch.zeros(1, nh, hd, dtype=torch.bfloat16, device=DEV)
    qf[0, :, 5] = 48.0
    one = torch.zeros(hd, dtype=torch.bfloat16, device=DEV)
    one[5] = 48.0
    for splits, nw in shapes:
        for far in edge_keys(L, splits, nw):
            pg, off = int(table[0, far // PAGE]), far % PAGE
            saved = []
            for h in range(nkv):
                where = key_elements(off, h, nkv, hd, PAGE).to(DEV)
                flat = kpool[pg].view(-1)
                saved.append((where, flat[where].clone()))
                flat[where] = one
            out = run_mfma(ops, qf, nh, nkv, hd, kpool, vpool, table, [L - 1], splits, nw).double().view(nh, hd)
            want = V[far].repeat_interleave(nh // nkv, 0)
            for where, old in saved:
                kpool[pg].view(-1)[where] = old
            assert float((out - want).abs().max()) < 2e-2, f"key {far} of {L}, {splits} shares, {nw} waves"


def random_block_lists(positions, nkv, bs, n_top, n_window, seed):
    """Ascending block lists: n_top random earlier blocks, then the n_window blocks up to the query's own."""
    g = torch.Generator().manual_seed(seed)
    n = len(positions)
    max_sel = n_top + n_window
    sb = torch.zeros(n, nkv, max_sel, dtype=torch.int32)
    sc = torch.zeros(n, nkv, dtype=torch.int32)
    for t, p in enumerate(positions):
        own = p // bs
        first_w = max(own - n_window + 1, 0)
        for h in range(nkv):
            top = sorted(torch.randperm(first_w, generator=g)[:n_top].tolist()) if first_w > 0 else []
            blocks = top + list(range(first_w, own + 1))
            sc[t, h] = len(blocks)
            sb[t, h, :len(blocks)] = torch.tensor(blocks, dtype=torch.int32)
    return sb, sc


def allowed_from_lists(sb, sc, bs, L):
    n, nkv, _ = sb.shape
    allowed = torch.zeros(n, nkv, L, dtype=torch.bool)
    for t in range(n):
        for h in range(nkv):
            for b in sb[t, h, :int(sc[t, h])].tolist():
                allowed[t, h, b * bs:(b + 1) * bs] = True
    return allowed.to(DEV)


@pytest.mark.parametrize("L,nh,nkv,hd", [(33000, 32, 2, 128), (20000, 6, 2, 32)])
def test_block_list_attention_with_long_lists(L, nh, nkv, hd):
    """Lists of 96 chosen + 32 window blocks of 64 keys (256 chunks: four batches of lookups for a lone
    wavefront): steps of few tokens with shares, and a run of prompt tokens a wavefront each, window first."""
    from cpmcu_amd import ops
    bs = 64
    K, V, kpool, vpool, table = long_paged(L, nkv, hd, seed=L + 1)
    # few tokens (decode steps)
    positions = [L - 1, L - 70, 9000]
    sb, sc = random_block_lists(positions, nkv, bs, 96, 32, seed=3)
    q = rnd(len(positions), nh, hd, seed=9, dtype=torch.bfloat16)
    ref = reference(q, K, V, positions, nh, hd ** -0.5, allowed_from_lists(sb, sc, bs, L))
    for splits, nw in ((1, 1), (1, 4), (8, 4), (16, 4)):
        out = run_mfma(ops, q, nh, nkv, hd, kpool, vpool, table, positions, splits, nw, (sb.to(DEV), sc.to(DEV), bs))
        close(out, ref, f"lists, {splits} shares, {nw} waves")
    # a chunk of a prompt: 70 consecutive tokens, a wavefront each, four a workgroup, the window visited first
    positions = list(range(L - 70, L))
    sb, sc = random_block_lists(positions, nkv, bs, 96, 32, seed=4)
    q = rnd(len(positions), nh, hd, seed=10, dtype=torch.bfloat16)
    ref = reference(q, K, V, positions, nh, hd ** -0.5, allowed_from_lists(sb, sc, bs, L))
    for first in (0, 32):
        out = run_mfma(ops, q, nh, nkv, hd, kpool, vpool, table, positions, 1, 0, (sb.to(DEV), sc.to(DEV), bs), first=first)
        close(out, ref, f"prompt tokens with lists, window first {first}")


class _Ctx:
    """What ops.attention reads of a step."""

    def __init__(self, q_lens, positions, max_pos, single):
        from cpmcu_amd.parts.base import Workspace
        self.q_lens, self.max_pos, self.single_token = q_lens, max_pos, single
        self.positions = torch.tensor(positions, dtype=torch.int32, device=DEV)
        self.tok_slot = torch.zeros(len(positions), dtype=torch.int32, device=DEV)
        self.extras = {}
        self.ws = Workspace(DEV)


@pytest.mark.parametrize("n_tokens,start", [(1100, 0), (16500, 0), (2048, 14000), (700, 3000)])
@pytest.mark.parametrize("nh,nkv,hd", [(8, 2, 32), (32, 2, 128), (4, 1, 128)])
def test_prompt_attention_of_long_prompts_through_the_dispatcher(n_tokens, start, nh, nkv, hd):
    """Whole prompts on either side of the sizes where the dispatcher changes the kernel's shape (1,024 and
    16,384 tokens), and chunks that continue a long sequence: tokens at the edges of tiles, pages and the
    prompt against the float64 reference."""
    from cpmcu_amd import ops
    if n_tokens > 4096 and hd == 128 and nh > 4:
        pytest.skip("this length at the head size of 128 runs with 4 heads (the next parameters)")
    L = start + n_tokens
    K, V, kpool, vpool, table = long_paged(L, nkv, hd, seed=n_tokens + hd)
    positions = list(range(start, L))
    q = rnd(n_tokens, nh, hd, seed=2, dtype=torch.bfloat16)
    out = torch.full((n_tokens, nh * hd), float("nan"), dtype=torch.bfloat16, device=DEV)
    ctx = _Ctx([n_tokens], positions, L - 1, False)
    assert ops.attention(q.view(n_tokens, -1), out, nh, nkv, hd, hd ** -0.5, kpool, vpool, table, PAGE, ctx) is None
    assert not bool(out.isnan().any())
    probe = sorted({0, 1, 15, 16, 31, 32, 63, 64, 65, 127, 128, 1023, 1024, 1025, 2047, 4095, 4096, 8191, 8192,
                    16383, 16384, n_tokens // 2, n_tokens - 65, n_tokens - 33, n_tokens - 2, n_tokens - 1}
                   & set(range(n_tokens)))
    ref = reference(q[probe], K, V, [start + i for i in probe], nh, hd ** -0.5)
    close(out[probe], ref, f"prompt of {n_tokens} tokens from {start}")


def compressed_cache(L, nkv, hd, ks, st, seed):
    from cpmcu_amd import ops
    K, V, kpool, vpool, table = long_paged(L, nkv, hd, seed=seed)
    ck = torch.zeros(kpool.shape[0], PAGE // st, nkv * hd, dtype=torch.bfloat16, device=DEV)
    ops.compress_keys(kpool, ck, nkv, table, PAGE, torch.arange(L, dtype=torch.int32, device=DEV),
                      torch.zeros(L, dtype=torch.int32, device=DEV), ks, st)
    return ck, table


def select(ops, q, ck, table, nh, nkv, hd, positions, sp, max_pos, force_plain, scratch):
    ks, st, bs, init, topk, window, dense_len = sp
    n = q.shape[0]
    lb = window // bs
    sb = torch.full((n, nkv, topk + lb), -7, dtype=torch.int32, device=DEV)
    sc = torch.full((n, nkv), -7, dtype=torch.int32, device=DEV)
    if scratch is None and force_plain is True:
        # the plain kernel needs scratch only where its arrays exceed a workgroup's LDS
        need = ops.sparse_select_scratch(q.dtype, n, nh, nkv, hd, max_pos, ks, st, bs, force_plain=True)
        scratch = torch.full((need,), float("nan"), device=DEV) if need else None
    ops.sparse_select(q.view(n, -1), ck, nh, nkv, hd, hd ** -0.5, table, PAGE,
                      torch.tensor(positions, dtype=torch.int32, device=DEV), torch.zeros(n, dtype=torch.int32, device=DEV),
                      ks, st, bs, init, topk, lb, dense_len, max_pos, sb, sc, force_plain, scratch=scratch)
    return sb.cpu(), sc.cpu()


@pytest.mark.parametrize("L,nh,nkv,hd,sp", [
    (33000, 32, 2, 128, (32, 16, 64, 1, 64, 2048, 8192)),
    (60000, 8, 2, 32, (32, 16, 64, 1, 16, 512, 1000)),
    (20000, 6, 1, 32, (8, 4, 16, 2, 24, 64, 0)),
])
def test_block_selection_at_long_contexts_in_all_its_forms(L, nh, nkv, hd, sp):
    """Tens of thousands of positions, i.e. hundreds of groups of 64 compressed keys and up to a thousand
    candidate blocks: the fused matrix-core kernel, the kernels of steps of few tokens (with and without the
    separate normalising kernel) and the plain kernel must list the same blocks; the bound of the launch
    (max_pos) may lie beyond the step's positions, as under a captured graph."""
    from cpmcu_amd import ops
    ks, st, bs, init, topk, window, dense_len = sp
    ck, table = compressed_cache(L, nkv, hd, ks, st, seed=L + 2)
    positions = [L - 1, L - 2, L - bs, L // 2 + 3, dense_len + 1, 5000]
    q = rnd(len(positions), nh, hd, seed=6, dtype=torch.bfloat16)
    for max_pos in (L - 1, min(2 * L, 65535) if L < 65536 else L - 1):
        want_b, want_c = select(ops, q, ck, table, nh, nkv, hd, positions, sp, max_pos, True, None)
        for t, p in enumerate(positions):               # -1: the position lies within dense_len
            assert all((c == -1) if p + 1 <= dense_len else (0 < c <= topk + window // bs) for c in want_c[t].tolist()), p
        scratch = torch.full((ops.sparse_select_scratch(torch.bfloat16, len(positions), nh, nkv, hd, max_pos, ks, st, bs),), float("nan"), device=DEV)
        # the fused kernel serves steps of many tokens: the same queries over and over, 264 tokens in all (its
        # scores and ranking arrays move to scratch rows where they exceed LDS)
        reps = -(-264 // len(positions))
        many_q, many_pos = q.repeat(reps, 1, 1), positions * reps
        need = ops.sparse_select_scratch(torch.bfloat16, len(many_pos), nh, nkv, hd, max_pos, ks, st, bs)
        many_scr = torch.full((need,), float("nan"), device=DEV) if need else None
        for force, scr, what in ((False, None, "fused"), (False, scratch, "few tokens"), (2, scratch, "few tokens, normalised apart")):
            if what == "fused":
                got_b, got_c = select(ops, many_q, ck, table, nh, nkv, hd, many_pos, sp, max_pos, force, many_scr)
                assert torch.equal(got_c[:len(positions)], got_c[-len(positions):])
                got_b, got_c = got_b[:len(positions)], got_c[:len(positions)]
            else:
                got_b, got_c = select(ops, q, ck, table, nh, nkv, hd, positions, sp, max_pos, force, scr)
            assert torch.equal(got_c, want_c), (what, max_pos, got_c.tolist(), want_c.tolist())
            for t in range(len(positions)):
                for h in range(nkv):
                    c = int(want_c[t, h])
                    assert got_b[t, h, :c].tolist() == want_b[t, h, :c].tolist(), (what, max_pos, positions[t], h)


def test_block_selection_finds_one_far_block():
    """One compressed key far back is made to match the query: its block must be chosen, wherever it lies among
    the groups of 64 compressed keys (first and last of a group, first and last visible)."""
    from cpmcu_amd import ops
    L, nh, nkv, hd = 40000, 4, 1, 32
    sp = (32, 16, 64, 1, 4, 128, 0)
    ks, st, bs, init, topk, window, dense_len = sp
    ck, table = compressed_cache(L, nkv, hd, ks, st, seed=77)
    p = L - 1
    n_vis = (p - ks) // st + 1
    q = torch.zeros(1, nh, hd, dtype=torch.bfloat16, device=DEV)
    q[0, :, 3] = 30.0
    one = torch.zeros(hd, dtype=torch.bfloat16, device=DEV)
    one[3] = 30.0
    rpp = PAGE // st
    scratch = torch.zeros(ops.sparse_select_scratch(torch.bfloat16, 1, nh, nkv, hd, p, ks, st, bs), device=DEV)
    n_cand = p // bs - window // bs + 1
    for j in (5, 63, 64, 65, 1023, 1024, n_vis // 2, n_vis - 200, n_cand * (bs // st) - 1):
        pg, row = int(table[0, (st * j) // PAGE]), ((st * j) % PAGE) // st
        view = ck[pg].view(nkv, hd // 8, rpp, 8)
        saved = view[0, :, row].clone()
        view[0, :, row] = one.view(hd // 8, 8)
        # the blocks that compressed key j (keys st*j .. st*j+ks-1) overlaps
        blocks = set(range((st * j) // bs, (st * j + ks - 1) // bs + 1))
        for force, scr in ((True, None), (False, None), (False, scratch), (2, scratch)):
            sb, sc = select(ops, q, ck, table, nh, nkv, hd, [p], sp, p, force, scr)
            chosen = set(sb[0, 0, :int(sc[0, 0])].tolist())
            assert blocks & set(range(n_cand)) <= chosen, (j, force, scr is not None, sorted(chosen)[:8])
        view[0, :, row] = saved


# ---------------------------------------------------------------------------- the engine far beyond what LDS holds
def _long_model(tmp_path):
    import tiny
    raw = tiny.tiny_b()
    raw["max_position_embeddings"] = 131072
    d = str(tmp_path / "tiny_b_long")
    tiny.write_model(raw, d, seed=77)
    return raw, d


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_engine_selects_blocks_at_position_70000(tmp_path, dtype):
    """A model that allows 131,072 positions (compressed keys every 4 tokens, blocks of 16: 17,500 scores and
    4,375 candidate blocks at position 70,000, several times what a workgroup's LDS holds).  The same tokens
    as one long prompt, and with their last tokens fed one by one (bfloat16: from a captured graph, whose
    launches are sized for 131,072 positions), must give the same logits."""
    from cpmcu_amd import Engine, EngineOptions, StepEntry
    import tiny
    raw, d = _long_model(tmp_path)
    n, tail = 70016, 6
    toks = tiny.random_tokens(n, raw["vocab_size"], 5)
    common = dict(dtype=dtype, max_tokens=n + 64, max_slots=1, max_seq_len=131072, max_step_tokens=4096)
    whole = Engine.from_dir(d, EngineOptions(**common))
    s = whole.acquire()
    ref = whole.step([StepEntry(s, toks, list(range(n - tail, n)))]).cpu()
    whole.release(s)
    del whole
    assert bool(torch.isfinite(ref).all())
    eng = Engine.from_dir(d, EngineOptions(hip_graph=(dtype == "bfloat16"), **common))
    s = eng.acquire()
    eng.step([StepEntry(s, toks[:n - tail], [])])
    rows = [eng.step([StepEntry(s, [t], [0])]).cpu() for t in toks[n - tail:]]
    assert eng.length(s) == n
    eng.release(s)
    got = torch.cat(rows)
    tol = 2e-5 if dtype == "float32" else 0.02 * float(ref.abs().max())
    err = (got - ref).abs().amax(1)
    assert float(err.max()) <= tol, f"first wrong position {n - tail + int((err > tol).nonzero()[0])}: {float(err.max()):.3g} > {tol:.3g}"
