"""Each part of a layer alone against its plain formula (GPU)."""
import math

import pytest
import torch
import torch.nn.functional as F

import plain_minicpm as plain

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


def make_ctx(needs, seqs, dtype, page=64, max_slots=4, start=None):
    """A StepContext for sequences (lists of token ids) that each bring all their tokens, over a fresh cache.
    ``start``: tokens each sequence already holds (the step's positions begin there)."""
    from cpmcu_amd.cache import SequenceCache
    from cpmcu_amd.parts import StepContext, Workspace
    cache = SequenceCache(needs, 1024, max_slots, 512, page, DEV, dtype)
    tok, pos, tslot, cu, sslot, slen = [], [], [], [0], [], []
    for i, toks in enumerate(seqs):
        s = cache.acquire()
        if start and start[i]:
            cache.extend(s, start[i])
        first = cache.extend(s, len(toks))
        tok += toks
        pos += list(range(first, first + len(toks)))
        tslot += [s] * len(toks)
        cu.append(len(tok))
        sslot.append(s)
        slen.append(first + len(toks))
    cache.sync()
    t = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    return StepContext(n_tokens=len(tok), n_seqs=len(seqs), token_ids=t(tok), positions=t(pos), tok_slot=t(tslot),
                       cu_q=t(cu), seq_slot=t(sslot), seq_len=t(slen), q_lens=[len(s) for s in seqs], kv_lens=slen,
                       max_pos=max(pos), single_token=all(len(s) == 1 for s in seqs), ws=Workspace(DEV), cache=cache)


def runtime(dtype, max_seq_len=512):
    from cpmcu_amd.parts import Runtime, Workspace
    return Runtime(DEV, dtype, Workspace(DEV), max_seq_len)


def rnd(*shape, seed=0, scale=1.0):
    return (torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale)


DTYPES = [torch.float32, torch.bfloat16]


def tol_for(dtype, ref):
    return 1e-5 * float(ref.abs().max() + 1) if dtype == torch.float32 else 2 ** -6 * float(ref.abs().max())


@pytest.mark.parametrize("dtype", DTYPES)
def test_embedding_and_head(dtype):
    from cpmcu_amd.parts import LMHead, TokenEmbedding
    E = rnd(50, 24, seed=1).bfloat16()
    emb = TokenEmbedding("e", 50, 24, scale=7.0)
    head_tied = LMHead("h", 50, 24, scale=0.25, tied_to=emb)
    head = LMHead("h", 50, 24, scale=0.25)
    Hw = rnd(50, 24, seed=2).bfloat16()
    rt = runtime(dtype)
    for p in (emb, head_tied, head):
        p.bind({"e": E.to(DEV), "h": Hw.to(DEV)}, rt)
    assert [s.name for s in head_tied.weight_specs()] == [] and [s.name for s in head.weight_specs()] == ["h"]
    ctx = make_ctx([], [[3, 49, 0, 3]], dtype)
    x = emb.forward(ctx)
    assert torch.equal(x.cpu(), E.float()[[3, 49, 0, 3]] * 7.0)
    y = rnd(4, 24, seed=3).to(dtype).to(DEV)
    ref_t = 0.25 * (y.double().cpu() @ E.double().T)                     # the tied head reads the unscaled table
    ref_u = 0.25 * (y.double().cpu() @ Hw.double().T)
    assert float((head_tied.forward(y, ctx).double().cpu() - ref_t).abs().max()) < 1e-4
    assert float((head.forward(y, ctx).double().cpu() - ref_u).abs().max()) < 1e-4


@pytest.mark.parametrize("dtype", DTYPES)
def test_norm_part_adds_the_pending_branch(dtype):
    from cpmcu_amd.parts import NORMS
    norm = NORMS.build("rms_norm", name="n", hidden_size=40, eps=1e-5)
    w = (1 + 0.1 * rnd(40, seed=1)).bfloat16()
    norm.bind({"n": w.to(DEV)}, runtime(dtype))
    ctx = make_ctx([], [[1, 2, 3]], dtype)
    x0, b = rnd(3, 40, seed=2), rnd(3, 40, seed=3)
    x = x0.to(DEV).clone()
    out = norm.forward(x, b.to(DEV), 0.3, ctx)
    xs = x0.double() + 0.3 * b.double()
    ref = plain.rms_norm(xs, w.double(), 1e-5)
    assert float((x.double().cpu() - xs).abs().max()) < 1e-6
    assert out.dtype == dtype and float((out.double().cpu() - ref).abs().max()) < tol_for(dtype, ref)


@pytest.mark.parametrize("dtype", DTYPES)
def test_rotary_parts_choose_factors_and_magnitude(dtype):
    from cpmcu_amd.parts import POSITION_ENCODINGS
    short, long_ = [1.0 + 0.1 * i for i in range(8)], [2.0 + 0.2 * i for i in range(8)]
    cfg = {"hidden_size": 16, "num_attention_heads": 1, "rope_theta": 5000.0, "max_position_embeddings": 512,
           "rope_scaling": {"rope_type": "longrope", "short_factor": short, "long_factor": long_,
                            "original_max_position_embeddings": 128}}
    for max_seq_len in (128, 129, 512):
        pe = POSITION_ENCODINGS.build("longrope", head_dim=16, theta=5000.0, short_factor=short, long_factor=long_,
                                      original_max_position=128, max_position=512)
        pe.bind({}, runtime(dtype, max_seq_len))
        inv, m = pe.rotary_params()
        inv_ref, m_ref = plain.rope_inv_freq(cfg, max_seq_len)
        assert torch.allclose(inv.double().cpu(), inv_ref, rtol=1e-6) and m == pytest.approx(m_ref)
    plain_pe = POSITION_ENCODINGS.build("rope", head_dim=16, theta=5000.0)
    plain_pe.bind({}, runtime(dtype))
    inv, m = plain_pe.rotary_params()
    assert m == 1.0 and torch.allclose(inv.double().cpu(), 5000.0 ** (-torch.arange(0, 16, 2).double() / 16), rtol=1e-6)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,hd", [(4, 2, 16), (3, 1, 32), (6, 6, 48)])
def test_attention_part_alone(dtype, nh, nkv, hd):
    """The dense attention mixer: projections, rotation, cache, attention, output projection; a prompt of two
    sequences in one step, then the following token of each."""
    from cpmcu_amd.parts import MIXERS, POSITION_ENCODINGS
    H = 40
    pe = POSITION_ENCODINGS.build("rope", head_dim=hd, theta=10000.0)
    mixer = MIXERS.build("gqa_attention", prefix="a.", hidden_size=H, num_heads=nh, num_kv_heads=nkv, head_dim=hd,
                         position=pe)
    w = {"a.q_proj.weight": rnd(nh * hd, H, seed=1, scale=0.2), "a.k_proj.weight": rnd(nkv * hd, H, seed=2, scale=0.2),
         "a.v_proj.weight": rnd(nkv * hd, H, seed=3, scale=0.2), "a.o_proj.weight": rnd(H, nh * hd, seed=4, scale=0.2)}
    w = {k: v.bfloat16() for k, v in w.items()}
    assert {s.name: s.shape for s in mixer.all_weight_specs()} == {k: tuple(v.shape) for k, v in w.items()}
    rt = runtime(dtype)
    mixer.bind_all({k: v.to(DEV) for k, v in w.items()}, rt)
    lens = [70, 9]
    hs = [rnd(L + 1, H, seed=10 + i).to(dtype) for i, L in enumerate(lens)]
    cfg = {"hidden_size": H, "num_attention_heads": nh, "num_key_value_heads": nkv, "head_dim": hd, "rope_theta": 10000.0,
           "max_position_embeddings": 512}
    inv, m = plain.rope_inv_freq(cfg)
    wd = {"x.self_attn." + k[2:]: v.double() for k, v in w.items()}
    refs = [plain.attention_layer(cfg, wd, "x.", h.double(), torch.arange(h.shape[0]), inv, m) for h in hs]
    ctx = make_ctx([mixer.cache_needs()], [[0] * L for L in lens], dtype)
    h_in = torch.cat([h[:L] for h, L in zip(hs, lens)]).to(DEV)
    out = mixer.forward(h_in, ctx, ctx.cache.view(0))
    out = out.sum(0) if out.dim() == 3 else out
    ref = torch.cat([r[:L] for r, L in zip(refs, lens)])
    assert float((out.double().cpu() - ref).abs().max()) < tol_for(dtype, ref)
    # one more token each, from the cache
    cache = ctx.cache
    from cpmcu_amd.parts import StepContext
    firsts = [cache.extend(s, 1) for s in (0, 1)]
    cache.sync()
    t = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    ctx2 = StepContext(n_tokens=2, n_seqs=2, token_ids=t([0, 0]), positions=t(firsts), tok_slot=t([0, 1]),
                       cu_q=t([0, 1, 2]), seq_slot=t([0, 1]), seq_len=t([f + 1 for f in firsts]), q_lens=[1, 1],
                       kv_lens=[f + 1 for f in firsts], max_pos=max(firsts), single_token=True, ws=ctx.ws, cache=cache)
    h2 = torch.stack([hs[0][lens[0]], hs[1][lens[1]]]).to(DEV)
    out2 = mixer.forward(h2, ctx2, cache.view(0))
    out2 = out2.sum(0) if out2.dim() == 3 else out2
    ref2 = torch.stack([refs[0][lens[0]], refs[1][lens[1]]])
    assert float((out2.double().cpu() - ref2).abs().max()) < tol_for(dtype, ref)


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_layer_can_read_the_cache_another_layer_wrote(dtype):
    """writes_cache=False: only queries are projected; keys and values are those of the entry given."""
    from cpmcu_amd.parts import MIXERS, POSITION_ENCODINGS
    H, nh, nkv, hd = 32, 4, 2, 16
    def build(prefix):
        return MIXERS.build("gqa_attention", prefix=prefix, hidden_size=H, num_heads=nh, num_kv_heads=nkv, head_dim=hd,
                            position=POSITION_ENCODINGS.build("rope", head_dim=hd, theta=10000.0))
    a, b = build("a."), build("b.")
    w = {}
    for i, p in enumerate(("a.", "b.")):
        w.update({p + "q_proj.weight": rnd(nh * hd, H, seed=i * 10 + 1, scale=0.2), p + "k_proj.weight": rnd(nkv * hd, H, seed=i * 10 + 2, scale=0.2),
                  p + "v_proj.weight": rnd(nkv * hd, H, seed=i * 10 + 3, scale=0.2), p + "o_proj.weight": rnd(H, nh * hd, seed=i * 10 + 4, scale=0.2)})
    w = {k: v.bfloat16() for k, v in w.items()}
    rt = runtime(dtype)
    for m_ in (a, b):
        m_.bind_all({k: v.to(DEV) for k, v in w.items()}, rt)
    L = 20
    h = rnd(L, H, seed=5).to(dtype)
    ctx = make_ctx([a.cache_needs()], [[0] * L], dtype)
    a.forward(h.to(DEV), ctx, ctx.cache.view(0))                           # writes entry 0
    out = b.forward(h.to(DEV), ctx, ctx.cache.view(0), writes_cache=False)
    out = out.sum(0) if out.dim() == 3 else out
    # plain: b's queries against a's keys and values
    cfg = {"hidden_size": H, "num_attention_heads": nh, "num_key_value_heads": nkv, "head_dim": hd, "rope_theta": 10000.0,
           "max_position_embeddings": 512}
    inv, m = plain.rope_inv_freq(cfg)
    hd_ = h.double()
    q = plain.apply_rope((hd_ @ w["b.q_proj.weight"].double().T).view(L, nh, hd), torch.arange(L), inv, m)
    k = plain.apply_rope((hd_ @ w["a.k_proj.weight"].double().T).view(L, nkv, hd), torch.arange(L), inv, m)
    v = (hd_ @ w["a.v_proj.weight"].double().T).view(L, nkv, hd)
    ref = plain.dense_attention(q, k, v).reshape(L, nh * hd) @ w["b.o_proj.weight"].double().T
    assert float((out.double().cpu() - ref).abs().max()) < tol_for(dtype, ref)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n", [3, 80])
def test_feed_forward_part_alone(dtype, n):
    from cpmcu_amd.parts import FEED_FORWARDS
    ff = FEED_FORWARDS.build("gated_silu", prefix="m.", hidden_size=48, intermediate_size=72)
    w = {"m.gate_proj.weight": rnd(72, 48, seed=1, scale=0.3), "m.up_proj.weight": rnd(72, 48, seed=2, scale=0.3),
         "m.down_proj.weight": rnd(48, 72, seed=3, scale=0.3)}
    w = {k: v.bfloat16() for k, v in w.items()}
    ff.bind_all({k: v.to(DEV) for k, v in w.items()}, runtime(dtype))
    ctx = make_ctx([], [[0] * n], dtype)
    x = rnd(n, 48, seed=4).to(dtype)
    out = ff.forward(x.to(DEV), ctx)
    out = out.sum(0) if out.dim() == 3 else out
    ref = plain.gated_ffn(x.double(), *(w[k].double() for k in ("m.gate_proj.weight", "m.up_proj.weight", "m.down_proj.weight")))
    assert float((out.double().cpu() - ref).abs().max()) < tol_for(dtype, ref)


@pytest.mark.parametrize("dtype", DTYPES)
def test_block_arrangement(dtype):
    """pre_norm: x += s*mixer(norm1(x)); x += s*ff(norm2(x)), the second branch left pending for the next norm."""
    from cpmcu_amd.parts import BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS, ResidualStream
    H, nh, nkv, hd, I = 32, 2, 1, 16, 40
    blk = BLOCKS.build(
        "pre_norm",
        mixer_norm=NORMS.build("rms_norm", name="n1", hidden_size=H, eps=1e-6),
        mixer=MIXERS.build("gqa_attention", prefix="a.", hidden_size=H, num_heads=nh, num_kv_heads=nkv, head_dim=hd,
                           position=POSITION_ENCODINGS.build("rope", head_dim=hd, theta=100.0)),
        ff_norm=NORMS.build("rms_norm", name="n2", hidden_size=H, eps=1e-6),
        feed_forward=FEED_FORWARDS.build("gated_silu", prefix="m.", hidden_size=H, intermediate_size=I),
        residual_scale=0.7)
    shapes = {s.name: s.shape for s in blk.all_weight_specs()}
    w = {k: (rnd(*v, seed=i, scale=0.2) + (1.0 if len(v) == 1 else 0.0)).bfloat16() for i, (k, v) in enumerate(shapes.items())}
    blk.bind_all({k: v.to(DEV) for k, v in w.items()}, runtime(dtype))
    L = 12
    ctx = make_ctx([blk.mixer.cache_needs()], [[0] * L], dtype)
    x0 = rnd(L, H, seed=99)
    stream = ResidualStream(x0.to(DEV).clone())
    blk.forward(stream, ctx, ctx.cache.view(0))
    W = {k: v.double() for k, v in w.items()}
    cfg = {"hidden_size": H, "num_attention_heads": nh, "num_key_value_heads": nkv, "head_dim": hd, "rope_theta": 100.0,
           "max_position_embeddings": 512}
    inv, m = plain.rope_inv_freq(cfg)
    x = x0.double()
    wa = {"x.self_attn." + k[2:]: v for k, v in W.items() if k.startswith("a.")}
    x = x + 0.7 * plain.attention_layer(cfg, wa, "x.", plain.rms_norm(x, W["n1"], 1e-6), torch.arange(L), inv, m)
    pend = plain.gated_ffn(plain.rms_norm(x, W["n2"], 1e-6), W["m.gate_proj.weight"], W["m.up_proj.weight"], W["m.down_proj.weight"])
    got_pend = stream.pending.sum(0) if stream.pending.dim() == 3 else stream.pending
    assert stream.pending_scale == 0.7
    assert float((stream.x.double().cpu() - x).abs().max()) < tol_for(dtype, x)
    assert float((got_pend.double().cpu() - pend).abs().max()) < tol_for(dtype, pend)


def test_a_branch_left_to_the_next_norm_equals_the_branch_run_by_its_part():
    """Decode steps in bfloat16: the attention and the feed-forward leave their last product to the norm that
    follows (DeferredBranch), which runs it fused with the residual add.  Two blocks in a row, once with the
    package's norm, once with a norm defined here that knows nothing of that hand-over and must be given
    tensors: the same residual stream and the same pending branch, beyond rounding."""
    from cpmcu_amd import ops
    from cpmcu_amd.parts import BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS, ResidualStream
    from cpmcu_amd.parts.base import DeferredBranch, Norm, WeightSpec

    class PlainNorm(Norm):                      # no takes_deferred_branch, no forward_unscaled
        def __init__(self, name, hidden_size, eps):
            self.name, self.hidden_size, self.eps = name, hidden_size, eps

        def weight_specs(self):
            return [WeightSpec(self.name, (self.hidden_size,), "norm")]

        def bind(self, tensors, rt):
            self.weight, self.rt = tensors[self.name].float().contiguous(), rt

        def forward(self, x, branch, branch_scale, ctx, rows=None, tag="norm"):
            assert branch is None or isinstance(branch, torch.Tensor)
            out = ctx.ws.get(tag, (x.shape[0], self.hidden_size), self.rt.dtype)
            ops.add_rms_norm(x, branch, branch_scale, self.weight, self.eps, out, rows)
            return out

    H, nh, nkv, hd, I, n_seq = 64, 4, 2, 16, 96, 5
    results = []
    for norm_ctor in (lambda name: NORMS.build("rms_norm", name=name, hidden_size=H, eps=1e-5),
                      lambda name: PlainNorm(name, H, 1e-5)):
        blocks = [BLOCKS.build(
            "pre_norm", mixer_norm=norm_ctor(f"{i}.n1"),
            mixer=MIXERS.build("gqa_attention", prefix=f"{i}.a.", hidden_size=H, num_heads=nh, num_kv_heads=nkv,
                               head_dim=hd, position=POSITION_ENCODINGS.build("rope", head_dim=hd, theta=100.0)),
            ff_norm=norm_ctor(f"{i}.n2"),
            feed_forward=FEED_FORWARDS.build("gated_silu", prefix=f"{i}.m.", hidden_size=H, intermediate_size=I),
            residual_scale=0.7) for i in range(2)]
        rt = runtime(torch.bfloat16)
        for i, blk in enumerate(blocks):
            shapes = {s.name: s.shape for s in blk.all_weight_specs()}
            w = {k: (rnd(*v, seed=31 * i + j, scale=0.2) + (1.0 if len(v) == 1 else 0.0)).bfloat16().to(DEV)
                 for j, (k, v) in enumerate(shapes.items())}
            blk.bind_all(w, rt)
        # one token each of five sequences that already hold some tokens: a decode step
        ctx = make_ctx([b.mixer.cache_needs() for b in blocks], [[0]] * n_seq, torch.bfloat16, max_slots=8,
                       start=[3, 70, 1, 64, 20])
        for grp in ctx.cache.groups:
            for st in grp.storage.values():
                for t in st.values():
                    t.copy_(rnd(*t.shape, seed=5, scale=0.5))
        stream = ResidualStream(rnd(n_seq, H, seed=9).to(DEV))
        kinds = []
        for i, blk in enumerate(blocks):
            blk.forward(stream, ctx, ctx.cache.view(i))
            kinds.append(type(stream.take_pending()))
        pend = stream.pending
        results.append((stream.x.clone(), (pend.sum(0) if pend.dim() == 3 else pend).clone(), kinds))
    (xa, pa, ka), (xb, pb, kb) = results
    assert ka == [DeferredBranch, DeferredBranch] and kb == ka      # the parts hand over either way
    assert float((xa - xb).abs().max()) <= 2 ** -7 * float(xb.abs().max())
    assert float((pa - pb).abs().max()) <= 2 ** -6 * float(pb.abs().max())


@pytest.mark.parametrize("dtype", DTYPES)
def test_block_sparse_attention_part_alone(dtype):
    """The InfLLM-v2 mixer against the plain layer, whole prompt and then token by token across block edges;
    with topk covering every block it equals the dense mixer."""
    from cpmcu_amd.parts import MIXERS, POSITION_ENCODINGS, StepContext
    H, nh, nkv, hd = 48, 4, 2, 16
    sc = {"kernel_size": 8, "kernel_stride": 4, "block_size": 16, "init_blocks": 1, "topk": 3, "window_size": 32,
          "dense_len": 40}
    w = {"a.q_proj.weight": rnd(nh * hd, H, seed=1, scale=0.3), "a.k_proj.weight": rnd(nkv * hd, H, seed=2, scale=0.3),
         "a.v_proj.weight": rnd(nkv * hd, H, seed=3, scale=0.3), "a.o_proj.weight": rnd(H, nh * hd, seed=4, scale=0.3)}
    w = {k: v.bfloat16() for k, v in w.items()}
    L, L0 = 190, 150
    h = rnd(L, H, seed=7).to(dtype)
    cfg = {"hidden_size": H, "num_attention_heads": nh, "num_key_value_heads": nkv, "head_dim": hd, "rope_theta": 10000.0,
           "max_position_embeddings": 512, "sparse_config": sc}
    inv, m = plain.rope_inv_freq(cfg)
    wd = {"x.self_attn." + k[2:]: v.double() for k, v in w.items()}
    # the plain layer from the same inputs; in bf16 the engine rounds q, k to bf16 before scoring, so near-ties
    # between blocks may fall differently: compare where the plain scores leave a margin
    ref = plain.attention_layer(cfg, wd, "x.", h.double(), torch.arange(L), inv, m)
    ref_dense = plain.attention_layer(cfg, wd, "x.", h.double(), torch.arange(L), inv, m, sparse=False)
    assert float((ref - ref_dense).abs().max()) > 1e-3                    # the selection really prunes

    def run(mixer):
        mixer.bind_all({k: v.to(DEV) for k, v in w.items()}, runtime(dtype))
        ctx = make_ctx([mixer.cache_needs()], [[0] * L0], dtype)
        out = mixer.forward(h[:L0].to(DEV), ctx, ctx.cache.view(0))
        outs = [(out.sum(0) if out.dim() == 3 else out).double().cpu()]
        t = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
        for p in range(L0, L):
            ctx.cache.extend(0, 1)
            ctx.cache.sync()
            c1 = StepContext(n_tokens=1, n_seqs=1, token_ids=t([0]), positions=t([p]), tok_slot=t([0]), cu_q=t([0, 1]),
                             seq_slot=t([0]), seq_len=t([p + 1]), q_lens=[1], kv_lens=[p + 1], max_pos=p,
                             single_token=True, ws=ctx.ws, cache=ctx.cache)
            o = mixer.forward(h[p:p + 1].to(DEV), c1, ctx.cache.view(0))
            outs.append((o.sum(0) if o.dim() == 3 else o).double().cpu())
        return torch.cat(outs)

    pe = lambda: POSITION_ENCODINGS.build("rope", head_dim=hd, theta=10000.0)
    base = dict(prefix="a.", hidden_size=H, num_heads=nh, num_kv_heads=nkv, head_dim=hd)
    got = run(MIXERS.build("infllm_v2_attention", position=pe(), **base, **sc))
    if dtype == torch.float32:
        assert float((got - ref).abs().max()) < tol_for(dtype, ref)
    else:
        rows_ok = ((got - ref).abs().amax(dim=1) < tol_for(dtype, ref)).double().mean()
        assert rows_ok > 0.9, float(rows_ok)
    got_all = run(MIXERS.build("infllm_v2_attention", position=pe(), **base, **dict(sc, topk=64)))
    assert float((got_all - ref_dense).abs().max()) < tol_for(dtype, ref_dense)
