"""Kernels and the engine at the widths they are benchmarked at: the MiniCPM4-8B layer shape (hidden 4096, 32
heads in 2 groups, head size 128, intermediate 16384, vocabulary 73448), where the decode products run 1,024 /
256 / 288 / 4,591 strips and the norm cut by columns 64 slices (GPU).

Products are compared element by element with float64 products of the same bf16 values, so a strip written
to the wrong place, or left out, fails.  The engine is a two-layer model of that shape: the bfloat16 engine
(captured decode steps; and without the re-laid weights) against the float32 engine of the same weights, and
the float32 engine against the plain implementation."""
import math

import pytest
import torch
import torch.nn.functional as F

import plain_minicpm as plain
from test_kernels_gpu import DEV, key_tiles, read_cache_rows, rnd, value_tiles

pytestmark = pytest.mark.gpu

H, NH, NKV, HD, I, V = 4096, 32, 2, 128, 16384, 73448


def bf(*shape, seed, scale=1.0):
    g = torch.Generator(device=DEV).manual_seed(seed)
    return (torch.randn(*shape, generator=g, device=DEV) * scale).to(torch.bfloat16)


def product64(x, w):
    return x.double() @ w.double().T


@pytest.mark.parametrize("n", [1, 8, 16])
def test_gated_product_by_strips_at_full_width(n):
    from cpmcu_amd import ops
    x, w = bf(n, H, seed=1), bf(2 * I, H, seed=2, scale=2.0 * H ** -0.5)
    sums = torch.rand(n, ops.norm_slices(H), device=DEV) + 0.5
    r = torch.rsqrt(sums.double().sum(1) / H + 1e-6)[:, None]
    y = product64(x, w) * r
    ref = F.silu(y[:, :I]) * y[:, I:]
    tol = 2 ** -7 * ref.abs().clamp(min=1.0)
    tw = ops.TiledWeight(w)
    for kernel in ("strip", "skinny"):
        out = torch.full((n, I), float("nan"), dtype=torch.bfloat16, device=DEV)
        if kernel == "strip":
            ops.gated_strip(x, tw, out, row_scale=ops.RowScale(sums, 1e-6))
        else:
            ops.gemm_skinny(x, tw, out, mode="gated", row_scale=ops.RowScale(sums, 1e-6))
        bad = ((out.double() - ref).abs() > tol).nonzero()
        assert bad.numel() == 0, f"{kernel}: first wrong element (row, column) {bad[0].tolist()} of {bad.shape[0]}"


@pytest.mark.parametrize("n", [33, 64])
def test_gated_product_of_many_rows_at_full_width(n):
    from cpmcu_amd import ops
    x, w = bf(n, H, seed=3), bf(2 * I, H, seed=4, scale=2.0 * H ** -0.5)
    y = product64(x, w)
    ref = F.silu(y[:, :I]) * y[:, I:]
    out = torch.full((n, I), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops.gemm_skinny(x, ops.TiledWeight(w), out, mode="gated")
    bad = ((out.double() - ref).abs() > 2 ** -7 * ref.abs().clamp(min=1.0)).nonzero()
    assert bad.numel() == 0, f"first wrong element {bad[0].tolist()} of {bad.shape[0]}"


@pytest.mark.parametrize("n,N,K", [(8, H, I), (16, H, I), (8, H, NH * HD), (1, H, I)])
def test_product_with_residual_and_norm_at_full_width(n, N, K):
    """down (K = 16384) and o (K = 4096) fused with the residual add and the next norm's column work."""
    from cpmcu_amd import ops
    a, w = bf(n, K, seed=5), bf(N, K, seed=6, scale=K ** -0.5)
    x0 = torch.randn(n, N, device=DEV, generator=torch.Generator(device=DEV).manual_seed(7))
    wn = torch.rand(N, device=DEV) + 0.5
    x = x0.clone()
    xw = torch.full((n, N), float("nan"), dtype=torch.bfloat16, device=DEV)
    sums = torch.full((n, N // 16), float("nan"), device=DEV)
    ops.proj_add_norm(a, ops.TiledWeight(w), 0.35, x, wn, xw, sums)
    xs = x0.double() + 0.35 * product64(a, w)
    bad = ((x.double() - xs).abs() > 2e-5 * xs.abs().clamp(min=1.0)).nonzero()
    assert bad.numel() == 0, f"residual: first wrong element {bad[0].tolist()} of {bad.shape[0]}"
    ref = xs * wn.double()
    assert float(((xw.double() - ref).abs() / ref.abs().clamp(min=1.0)).max()) <= 2 ** -8
    want = (xs * xs).view(n, N // 16, 16).sum(2)
    assert float((sums.double() - want).abs().max()) <= 1e-5 * float(want.max())
    # the split product and the norm cut by columns (what runs without the re-laid weights) agree
    S = ops.skinny_split(n, N, K)
    part = torch.full((S, n, N), float("nan"), device=DEV)
    ops.gemm_skinny(a, w, part if S > 1 else part[0], 1.0, mode="partial" if S > 1 else "plain")
    x2 = x0.clone()
    xw2 = torch.empty_like(xw)
    sums2 = torch.full((n, ops.norm_slices(N)), float("nan"), device=DEV)
    ops.add_norm_columns(x2, part if S > 1 else part[0], 0.35, wn, xw2, sums2)
    assert float((x2.double() - xs).abs().max()) <= 2e-5 * float(xs.abs().max())
    assert float((sums2.double().sum(1) - (xs * xs).sum(1)).abs().max()) <= 1e-5 * float((xs * xs).sum(1).max())


@pytest.mark.parametrize("n", [1, 8, 16])
def test_fused_projection_at_full_width(n):
    """q, k, v (4,608 rows of 4,096 columns, 288 strips), rotated, k and v read back from the pages."""
    from cpmcu_amd import ops
    page = 64
    w, x = bf((NH + 2 * NKV) * HD, H, seed=8, scale=H ** -0.5), bf(n, H, seed=9)
    g = torch.Generator().manual_seed(n)
    slots = torch.randint(0, 3, (n,), generator=g)
    positions = torch.randperm(4000, generator=g)[:n]
    table = torch.randperm(200, generator=g)[:189].view(3, 63).to(torch.int32)
    inv_freq = torch.rand(HD // 2, generator=g) * 0.5 + 1e-4
    kpool = torch.zeros(200, page, NKV * HD, dtype=torch.bfloat16, device=DEV)
    vpool = torch.zeros_like(kpool)
    q_out = torch.full((n, NH * HD), float("nan"), dtype=torch.bfloat16, device=DEV)
    sums = torch.rand(n, ops.norm_slices(H), device=DEV) + 0.5
    ops.qkv_rope(x, ops.qkv_rope_weight(w, NH, NKV, HD), q_out, NH, NKV, HD, positions.to(torch.int32).to(DEV),
                 slots.to(torch.int32).to(DEV), inv_freq.to(DEV), 1.1, kpool, vpool, table.to(DEV), page,
                 row_scale=ops.RowScale(sums, 1e-6))
    r = torch.rsqrt(sums.double().sum(1) / H + 1e-6).view(n, 1, 1).cpu()
    y = product64(x, w).cpu().view(n, NH + 2 * NKV, HD) * r
    ang = positions.double()[:, None] * inv_freq.float().double()[None, :]
    cs, sn = (torch.cos(ang) * 1.1)[:, None, :], (torch.sin(ang) * 1.1)[:, None, :]
    a, b = y[:, :NH + NKV, :HD // 2].clone(), y[:, :NH + NKV, HD // 2:].clone()
    y[:, :NH + NKV] = torch.cat([a * cs - b * sn, a * sn + b * cs], dim=-1)
    # positions up to 4,000 times float32 angles: allow the angle's own rounding (2^-24 * 4000 rad) on top of bf16
    tol = 2 ** -7 * max(1.0, float(y.abs().max()))
    err = (q_out.double().cpu().view(n, NH, HD) - y[:, :NH]).abs()
    assert float(err.max()) <= tol, f"q: head {int(err.amax(dim=(0, 2)).argmax())}"
    for t in range(n):
        k_row = read_cache_rows(kpool, table, page, NKV, HD, int(slots[t]), [int(positions[t])], key_tiles)[0]
        v_row = read_cache_rows(vpool, table, page, NKV, HD, int(slots[t]), [int(positions[t])], value_tiles)[0]
        assert float((k_row.double() - y[t, NH:NH + NKV]).abs().max()) <= tol, t
        assert float((v_row.double() - y[t, NH + NKV:]).abs().max()) <= tol, t
    assert int((kpool != 0).sum()) <= n * NKV * HD


@pytest.mark.parametrize("n", [1, 8, 64])
def test_head_product_at_full_width(n):
    """The output head: 73,448 rows (4,591 strips, the last one padded) of 4,096 columns, float32 logits."""
    from cpmcu_amd import ops
    w, x = bf(V, H, seed=10, scale=0.02), bf(n, H, seed=11)
    ref = product64(x, w) * 0.0625
    for weight in (w, ops.TiledWeight(w)):
        out = torch.full((n, V), float("nan"), device=DEV)
        ops.gemm_skinny(x, weight, out, 0.0625)
        bad = ((out.double() - ref).abs() > 1e-5 * ref.abs().clamp(min=1.0)).nonzero()
        assert bad.numel() == 0, f"first wrong element {bad[0].tolist()} of {bad.shape[0]}"


@pytest.mark.parametrize("M,N,K", [(8, 4608, 4096), (64, 4096, 16384), (33, 4096, 4096), (64, 32768, 4096)])
def test_split_products_at_full_width(M, N, K):
    """The products that the engine runs without the strip kernels (17 to 64 rows, or no re-laid weights):
    partial sums over the slices of K that the heuristic chooses."""
    from cpmcu_amd import ops
    x, w = bf(M, K, seed=12), bf(N, K, seed=13, scale=K ** -0.5)
    ref = product64(x, w)
    S = ops.skinny_split(M, N, K)
    for weight in (w, ops.TiledWeight(w)):
        if S > 1:
            part = torch.full((S, M, N), float("nan"), device=DEV)
            ops.gemm_skinny(x, weight, part, 1.0, mode="partial")
            got = part.double().sum(0)
        else:
            out = torch.full((M, N), float("nan"), device=DEV)
            ops.gemm_skinny(x, weight, out)
            got = out.double()
        bad = ((got - ref).abs() > 2e-5 * ref.abs().clamp(min=1.0)).nonzero()
        assert bad.numel() == 0, f"{S} slices: first wrong element {bad[0].tolist()} of {bad.shape[0]}"


# ---------------------------------------------------------------------------- a two-layer model of the 8B layer shape
def raw_config():
    g = torch.Generator().manual_seed(1234)
    fac = lambda: [float(v) for v in (1.0 + 3.0 * torch.rand(HD // 2, generator=g, dtype=torch.float64))]
    return {
        "architectures": ["MiniCPMForCausalLM"], "model_type": "minicpm",
        "num_hidden_layers": 2, "hidden_size": H, "num_attention_heads": NH, "num_key_value_heads": NKV,
        "head_dim": HD, "intermediate_size": I, "vocab_size": V, "rms_norm_eps": 1e-6, "rope_theta": 10000.0,
        "max_position_embeddings": 32768,
        "rope_scaling": {"rope_type": "longrope", "short_factor": fac(), "long_factor": fac(),
                         "original_max_position_embeddings": 32768},
        "scale_emb": 12, "dim_model_base": 256, "scale_depth": 1.4, "tie_word_embeddings": False,
        "hidden_act": "silu", "torch_dtype": "bfloat16",
    }


@pytest.fixture(scope="module")
def model():
    from cpmcu_amd import Engine, EngineOptions
    from cpmcu_amd.config import MiniCPMConfig
    from cpmcu_amd.weights import random_tensors
    raw = raw_config()
    cfg = MiniCPMConfig.from_dict(raw)
    tensors = random_tensors(cfg, seed=5, norm_std=0.1, device=DEV)
    common = dict(max_tokens=64 * 192 + 4096, max_slots=64, max_step_tokens=2048, device=DEV)
    engines = {
        "float32": Engine.from_tensors(cfg, tensors, EngineOptions(dtype="float32", **common)),
        "bfloat16": Engine.from_tensors(cfg, tensors, EngineOptions(dtype="bfloat16", hip_graph=True, **common)),
        "bfloat16, weights not re-laid": Engine.from_tensors(cfg, tensors, EngineOptions(dtype="bfloat16", tiled_weights=False,
                                                                                         **common)),
    }
    yield raw, tensors, engines
    engines.clear()
    torch.cuda.empty_cache()


def tokens(n, seed):
    g = torch.Generator().manual_seed(seed)
    return [int(t) for t in torch.randint(0, V, (n,), generator=g)]


def assert_close(got, ref, what, frac=0.02):
    err = (got - ref).abs().amax(1)
    lim = frac * ref.abs().amax(1)
    bad = (err > lim).nonzero().flatten()
    assert bad.numel() == 0, f"{what}: first wrong row {int(bad[0])}: error {float(err[bad[0]]):.3g} > {float(lim[bad[0]]):.3g}"
    return float((err / lim).max())


def test_float32_engine_equals_the_plain_implementation_at_full_width(model):
    from cpmcu_amd import StepEntry
    raw, tensors, engines = model
    toks = tokens(96, 1)
    ref = plain.forward(raw, {k: v.cpu() for k, v in tensors.items()}, toks)
    eng = engines["float32"]
    s = eng.acquire()
    got = eng.step([StepEntry(s, toks, list(range(len(toks))))]).double().cpu()
    eng.release(s)
    assert_close(got, ref, "float32 engine against the plain implementation", frac=2e-4)


def test_prompt_of_2048_tokens_at_full_width(model):
    from cpmcu_amd import StepEntry
    raw, tensors, engines = model
    toks = tokens(2048, 2)
    want = [0, 1, 63, 64, 1000, 2046, 2047]
    outs = {}
    for name, eng in engines.items():
        s = eng.acquire()
        outs[name] = eng.step([StepEntry(s, toks, want)]).double().cpu()
        eng.release(s)
    for name in list(engines)[1:]:
        assert_close(outs[name], outs["float32"], f"{name}: prompt of 2,048 tokens")


@pytest.mark.parametrize("batch", [1, 8, 64])
def test_decode_steps_at_full_width(model, batch):
    """Unequal prompts start together, then 6 single-token steps of the whole batch (the captured graph from the
    second on): every step's logits against the float32 engine's."""
    from cpmcu_amd import StepEntry
    raw, tensors, engines = model
    g = torch.Generator().manual_seed(batch)
    lens = [int(v) for v in torch.randint(20, 120, (batch,), generator=g)]
    prompts = [tokens(n, 100 + i) for i, n in enumerate(lens)]
    feed = [tokens(batch, 500 + i) for i in range(6)]
    outs = {}
    for name, eng in engines.items():
        slots = [eng.acquire() for _ in range(batch)]
        steps = [eng.step([StepEntry(s, p, [len(p) - 1]) for s, p in zip(slots, prompts)]).double().cpu()]
        for f in feed:
            steps.append(eng.step([StepEntry(s, [t], [0]) for s, t in zip(slots, f)]).double().cpu())
        for s in slots:
            eng.release(s)
        outs[name] = steps
    for name in list(engines)[1:]:
        for i, (got, ref) in enumerate(zip(outs[name], outs["float32"])):
            assert_close(got, ref, f"{name}: batch {batch}, step {i}")
