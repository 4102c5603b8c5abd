"""The decode-step kernels and the attention kernels at drawn shapes (rows 1..64, widths that are multiples of 8
only, 1..33 query heads a kv head, every head size, pages of 32..128 tokens) against float64 references (GPU)."""
import random

import pytest
import torch
import torch.nn.functional as F

import test_kernels_gpu as tk

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def rnd(*shape, scale=1.0, dtype=torch.float32, seed=0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(DEV)


@pytest.mark.parametrize("case", range(24))
def test_skinny_product_and_column_norm_at_drawn_shapes(case):
    from cpmcu_amd import ops
    rng = random.Random(500 + case)
    M = rng.choice([1, 2, 3, 7, 8, 15, 16, 17, 31, 32, 33, 48, 63, 64])
    K = 8 * rng.randint(1, 160)
    N = rng.choice([16, 24, 40, 100, 136, 250, 1000, 2 * rng.randint(8, 700)])
    tiled = rng.random() < 0.7
    x = rnd(M, K, dtype=torch.bfloat16, seed=case)
    w = rnd(N, K, scale=K ** -0.5, dtype=torch.bfloat16, seed=case + 1)
    wt = ops.TiledWeight(w) if tiled else w
    y = x.double().cpu() @ w.double().cpu().T
    rs = None
    if rng.random() < 0.5:                       # the row factor of a norm cut by columns
        sums = torch.rand(M, ops.norm_slices(K), generator=torch.Generator().manual_seed(case)) + 0.05
        rs = ops.RowScale(sums.to(DEV), 1e-4)
        y = y * torch.rsqrt(sums.double().sum(1) / K + 1e-4)[:, None]
    top = max(1.0, float(y.abs().max()))
    out = torch.full((M, N), float("nan"), device=DEV)
    ops.gemm_skinny(x, wt, out, 0.75, row_scale=rs)
    assert float((out.double().cpu() - 0.75 * y).abs().max()) <= 2e-4 * top
    for splits in {ops.skinny_split(M, N, K), 2, 3}:
        ks = -(-(-(-K // splits)) // 128) * 128
        if -(-K // ks) != splits:
            continue                             # K cannot be cut into that many slices of whole 128-blocks
        part = torch.full((splits, M, N), float("nan"), device=DEV)
        ops.gemm_skinny(x, wt, part, 1.0, mode="partial", row_scale=rs)
        assert float((part.double().cpu().sum(0) - y).abs().max()) <= 2e-4 * top, splits
    if N % 2 == 0 and (not tiled or (N // 2) % 16 == 0):
        act = torch.full((M, N // 2), float("nan"), device=DEV, dtype=torch.bfloat16)
        ops.gemm_skinny(x, wt, act, mode="gated", row_scale=rs)
        ref = F.silu(y[:, :N // 2]) * y[:, N // 2:]
        assert float((act.double().cpu() - ref).abs().max()) <= 2 ** -7 * max(1.0, float(ref.abs().max()))
    # the norm cut by columns
    H, n, parts = 4 * rng.randint(2, 1100), rng.choice([1, 2, 5, 8, 16]), rng.choice([0, 1, 3, 8])
    x0, wn = rnd(n, H, seed=case + 2), rnd(H, seed=case + 3) + 1.0
    b = rnd(parts, n, H, seed=case + 4) if parts else None
    xx = x0.clone()
    xw = torch.empty(n, H, dtype=torch.bfloat16, device=DEV)
    sums = torch.full((n, ops.norm_slices(H)), float("nan"), device=DEV)
    ops.add_norm_columns(xx, None if b is None else (b if parts > 1 else b[0]), 0.3, wn, xw, sums)
    xs = x0.double().cpu() + (0.3 * b.double().cpu().sum(0) if parts else 0.0)
    assert float((xx.double().cpu() - xs).abs().max()) <= 1e-5 * max(1.0, float(xs.abs().max()))
    assert float((xw.double().cpu() - xs * wn.double().cpu()).abs().max()) <= 2 ** -8 * float((xs * wn.double().cpu()).abs().max())
    assert float((sums.double().cpu().sum(1) - (xs * xs).sum(1)).abs().max()) <= 1e-5 * float((xs * xs).sum(1).max())


@pytest.mark.parametrize("case", range(16))
def test_attention_kernels_at_drawn_shapes(case):
    from cpmcu_amd import ops
    rng = random.Random(900 + case)
    hd = rng.choice([16, 32, 48, 64, 80, 96, 112, 128])
    nkv = rng.choice([1, 2, 3])
    group = rng.choice([1, 2, 4, 5, 16, 17, 33])
    nh = nkv * group
    page = rng.choice([32, 64, 96, 128])
    lens = [rng.randint(1, 700) for _ in range(rng.randint(1, 5))]
    ks, vs, kpool, vpool, table = tk.paged_setup(lens, nkv, hd, page, torch.bfloat16, seed=case)
    scale = hd ** -0.5
    for mode in ("decode", "prompt"):
        positions, seq_of, q_lens = [], [], []
        for s, L in enumerate(lens):
            k = 1 if mode == "decode" else min(L, rng.randint(1, 40))
            positions += list(range(L - k, L))
            seq_of += [s] * k
            q_lens.append(k)
        n = len(positions)
        q = tk.rnd(n, nh, hd, seed=case + 7, dtype=torch.bfloat16)
        ref = tk.attention_reference(q.double().cpu(), ks, vs, positions, seq_of, nh, scale)
        pos_t = torch.tensor(positions, dtype=torch.int32, device=DEV)
        slot_t = torch.tensor(seq_of, dtype=torch.int32, device=DEV)
        top = max(1.0, float(ref.abs().max()))
        if mode == "decode":
            runs = [(s, None) for s in {1, rng.choice([2, 3, 5, 8, 16]), ops.attention_splits(n, nkv, group, max(lens))}]
        else:
            runs = [(None, shape) for shape in ((2, 1), (2, 2), (2, 4), (4, 1))] + [(1, None)]
        for splits, shape in runs:
            out = torch.full((n, nh * hd), float("nan"), dtype=torch.bfloat16, device=DEV)
            if shape is None:
                po = torch.full((n, nh, splits, hd), float("nan"), device=DEV) if splits > 1 else None
                pm = torch.full((n, nh, splits, 2), float("nan"), device=DEV) if splits > 1 else None
                ops.attention_mfma(q.view(n, -1), out, nh, nkv, hd, scale, kpool, vpool, table, page, pos_t, slot_t,
                                   splits, po, pm)
            else:
                tiles = ops.prefill_tiles(q_lens, ops.attention_prefill_tokens_per_wave(nh, nkv, shape[0]), DEV)
                ops.attention_prefill_mfma(q.view(n, -1), out, tiles, nh, nkv, hd, scale, kpool, vpool, table, page,
                                           pos_t, slot_t, shape[0], shape[1])
            err = float((out.double().cpu().view(n, nh, hd) - ref).abs().max())
            assert err <= 2 ** -7 * top, (mode, splits, shape, nh, nkv, hd, page, lens)
