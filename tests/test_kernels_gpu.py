"""Each kernel alone against a plain float reference, at sizes other than the engine's (GPU)."""
import math

import pytest
import torch
import torch.nn.functional as F

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def rnd(*shape, seed=0, dtype=torch.float32, scale=1.0):
    g = torch.Generator(device="cpu").manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(DEV)


# ---------------------------------------------------------------------------- products
@pytest.mark.parametrize("M,N,K", [(1, 40, 64), (7, 129, 96), (64, 512, 160), (65, 100, 72), (200, 333, 50), (3, 17, 5)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_plain_product(M, N, K, dtype):
    from cpmcu_amd import ops
    x, w = rnd(M, K, seed=1, dtype=dtype), rnd(N, K, seed=2, dtype=dtype)
    ref = 0.5 * (x.double() @ w.double().T)
    for out_dtype in ([torch.float32] if dtype == torch.float32 else [torch.float32, torch.bfloat16]):
        out = torch.empty(M, N, dtype=out_dtype, device=DEV)
        ops.gemm_nt_plain(x, w, out, 0.5)
        tol = 1e-5 * math.sqrt(K) if out_dtype == torch.float32 else 2 ** -8 * float(ref.abs().max())
        assert float((out.double() - ref).abs().max()) <= tol


@pytest.mark.parametrize("M", [1, 5, 16, 17, 33, 48, 64])
@pytest.mark.parametrize("N,K", [(96, 64), (136, 160), (1000, 96), (4608, 1024), (250, 520), (73448 // 8 + 3, 256)])
def test_skinny_product_all_modes(M, N, K):
    """bf16 operands are exact in float, so the matrix-core product must match a float64 product of the same
    bf16 values up to float32 accumulation."""
    from cpmcu_amd import ops
    x, w = rnd(M, K, seed=3, dtype=torch.bfloat16), rnd(N, K, seed=4, dtype=torch.bfloat16, scale=0.1)
    ref = x.double() @ w.double().T
    tol = 2e-6 * math.sqrt(K) * float(ref.abs().max() + 1)
    out = torch.empty(M, N, dtype=torch.float32, device=DEV)
    ops.gemm_skinny(x, w, out, 1.0)
    assert float((out.double() - ref).abs().max()) <= tol
    ops.gemm_skinny(x, w, out, 0.25)
    assert float((out.double() - 0.25 * ref).abs().max()) <= tol
    out16 = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    ops.gemm_skinny(x, w, out16, 1.0)
    assert float((out16.double() - ref).abs().max()) <= 2 ** -8 * float(ref.abs().max())
    for S in (2, 3):                                    # slices of K, summed by the consumer
        ks = -(-(-(-K // S)) // 128) * 128
        S_real = -(-K // ks)
        part = torch.full((S_real, M, N), float("nan"), dtype=torch.float32, device=DEV)
        ops.gemm_skinny(x, w, part, 1.0, mode="partial")
        assert float((part.double().sum(0) - ref).abs().max()) <= tol
    if N % 2 == 0:
        I = N // 2
        act = torch.empty(M, I, dtype=torch.bfloat16, device=DEV)
        ops.gemm_skinny(x, w, act, mode="gated")
        want = F.silu(ref[:, :I]) * ref[:, I:]
        assert float((act.double() - want).abs().max()) <= 2 ** -8 * float(want.abs().max()) + tol
    # the same from the weight re-laid for this kernel
    wt = ops.TiledWeight(w)
    out.fill_(float("nan"))
    ops.gemm_skinny(x, wt, out, 0.25)
    assert float((out.double() - 0.25 * ref).abs().max()) <= tol
    ks = -(-(-(-K // 2)) // 128) * 128
    part = torch.full((-(-K // ks), M, N), float("nan"), dtype=torch.float32, device=DEV)
    ops.gemm_skinny(x, wt, part, 1.0, mode="partial")
    assert float((part.double().sum(0) - ref).abs().max()) <= tol
    if N % 32 == 0:
        act = torch.full((M, N // 2), float("nan"), dtype=torch.bfloat16, device=DEV)
        ops.gemm_skinny(x, wt, act, mode="gated")
        want = F.silu(ref[:, :N // 2]) * ref[:, N // 2:]
        assert float((act.double() - want).abs().max()) <= 2 ** -8 * float(want.abs().max()) + tol


def test_skinny_split_heuristic_gives_slices_that_sum_to_the_product():
    """Whatever number of slices the heuristic chooses for a shape, the kernel takes it and the slices' partial
    sums add up to the product (one-hot rows of x pick out columns of w, so the expected value is exact)."""
    from cpmcu_amd import ops
    for M in (1, 8, 64):
        for N, K in [(4608, 4096), (4096, 4096), (4096, 16384), (73448, 4096), (64, 64), (96, 160), (1000, 96)]:
            S = ops.skinny_split(M, N, K)
            assert 1 <= S <= 16 and (S == 1 or K // S >= 128)
            x = torch.zeros(M, K, dtype=torch.bfloat16, device=DEV)
            cols = [(7 * m + 3) * K // (7 * M + 4) for m in range(M)]            # spread over all slices
            for m, c in enumerate(cols):
                x[m, c] = 1.0
            w = rnd(N, K, seed=N % 97, dtype=torch.bfloat16)
            want = w[:, cols].T.float()
            if S > 1:
                part = torch.full((S, M, N), float("nan"), dtype=torch.float32, device=DEV)
                ops.gemm_skinny(x, w, part, mode="partial")
                got = part.sum(0)
            else:
                got = torch.full((M, N), float("nan"), dtype=torch.float32, device=DEV)
                ops.gemm_skinny(x, w, got)
            assert torch.equal(got, want), (M, N, K, S)


def test_products_refuse_what_they_do_not_take():
    from cpmcu_amd import ops
    x, w = torch.zeros(65, 64, dtype=torch.bfloat16, device=DEV), torch.zeros(32, 64, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(ops.KernelError, match="1..64"):
        ops.gemm_skinny(x, w, torch.empty(65, 32, dtype=torch.float32, device=DEV))
    with pytest.raises(ops.KernelError, match="multiple of 8"):
        ops.gemm_skinny(torch.zeros(2, 20, dtype=torch.bfloat16, device=DEV), torch.zeros(8, 20, dtype=torch.bfloat16, device=DEV),
                        torch.empty(2, 8, dtype=torch.float32, device=DEV))
    with pytest.raises(ops.KernelError, match="GPU tensor"):
        ops.gemm_nt_plain(torch.zeros(2, 8), torch.zeros(4, 8), torch.zeros(2, 4))
    with pytest.raises(ops.KernelError, match="shape"):
        ops.gemm_nt_plain(x, w, torch.empty(65, 33, dtype=torch.float32, device=DEV))


# ---------------------------------------------------------------------------- row-wise kernels
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embedding(dtype):
    from cpmcu_amd import ops
    table = rnd(37, 50, dtype=dtype)
    ids = torch.tensor([0, 36, 5, 5, 17], dtype=torch.int32, device=DEV)
    out = torch.empty(5, 50, dtype=torch.float32, device=DEV)
    ops.embed(table, ids, out, 12.0)
    assert torch.equal(out, table.float()[ids.long()] * 12.0)


@pytest.mark.parametrize("H,n", [(24, 6), (100, 6), (1000, 6), (4096 + 8, 6), (7, 3), (66, 3), (96, 600),
                                 (1100, 301), (4096, 257), (2052, 300), (4096 + 8, 258)])
@pytest.mark.parametrize("bdtype,odtype", [(torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16),
                                           (torch.float32, torch.bfloat16), (torch.bfloat16, torch.float32)])
def test_add_rms_norm(H, n, bdtype, odtype):
    from cpmcu_amd import ops
    eps = 1e-5
    x0, w = rnd(n, H, seed=1), rnd(H, seed=2) + 1.0
    otol = 1e-5 if odtype == torch.float32 else 2 ** -8
    # plain norm
    x = x0.clone()
    out = torch.empty(n, H, dtype=odtype, device=DEV)
    ops.add_rms_norm(x, None, 1.0, w, eps, out)
    ref = F.rms_norm(x0.double(), (H,), w.double(), eps)
    assert torch.equal(x, x0) and float((out.double() - ref).abs().max()) <= otol * float(ref.abs().max())
    # with a branch, as one tensor and as 3 partial sums
    for parts in (1, 3):
        b = rnd(parts, n, H, seed=3, dtype=bdtype)
        x = x0.clone()
        ops.add_rms_norm(x, b if parts > 1 else b[0], 0.7, w, eps, out)
        xs = x0.double() + 0.7 * b.double().sum(0)
        assert float((x.double() - xs).abs().max()) <= 1e-5
        ref = F.rms_norm(xs, (H,), w.double(), eps)
        assert float((out.double() - ref).abs().max()) <= otol * float(ref.abs().max())
        # chosen rows only (one of them twice): x stays as it was
        rows = torch.tensor([n - 2, 0, n - 2], dtype=torch.int32, device=DEV)
        x = x0.clone()
        out_r = torch.empty(3, H, dtype=odtype, device=DEV)
        ops.add_rms_norm(x, b if parts > 1 else b[0], 0.7, w, eps, out_r, rows)
        assert torch.equal(x, x0)
        assert float((out_r.double() - ref[rows.long()]).abs().max()) <= otol * float(ref.abs().max())
    # eps inside the root: a tiny constant row
    c = 3e-3
    x = torch.full((1, H), c, device=DEV)
    o = torch.empty(1, H, dtype=torch.float32, device=DEV)
    ops.add_rms_norm(x, None, 1.0, torch.ones(H, device=DEV), eps, o)
    assert float((o - c / math.sqrt(c * c + eps)).abs().max()) < 1e-6


@pytest.mark.parametrize("H,n", [(64, 1), (200, 7), (4096 + 8, 16), (328, 17), (96, 64)])
@pytest.mark.parametrize("bdtype,parts", [(torch.float32, 0), (torch.float32, 1), (torch.float32, 5), (torch.bfloat16, 1)])
def test_norm_cut_by_columns_and_finished_by_the_product(H, n, bdtype, parts):
    """add_norm_columns leaves x * w and slice sums of x^2; the products multiply their rows by
    rsqrt(sum / H + eps): together they equal product(rmsnorm(x) * w), gated and plain and in partial sums."""
    from cpmcu_amd import ops
    eps = 3e-4
    x0, w = rnd(n, H, seed=1), rnd(H, seed=2) + 1.0
    b = rnd(parts, n, H, seed=3, dtype=bdtype) if parts else None
    x = x0.clone()
    xw = torch.empty(n, H, dtype=torch.bfloat16, device=DEV)
    sums = torch.full((n, ops.norm_slices(H)), float("nan"), device=DEV)
    ops.add_norm_columns(x, None if b is None else (b if parts > 1 else b[0]), 0.7, w, xw, sums)
    xs = x0.double() + (0.7 * b.double().sum(0) if parts else 0.0)
    assert float((x.double() - xs).abs().max()) <= 1e-5
    assert float((xw.double() - xs * w.double()).abs().max()) <= 2 ** -8 * float((xs * w.double()).abs().max())
    ss = (xs * xs).sum(1)
    assert float((sums.double().sum(1) - ss).abs().max()) <= 1e-5 * float(ss.max())
    assert float((sums[:, 0].double() - (xs[:, :64] ** 2).sum(1)).abs().max()) <= 1e-5 * float(ss.max())
    # the products finish the norm: against the float64 product of the rounded x * w, scaled row by row
    rs = ops.RowScale(sums, eps)
    r = torch.rsqrt(ss / H + eps)[:, None]
    if H % 8:
        return
    N = 160
    wm = rnd(N, H, seed=4, dtype=torch.bfloat16, scale=H ** -0.5)
    for weight in (wm, ops.TiledWeight(wm)):
        y = (xw.double() @ wm.double().T) * r
        out = torch.empty(n, N, device=DEV)
        ops.gemm_skinny(xw, weight, out, 0.5, row_scale=rs)
        assert float((out.double() - 0.5 * y).abs().max()) <= 1e-4 * float(y.abs().max())
        part = torch.empty(2, n, N, device=DEV)
        if H > 128:                            # two slices of whole 128-column blocks
            ops.gemm_skinny(xw, weight, part, 1.0, mode="partial", row_scale=rs)
            assert float((part.double().sum(0) - y).abs().max()) <= 1e-4 * float(y.abs().max())
        act = torch.empty(n, N // 2, dtype=torch.bfloat16, device=DEV)
        ops.gemm_skinny(xw, weight, act, mode="gated", row_scale=rs)
        ref = F.silu(y[:, :N // 2]) * y[:, N // 2:]
        assert float((act.double() - ref).abs().max()) <= 2 ** -7 * max(1.0, float(ref.abs().max()))


@pytest.mark.parametrize("n,N,K", [(1, 64, 128), (5, 100, 72), (16, 4096 + 16, 264), (17, 36, 1032), (32, 328, 520),
                                   (33, 68, 136), (64, 1024 + 4, 1160)])
def test_product_that_adds_into_the_residual_and_does_the_norms_column_work(n, N, K):
    """proj_add_norm: x += alpha * (a . W^T); x * w in bfloat16; sums of x^2 by strips of 16 columns; a product
    that reads them finishes the norm.  Against float64, and against the pair of kernels it replaces."""
    from cpmcu_amd import ops
    eps, alpha = 2e-5, 0.6
    a = rnd(n, K, seed=1, dtype=torch.bfloat16)
    wm = rnd(N, K, seed=2, dtype=torch.bfloat16, scale=K ** -0.5)
    x0, w = rnd(n, N, seed=3), rnd(N, seed=4) + 1.0
    x = x0.clone()
    xw = torch.full((n, N), float("nan"), dtype=torch.bfloat16, device=DEV)
    sums = torch.full((n, -(-N // 16)), float("nan"), device=DEV)
    ops.proj_add_norm(a, ops.TiledWeight(wm), alpha, x, w, xw, sums)
    xs = x0.double() + alpha * (a.double() @ wm.double().T)
    assert float((x.double() - xs).abs().max()) <= 1e-5 * max(1.0, float(xs.abs().max()))
    ref = xs * w.double()
    assert float((xw.double() - ref).abs().max()) <= 2 ** -8 * float(ref.abs().max())
    ss = (xs * xs).sum(1)
    assert float((sums.double().sum(1) - ss).abs().max()) <= 1e-5 * float(ss.max())
    assert float((sums[:, 1].double() - (xs[:, 16:32] ** 2).sum(1)).abs().max()) <= 1e-5 * float(ss.max())
    # the same through the split product and add_norm_columns
    if n <= 16:
        x2 = x0.clone()
        y = torch.empty(n, N, device=DEV)
        ops.gemm_skinny(a, wm, y)
        xw2 = torch.empty_like(xw)
        sums2 = torch.empty(n, ops.norm_slices(N), device=DEV)
        ops.add_norm_columns(x2, y, alpha, w, xw2, sums2)
        assert float((x - x2).abs().max()) <= 1e-5 * max(1.0, float(xs.abs().max()))
    # a product that reads x * w and the strips' sums finishes the norm
    if N % 8 == 0:
        N2 = 48
        w2 = rnd(N2, N, seed=5, dtype=torch.bfloat16, scale=N ** -0.5)
        out = torch.empty(n, N2, device=DEV)
        ops.gemm_skinny(xw, ops.TiledWeight(w2), out, 1.0, row_scale=ops.RowScale(sums, eps))
        yr = (xw.double() @ w2.double().T) * torch.rsqrt(ss / N + eps)[:, None]
        assert float((out.double() - yr).abs().max()) <= 1e-4 * float(yr.abs().max())


@pytest.mark.parametrize("n,I,K", [(1, 16, 72), (7, 48, 264), (16, 1008, 1032), (8, 4096, 128)])
@pytest.mark.parametrize("scaled", [False, True])
def test_gated_product_by_strips(n, I, K, scaled):
    """gated_strip: silu(x Wg^T) * (x Wu^T) with a workgroup a strip of gate rows and their up rows, with and
    without the row factor of a norm cut by columns; against float64 and against the skinny product."""
    from cpmcu_amd import ops
    x = rnd(n, K, seed=1, dtype=torch.bfloat16)
    w = rnd(2 * I, K, seed=2, dtype=torch.bfloat16, scale=2.0 * K ** -0.5)
    tw = ops.TiledWeight(w)
    rs, r = None, 1.0
    if scaled:
        sums = torch.rand(n, 5, generator=torch.Generator().manual_seed(n)) + 0.1
        rs = ops.RowScale(sums.to(DEV), 1e-3)
        r = torch.rsqrt(sums.double().sum(1) / K + 1e-3).view(n, 1).to(DEV)
    out = torch.full((n, I), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops.gated_strip(x, tw, out, row_scale=rs)
    y = (x.double() @ w.double().T) * r
    ref = F.silu(y[:, :I]) * y[:, I:]
    assert float((out.double() - ref).abs().max()) <= 2 ** -7 * max(1.0, float(ref.abs().max()))
    other = torch.empty_like(out)
    ops.gemm_skinny(x, tw, other, mode="gated", row_scale=rs)
    assert float((out.double() - other.double()).abs().max()) <= 2 ** -6 * max(1.0, float(ref.abs().max()))
    with pytest.raises(ops.KernelError):          # 17 rows
        ops.gated_strip(rnd(17, K, dtype=torch.bfloat16), tw, torch.empty(17, I, dtype=torch.bfloat16, device=DEV))


def test_gated_product_by_strips_refuses_gate_rows_that_are_no_multiple_of_16():
    from cpmcu_amd import ops
    tw = ops.TiledWeight(rnd(2 * 24, 64, dtype=torch.bfloat16))
    with pytest.raises(ops.KernelError):
        ops.gated_strip(rnd(2, 64, dtype=torch.bfloat16), tw, torch.empty(2, 24, dtype=torch.bfloat16, device=DEV))


def test_product_with_norm_refuses_what_it_does_not_take():
    from cpmcu_amd import ops
    a = rnd(65, 64, dtype=torch.bfloat16)
    tw = ops.TiledWeight(rnd(32, 64, dtype=torch.bfloat16))
    x, w = rnd(65, 32), rnd(32)
    with pytest.raises(ops.KernelError):          # too many rows
        ops.proj_add_norm(a, tw, 1.0, x, w, torch.empty(65, 32, dtype=torch.bfloat16, device=DEV), torch.empty(65, 2, device=DEV))
    with pytest.raises(ops.KernelError):          # a weight that is not tiled for these columns
        ops.proj_add_norm(a[:4, :32].contiguous(), tw, 1.0, x[:4].contiguous(), w,
                          torch.empty(4, 32, dtype=torch.bfloat16, device=DEV), torch.empty(4, 2, device=DEV))


@pytest.mark.parametrize("I", [77, 160, 1000])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_silu_mul(dtype, I):
    from cpmcu_amd import ops
    gu = rnd(5, 2 * I, dtype=dtype, scale=3.0)
    out = torch.empty(5, I, dtype=dtype, device=DEV)
    ops.silu_mul(gu, out)
    ref = F.silu(gu[:, :I].double()) * gu[:, I:].double()
    tol = 1e-6 if dtype == torch.float32 else 2 ** -8
    assert float((out.double() - ref).abs().max()) <= tol * float(ref.abs().max() + 1)


def test_silu_mul_of_many_rows():
    """Prompt chunks take the form with several pieces a thread in flight; the last workgroup's pieces run past
    the end."""
    from cpmcu_amd import ops
    n, I = 1100, 16392
    gu = rnd(n, 2 * I, dtype=torch.bfloat16, scale=3.0)
    out = torch.full((n, I), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops.silu_mul(gu, out)
    ref = F.silu(gu[:, :I].float()) * gu[:, I:].float()
    assert not bool(out.isnan().any())
    assert float((out.float() - ref).abs().max()) <= 2 ** -8 * float(ref.abs().max() + 1)
    # rows that differ everywhere: a wrong row or column offset cannot hide
    assert torch.equal(out[-1], (F.silu(gu[-1, :I].float()) * gu[-1, I:].float()).to(torch.bfloat16)) or \
        float((out[-1].float() - ref[-1]).abs().max()) <= 2 ** -8 * float(ref[-1].abs().max() + 1)


# ---------------------------------------------------------------------------- attention over the paged cache
def key_tiles(full):
    """[page tokens, kv heads, d] -> the cache's layout of keys: per chunk of 32 tokens and kv head two tiles of
    16 key slots (token 8a + 4u + i of the chunk is slot 4a + i of tile u), a tile [d / 8][slot][d % 8]."""
    page, nkv, hd = full.shape
    x = full.view(page // 32, 4, 2, 4, nkv, hd // 8, 8)          # chunk, a, u, i, kv head, d / 8, d % 8
    return x.permute(0, 4, 2, 5, 1, 3, 6).contiguous()            # chunk, kv head, u, d / 8, a, i, d % 8


def key_elements(in_page, kvh, nkv, hd, page):
    """Where the hd elements of one key lie inside its page (flat indices), by the same rule as key_tiles."""
    c, t32 = divmod(in_page, 32)
    a_, r = divmod(t32, 8)
    u, i = divmod(r, 4)
    d = torch.arange(hd)
    return ((((c * nkv + kvh) * 2 + u) * (hd // 8) + d // 8) * 16 + a_ * 4 + i) * 8 + d % 8


def value_tiles(full):
    """[page tokens, kv heads, d] -> the cache's layout of values: per chunk of 32 tokens and kv head
    [d / 16][token / 8][d % 16][token % 8]."""
    page, nkv, hd = full.shape
    x = full.view(page // 32, 4, 8, nkv, hd // 16, 16)           # chunk, token / 8, token % 8, kv head, d / 16, d % 16
    return x.permute(0, 3, 4, 1, 5, 2).contiguous()


def paged_setup(lens, nkv, hd, page, dtype, seed=0, scramble=True):
    """Sequences of the given lengths in a paged cache whose pages are handed out in a scrambled order.
    Returns keys/values per sequence (float64) and the pools/page table as the kernels want them."""
    g = torch.Generator().manual_seed(seed)
    n_pages_seq = [-(-L // page) for L in lens]
    total = sum(n_pages_seq) + 3
    perm = torch.randperm(total, generator=g).tolist() if scramble else list(range(total))
    table = torch.zeros(len(lens), max(n_pages_seq), dtype=torch.int32)
    kpool = torch.zeros(total, page, nkv * hd, dtype=dtype)
    vpool = torch.zeros(total, page, nkv * hd, dtype=dtype)            # both in the matrix cores' operand order: same bytes
    ks, vs = [], []
    it = iter(perm)
    for s, L in enumerate(lens):
        k = torch.randn(L, nkv, hd, generator=g).to(dtype)
        v = torch.randn(L, nkv, hd, generator=g).to(dtype)
        ks.append(k.double())
        vs.append(v.double())
        for pn in range(n_pages_seq[s]):
            pg = next(it)
            table[s, pn] = pg
            a, b = pn * page, min((pn + 1) * page, L)
            full = torch.zeros(page, nkv, hd, dtype=dtype)
            full[:b - a] = k[a:b]
            kpool[pg] = key_tiles(full).reshape(page, nkv * hd)
            full = torch.zeros(page, nkv, hd, dtype=dtype)
            full[:b - a] = v[a:b]
            vpool[pg] = value_tiles(full).reshape(page, nkv * hd)
    return ks, vs, kpool.to(DEV), vpool.to(DEV), table.to(DEV)


def attention_reference(qs, ks, vs, positions, seq_of, nh, scale, allowed=None):
    out = []
    nkv = ks[0].shape[1]
    G = nh // nkv
    for t, (p, s) in enumerate(zip(positions, seq_of)):
        k, v = ks[s][:p + 1], vs[s][:p + 1]
        row = []
        for h in range(nh):
            sc = (k[:, h // G] @ qs[t, h]) * scale
            if allowed is not None:
                sc = sc.masked_fill(~allowed[t][h // G][:p + 1], float("-inf"))
            row.append(torch.softmax(sc, 0) @ v[:, h // G])
        out.append(torch.stack(row))
    return torch.stack(out)


@pytest.mark.parametrize("nh,nkv,hd", [(4, 2, 16), (3, 1, 32), (6, 3, 64), (32, 2, 128), (20, 1, 32), (2, 2, 48), (4, 1, 256),
                                       (6, 2, 80), (3, 1, 96), (4, 4, 112)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_over_scrambled_pages(nh, nkv, hd, dtype):
    """Prompt tokens and single tokens of three sequences at once; plain kernel, and the matrix-core kernel
    with 1, 3 and 8 shares of the keys where it takes the head size."""
    from cpmcu_amd import ops
    page = 64
    lens = [300, 70, 1]
    ks, vs, kpool, vpool, table = paged_setup(lens, nkv, hd, page, dtype, seed=hd)
    # queries: the last 40 positions of sequence 0, the last of sequence 1, the only one of sequence 2
    positions = list(range(260, 300)) + [69, 0]
    seq_of = [0] * 40 + [1, 2]
    n = len(positions)
    q = rnd(n, nh, hd, seed=5, dtype=dtype)
    scale = hd ** -0.5
    ref = attention_reference(q.double().cpu(), ks, vs, positions, seq_of, nh, scale)
    pos_t = torch.tensor(positions, dtype=torch.int32, device=DEV)
    slot_t = torch.tensor(seq_of, dtype=torch.int32, device=DEV)
    tol = 2e-6 if dtype == torch.float32 else 2 ** -7
    out = torch.empty(n, nh * hd, dtype=dtype, device=DEV)
    ops.attention_plain(q.view(n, -1), out, nh, nkv, hd, scale, kpool, vpool, table, page, pos_t, slot_t)
    assert float((out.double().cpu().view(n, nh, hd) - ref).abs().max()) <= tol
    if dtype == torch.bfloat16 and hd in ops.MFMA_HEAD_DIMS:
        for splits, nw in ((1, 1), (1, 4), (3, 1), (3, 4), (8, 4)):
            out.fill_(float("nan"))
            po = torch.full((n, nh, splits, hd), float("nan"), device=DEV) if splits > 1 else None
            pm = torch.full((n, nh, splits, 2), float("nan"), device=DEV) if splits > 1 else None
            ops.attention_mfma(q.view(n, -1), out, nh, nkv, hd, scale, kpool, vpool, table, page, pos_t, slot_t,
                               splits, po, pm, waves_per_group=nw)
            assert float((out.double().cpu().view(n, nh, hd) - ref).abs().max()) <= tol, f"splits={splits} waves={nw}"
        # the prompt kernel: runs of consecutive tokens of one sequence share a wavefront
        for r, nw in ((2, 1), (4, 1), (2, 2), (4, 2), (2, 4), (4, 4)):
            tpw = ops.attention_prefill_tokens_per_wave(nh, nkv, r)
            tiles = ops.prefill_tiles([40, 1, 1], tpw, DEV)
            out.fill_(float("nan"))
            ops.attention_prefill_mfma(q.view(n, -1), out, tiles, nh, nkv, hd, scale, kpool, vpool, table, page, pos_t,
                                       slot_t, r, nw)
            assert float((out.double().cpu().view(n, nh, hd) - ref).abs().max()) <= tol, "prompt kernel"
    elif dtype == torch.bfloat16:
        assert not ops.attention_mfma_ok(q.view(n, -1), hd, page)


@pytest.mark.parametrize("nh,nkv,hd", [(16, 1, 64), (8, 1, 32), (4, 2, 128), (5, 5, 16), (40, 2, 32), (6, 2, 48), (2, 1, 96)])
def test_prompt_attention_from_position_zero_and_continued(nh, nkv, hd):
    """Whole prompts from position 0 (where early tiles stop before late chunks) and a chunk that continues
    a sequence already in the cache, several sequences packed."""
    from cpmcu_amd import ops
    page, dtype = 64, torch.bfloat16
    lens = [150, 37, 64]
    ks, vs, kpool, vpool, table = paged_setup(lens, nkv, hd, page, dtype, seed=nh)
    starts = [0, 0, 41]                       # the third sequence already holds 41 tokens
    positions, seq_of, q_lens = [], [], []
    for s, (L, a) in enumerate(zip(lens, starts)):
        positions += list(range(a, L))
        seq_of += [s] * (L - a)
        q_lens.append(L - a)
    n = len(positions)
    q = rnd(n, nh, hd, seed=8, dtype=dtype)
    scale = hd ** -0.5
    ref = attention_reference(q.double().cpu(), ks, vs, positions, seq_of, nh, scale)
    pos_t = torch.tensor(positions, dtype=torch.int32, device=DEV)
    slot_t = torch.tensor(seq_of, dtype=torch.int32, device=DEV)
    for r, nw in ((2, 1), (4, 1), (2, 2), (4, 2), (2, 4), (4, 4)):
        tiles = ops.prefill_tiles(q_lens, ops.attention_prefill_tokens_per_wave(nh, nkv, r), DEV)
        out = torch.full((n, nh * hd), float("nan"), dtype=dtype, device=DEV)
        ops.attention_prefill_mfma(q.view(n, -1), out, tiles, nh, nkv, hd, scale, kpool, vpool, table, page, pos_t,
                                   slot_t, r, nw)
        # the output is rounded to bf16 (8 significant bits): allow its half ulp at the size of each token's values
        err = (out.double().cpu().view(n, nh, hd) - ref).abs().amax(dim=(1, 2))
        bad = (err > 2 ** -7 * ref.abs().amax(dim=(1, 2)).clamp(min=1.0)).nonzero().flatten()
        assert bad.numel() == 0, f"first wrong token {int(bad[0])} (position {positions[int(bad[0])]}), {r} tiles, {nw} waves"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nh,nkv,hd", [(6, 2, 48), (5, 1, 16)])
def test_attention_with_a_distance_bias(nh, nkv, hd, dtype):
    """head_slopes: the score of key j for the query at p is lowered by slope[head] * (p - j).  Checked against
    a library attention with that bias as its mask; a slope that large for one head that only the nearest keys
    count shows a wrong sign or a wrong head at once."""
    from cpmcu_amd import ops
    page = 64
    lens = [200, 33]
    ks, vs, kpool, vpool, table = paged_setup(lens, nkv, hd, page, dtype, seed=hd + 1)
    positions = list(range(150, 200)) + [32, 0]
    seq_of = [0] * 50 + [1, 1]
    n = len(positions)
    q = rnd(n, nh, hd, seed=6, dtype=dtype)
    slopes = torch.tensor([0.0, 0.01, 0.3, 12.0, 0.05, 1.0][:nh], dtype=torch.float32)
    G = nh // nkv
    ref = torch.empty(n, nh, hd, dtype=torch.float64)
    for t, (p, s) in enumerate(zip(positions, seq_of)):
        k, v = ks[s][:p + 1], vs[s][:p + 1]                      # [keys, nkv, hd]
        dist = (p - torch.arange(p + 1, dtype=torch.float64))
        mask = (-slopes.double()[:, None] * dist[None, :])[:, None, :]            # [head, 1, key]
        ref[t] = F.scaled_dot_product_attention(q[t].double().cpu()[:, None, :], k.repeat_interleave(G, 1).transpose(0, 1),
                                                v.repeat_interleave(G, 1).transpose(0, 1), attn_mask=mask)[:, 0]
    out = torch.empty(n, nh * hd, dtype=dtype, device=DEV)
    ops.attention_plain(q.view(n, -1), out, nh, nkv, hd, hd ** -0.5, kpool, vpool, table, page,
                        torch.tensor(positions, dtype=torch.int32, device=DEV),
                        torch.tensor(seq_of, dtype=torch.int32, device=DEV), head_slopes=slopes.to(DEV))
    tol = 2e-6 if dtype == torch.float32 else 2 ** -7
    assert float((out.double().cpu().view(n, nh, hd) - ref).abs().max()) <= tol
    # the head with slope 12 sees (almost) only the query's own position: its output is that position's value
    own = torch.stack([vs[s][p, 3 // G] for p, s in zip(positions, seq_of)])
    assert float((out.double().cpu().view(n, nh, hd)[:, 3] - own).abs().max()) < 0.02
    with pytest.raises(ops.KernelError, match="head slopes"):
        ops.attention_plain(q.view(n, -1), out, nh, nkv, hd, hd ** -0.5, kpool, vpool, table, page,
                            torch.tensor(positions, dtype=torch.int32, device=DEV),
                            torch.tensor(seq_of, dtype=torch.int32, device=DEV), head_slopes=slopes[:2].to(DEV))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_finds_one_far_key_among_hundreds(dtype):
    """One key far back is made to stand out: the output must be its value (a kernel that skips or misplaces
    a page, or mixes up the transposed values, fails this)."""
    from cpmcu_amd import ops
    nh, nkv, hd, page = 16, 1, 64, 64
    L = 1000
    ks, vs, kpool, vpool, table = paged_setup([L], nkv, hd, page, dtype, seed=3)
    for far in (0, 63, 64, 517, 998, 999):
        k = ks[0].clone()
        q = torch.zeros(1, nh, hd, dtype=torch.float64)
        q[0, :, 5] = 40.0
        pg, off = int(table[0, far // page]), far % page
        where = key_elements(off, 0, nkv, hd, page).to(DEV)
        flat = kpool[pg].view(-1)
        saved = flat[where].clone()
        one = torch.zeros(hd, dtype=dtype, device=DEV)
        one[5] = 40.0
        flat[where] = one
        pos_t = torch.tensor([L - 1], dtype=torch.int32, device=DEV)
        slot_t = torch.zeros(1, dtype=torch.int32, device=DEV)
        qd = q.to(dtype).to(DEV).view(1, -1)
        outs = []
        out = torch.empty(1, nh * hd, dtype=dtype, device=DEV)
        ops.attention_plain(qd, out, nh, nkv, hd, hd ** -0.5, kpool, vpool, table, page, pos_t, slot_t)
        outs.append(out.clone())
        if dtype == torch.bfloat16:
            for splits, nw in ((1, 1), (1, 4), (5, 4), (5, 1)):
                po = torch.empty(1, nh, splits, hd, device=DEV)
                pm = torch.empty(1, nh, splits, 2, device=DEV)
                ops.attention_mfma(qd, out, nh, nkv, hd, hd ** -0.5, kpool, vpool, table, page, pos_t, slot_t, splits,
                                   po, pm, waves_per_group=nw)
                outs.append(out.clone())
        for o in outs:
            assert float((o.double().cpu().view(nh, hd) - vs[0][far, 0]).abs().max()) < 1e-2, far
        flat[where] = saved


@pytest.mark.parametrize("bs", [16, 32, 64])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_with_block_lists(bs, dtype):
    """Only the listed key blocks are attended to; a count of -1 means all keys."""
    from cpmcu_amd import ops
    nh, nkv, hd, page = 6, 2, 32, 64
    L = 400
    ks, vs, kpool, vpool, table = paged_setup([L], nkv, hd, page, dtype, seed=9)
    positions = [399, 250, 131, 64]
    n = len(positions)
    q = rnd(n, nh, hd, seed=2, dtype=dtype)
    max_sel = 6
    sel_blocks = torch.zeros(n, nkv, max_sel, dtype=torch.int32)
    sel_count = torch.zeros(n, nkv, dtype=torch.int32)
    allowed = torch.zeros(n, nkv, L, dtype=torch.bool)
    g = torch.Generator().manual_seed(1)
    for t, p in enumerate(positions):
        for h in range(nkv):
            if t == 2 and h == 1:
                sel_count[t, h] = -1
                allowed[t, h] = True
                continue
            own = p // bs
            cand = torch.randperm(own, generator=g)[:4].tolist() if own > 0 else []
            blocks = sorted(set(cand + [own]))
            sel_count[t, h] = len(blocks)
            sel_blocks[t, h, :len(blocks)] = torch.tensor(blocks, dtype=torch.int32)
            for b in blocks:
                allowed[t, h, b * bs:(b + 1) * bs] = True
    ref = attention_reference(q.double().cpu(), ks, vs, positions, [0] * n, nh, hd ** -0.5, allowed)
    pos_t = torch.tensor(positions, dtype=torch.int32, device=DEV)
    slot_t = torch.zeros(n, dtype=torch.int32, device=DEV)
    out = torch.empty(n, nh * hd, dtype=dtype, device=DEV)
    tol = 2e-6 if dtype == torch.float32 else 2 ** -7
    ops.attention_plain(q.view(n, -1), out, nh, nkv, hd, hd ** -0.5, kpool, vpool, table, page, pos_t, slot_t,
                        sel_blocks.to(DEV), sel_count.to(DEV), bs)
    assert float((out.double().cpu().view(n, nh, hd) - ref).abs().max()) <= tol
    if dtype == torch.bfloat16 and bs % 32 == 0:
        for splits, nw in ((1, 1), (4, 4), (1, 4)):
            po = torch.empty(n, nh, splits, hd, device=DEV)
            pm = torch.empty(n, nh, splits, 2, device=DEV)
            ops.attention_mfma(q.view(n, -1), out, nh, nkv, hd, hd ** -0.5, kpool, vpool, table, page, pos_t, slot_t,
                               splits, po, pm, sel_blocks.to(DEV), sel_count.to(DEV), bs, waves_per_group=nw)
            assert float((out.double().cpu().view(n, nh, hd) - ref).abs().max()) <= tol


@pytest.mark.parametrize("first", [0, 2, 100])
def test_block_lists_of_a_prompt_chunk_in_any_visiting_order(first):
    """Steps of many tokens give each wavefront of a workgroup a token of its own and may visit the last blocks
    of every list first: neither changes which keys count."""
    from cpmcu_amd import ops
    nh, nkv, hd, page, bs = 6, 2, 32, 64, 32
    L = 400
    ks, vs, kpool, vpool, table = paged_setup([L], nkv, hd, page, torch.bfloat16, seed=11)
    positions = list(range(329, 400))                 # 71 tokens: the last workgroup is not full
    n = len(positions)
    q = rnd(n, nh, hd, seed=4, dtype=torch.bfloat16)
    max_sel = 7
    sel_blocks = torch.zeros(n, nkv, max_sel, dtype=torch.int32)
    sel_count = torch.zeros(n, nkv, dtype=torch.int32)
    allowed = torch.zeros(n, nkv, L, dtype=torch.bool)
    g = torch.Generator().manual_seed(5)
    for t, p in enumerate(positions):
        for h in range(nkv):
            if t % 17 == 3 and h == 0:
                sel_count[t, h] = -1
                allowed[t, h] = True
                continue
            own = p // bs
            blocks = sorted(set(torch.randperm(own - 1, generator=g)[:4].tolist() + [own - 1, own]))
            sel_count[t, h] = len(blocks)
            sel_blocks[t, h, :len(blocks)] = torch.tensor(blocks, dtype=torch.int32)
            for b in blocks:
                allowed[t, h, b * bs:(b + 1) * bs] = True
    ref = attention_reference(q.double().cpu(), ks, vs, positions, [0] * n, nh, hd ** -0.5, allowed)
    pos_t = torch.tensor(positions, dtype=torch.int32, device=DEV)
    slot_t = torch.zeros(n, dtype=torch.int32, device=DEV)
    out = torch.empty(n, nh * hd, dtype=torch.bfloat16, device=DEV)
    ops.attention_mfma(q.view(n, -1), out, nh, nkv, hd, hd ** -0.5, kpool, vpool, table, page, pos_t, slot_t,
                       1, None, None, sel_blocks.to(DEV), sel_count.to(DEV), bs, last_blocks_first=first)
    assert float((out.double().cpu().view(n, nh, hd) - ref).abs().max()) <= 2 ** -7


# ---------------------------------------------------------------------------- fused projection of decode steps
def read_cache_rows(pool, table, page, nkv, hd, slot, positions, tiles):
    """Rows [position][kv head][d] out of a paged pool whose pages lie as `tiles` (key_tiles / value_tiles) lays them."""
    probe = torch.arange(page * nkv * hd, dtype=torch.float64).view(page, nkv, hd)
    where = tiles(probe).reshape(-1).long()                      # flat place -> (token, kv head, d) index
    inv = torch.empty_like(where)
    inv[where] = torch.arange(where.numel())
    out = []
    for p in positions:
        flat = pool[int(table[slot, p // page])].reshape(-1).cpu()
        out.append(flat[inv.view(page, nkv, hd)[p % page]])
    return torch.stack(out)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n,nh,nkv,hd,parts,rotate,write_kv", [
    (1, 4, 2, 16, 0, True, True), (7, 5, 1, 48, 3, True, True), (70, 6, 2, 32, 0, True, True),
    (130, 32, 2, 128, 0, True, True), (67, 3, 3, 64, 0, False, True), (9, 2, 1, 80, 2, True, False),
    (100, 4, 1, 112, 0, True, False)])
def test_rotary_and_cache_write(dtype, n, nh, nkv, hd, parts, rotate, write_kv):
    """rope_store alone (the kernel of few tokens, which also sums a split product's partial sums, and the kernel
    of prompt chunks in bfloat16): q rotated into q_out, k rotated and v as they are into the pages, read back
    through the pages' layout; pairs (c, c + hd/2), angle = position * inv_freq[c], cos and sin times the
    magnitude; tokens of several slots at scattered positions."""
    from cpmcu_amd import ops
    page = 64
    width = (nh + 2 * nkv) * hd
    g = torch.Generator().manual_seed(n * 7 + hd)
    src = torch.randn((parts, n, width) if parts else (n, width), generator=g)
    src = src.to(dtype if not parts else torch.float32)              # partial sums are float32
    slots = torch.randint(0, 3, (n,), generator=g)
    positions = torch.randperm(190, generator=g)[:n]                 # distinct, so no two tokens share a cache row
    table = torch.randperm(12, generator=g)[:9].view(3, 3).to(torch.int32)
    inv_freq = (torch.rand(hd // 2, generator=g) * 0.5 + 0.01) if rotate else None
    mscale = 1.25 if rotate else 1.0
    kpool = torch.zeros(12, page, nkv * hd, dtype=dtype, device=DEV)
    vpool = torch.zeros_like(kpool)
    q_out = torch.full((n, nh * hd), float("nan"), dtype=dtype, device=DEV)
    ops.rope_store(src.to(DEV), q_out, nh, nkv, hd, positions.to(torch.int32).to(DEV), slots.to(torch.int32).to(DEV),
                   inv_freq.to(DEV) if rotate else None, mscale, kpool if write_kv else None,
                   vpool if write_kv else None, table.to(DEV) if write_kv else None, page, write_kv)
    y = (src.double().sum(0) if parts else src.double()).view(n, nh + 2 * nkv, hd).clone()
    if rotate:
        ang = positions.double()[:, None] * inv_freq.float().double()[None, :]
        cs, sn = (torch.cos(ang) * mscale)[:, None, :], (torch.sin(ang) * mscale)[:, None, :]
        a, b = y[:, :nh + nkv, :hd // 2].clone(), y[:, :nh + nkv, hd // 2:].clone()
        y[:, :nh + nkv] = torch.cat([a * cs - b * sn, a * sn + b * cs], dim=-1)
    tol = (1e-5 if dtype == torch.float32 else 2 ** -7) * max(1.0, float(y.abs().max()))
    assert float((q_out.double().cpu().view(n, nh, hd) - y[:, :nh]).abs().max()) <= tol
    if write_kv:
        for t in range(n):
            k_row = read_cache_rows(kpool, table, page, nkv, hd, int(slots[t]), [int(positions[t])], key_tiles)[0]
            v_row = read_cache_rows(vpool, table, page, nkv, hd, int(slots[t]), [int(positions[t])], value_tiles)[0]
            assert float((k_row.double() - y[t, nh:nh + nkv]).abs().max()) <= tol, t
            assert float((v_row.double() - y[t, nh + nkv:]).abs().max()) <= tol, t
        assert int((kpool != 0).sum()) <= n * nkv * hd and int((vpool != 0).sum()) <= n * nkv * hd


@pytest.mark.parametrize("n,nh,nkv,hd,H,rotate", [(1, 4, 2, 16, 64, True), (8, 32, 2, 128, 512, True), (16, 3, 1, 32, 96, True),
                                                  (5, 6, 3, 64, 200, False), (13, 2, 2, 48, 264, True),
                                                  (17, 4, 2, 32, 136, True), (24, 2, 1, 64, 1160, True), (32, 6, 2, 16, 72, True),
                                                  (33, 2, 1, 32, 392, True), (64, 5, 1, 16, 1032, True)])
@pytest.mark.parametrize("scaled", [False, True])
@pytest.mark.parametrize("R", [None, 18, 26, 32])
def test_fused_projection_rotation_and_cache_write(n, nh, nkv, hd, H, rotate, scaled, R):
    """q, k, v of a decode step in one kernel: against the float64 product, rotation (pairs c, c + hd/2) and the
    cache rows read back through the pages' layout; tokens of several slots at scattered positions.  R: rows of
    the weight a workgroup owns (None: the library's choice, 16 at these sizes; more than 16 rows straddle
    heads, and the last workgroup is not full)."""
    from cpmcu_amd import ops
    page = 64
    w = rnd((nh + 2 * nkv) * hd, H, seed=1, dtype=torch.bfloat16, scale=H ** -0.5)
    x = rnd(n, H, seed=2, dtype=torch.bfloat16)
    g = torch.Generator().manual_seed(n)
    slots = torch.randint(0, 3, (n,), generator=g)
    positions = torch.randperm(190, generator=g)[:n]             # distinct, so no two tokens share a cache row
    table = torch.randperm(12, generator=g)[:9].view(3, 3).to(torch.int32)
    inv_freq = (torch.rand(hd // 2, generator=g) * 0.5 + 0.01) if rotate else None
    mscale = 1.25
    kpool = torch.zeros(12, page, nkv * hd, dtype=torch.bfloat16, device=DEV)
    vpool = torch.zeros_like(kpool)
    q_out = torch.empty(n, nh * hd, dtype=torch.bfloat16, device=DEV)
    wt = ops.qkv_rope_weight(w, nh, nkv, hd, R)
    # with the row factor of a norm cut by columns (the sums need not belong to x: any positive numbers do)
    row_scale, r = None, 1.0
    if scaled:
        sums = torch.rand(n, ops.norm_slices(H), generator=g) + 0.1
        row_scale = ops.RowScale(sums.to(DEV), 1e-3)
        r = torch.rsqrt(sums.double().sum(1) / H + 1e-3).view(n, 1, 1)
    ops.qkv_rope(x, wt, q_out, nh, nkv, hd, positions.to(torch.int32).to(DEV), slots.to(torch.int32).to(DEV),
                 inv_freq.to(DEV) if rotate else None, mscale if rotate else 1.0, kpool, vpool, table.to(DEV), page,
                 row_scale=row_scale)
    y = (x.double().cpu() @ w.double().cpu().T).view(n, nh + 2 * nkv, hd) * r
    if rotate:
        ang = positions.double()[:, None] * inv_freq.float().double()[None, :]          # angles formed in float32 on the GPU
        cs, sn = (torch.cos(ang) * mscale)[:, None, :], (torch.sin(ang) * mscale)[:, None, :]
        a, b = y[:, :nh + nkv, :hd // 2], y[:, :nh + nkv, hd // 2:]
        y[:, :nh + nkv] = torch.cat([a * cs - b * sn, a * sn + b * cs], dim=-1)
    tol = 2 ** -7 * max(1.0, float(y.abs().max()))
    assert float((q_out.double().cpu().view(n, nh, hd) - y[:, :nh]).abs().max()) <= tol
    for t in range(n):
        k_row = read_cache_rows(kpool, table, page, nkv, hd, int(slots[t]), [int(positions[t])], key_tiles)[0]
        v_row = read_cache_rows(vpool, table, page, nkv, hd, int(slots[t]), [int(positions[t])], value_tiles)[0]
        assert float((k_row.double() - y[t, nh:nh + nkv]).abs().max()) <= tol, t
        assert float((v_row.double() - y[t, nh + nkv:]).abs().max()) <= tol, t
    # nothing but the n rows was written
    assert int((kpool != 0).sum()) <= n * nkv * hd and int((vpool != 0).sum()) <= n * nkv * hd


@pytest.mark.parametrize("n,ks,st", [(16, 8, 4), (5, 32, 16), (32, 12, 4), (1, 32, 16), (50, 8, 4)])
@pytest.mark.parametrize("R", [None, 18, 30])
def test_fused_projection_completes_compressed_keys(n, ks, st, R):
    """The projection kernel of decode steps also writes the compressed keys that its tokens complete: bit for
    bit what compress_keys writes after it, from keys of earlier steps and of this step (two sequences, each
    with consecutive tokens in the step, at different phases of the stride)."""
    from cpmcu_amd import ops
    nh, nkv, hd, H, page = 4, 2, 32, 136, 64
    w = rnd((nh + 2 * nkv) * hd, H, seed=1, dtype=torch.bfloat16, scale=H ** -0.5)
    x = rnd(n, H, seed=2, dtype=torch.bfloat16)
    g = torch.Generator().manual_seed(ks)
    n0 = (n + 1) // 2
    first = (47 if n > 1 else 16 * 5 + 32 - 1, 70)           # the lone token completes a compressed key
    positions = torch.tensor([first[0] + i for i in range(n0)] + [first[1] + i for i in range(n - n0)], dtype=torch.int32)
    slots = torch.tensor([0] * n0 + [1] * (n - n0), dtype=torch.int32)
    table = torch.randperm(8, generator=g).view(2, 4).to(torch.int32)
    inv_freq = torch.rand(hd // 2, generator=g) * 0.5 + 0.01
    wt = ops.qkv_rope_weight(w, nh, nkv, hd, R)
    results = []
    for fused in (True, False):
        kpool = rnd(8, page, nkv * hd, seed=5, dtype=torch.bfloat16)        # the keys of earlier steps
        vpool = torch.zeros_like(kpool)
        ck = torch.zeros(8, page // st, nkv * hd, dtype=torch.bfloat16, device=DEV)
        q_out = torch.empty(n, nh * hd, dtype=torch.bfloat16, device=DEV)
        ops.qkv_rope(x, wt, q_out, nh, nkv, hd, positions.to(DEV), slots.to(DEV), inv_freq.to(DEV), 1.0, kpool, vpool,
                     table.to(DEV), page, compress=(ck, ks, st) if fused else None)
        if not fused:
            ops.compress_keys(kpool, ck, nkv, table.to(DEV), page, positions.to(DEV), slots.to(DEV), ks, st)
        results.append((kpool, ck, q_out))
    (ka, ca, qa), (kb, cb, qb) = results
    assert torch.equal(ka, kb) and torch.equal(qa, qb)
    completed = sum(1 for p in positions.tolist() if p + 1 >= ks and (p + 1 - ks) % st == 0)
    assert completed > 0 and int((cb != 0).sum()) > 0
    assert torch.equal(ca, cb)


# ---------------------------------------------------------------------------- InfLLM-v2 kernels
@pytest.mark.parametrize("ks,st", [(8, 4), (32, 16), (16, 16), (12, 4)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_compressed_keys_are_means_written_when_their_last_key_arrives(ks, st, dtype):
    from cpmcu_amd import ops
    nkv, hd, page = 2, 16, 64
    lens = [150, 37]
    kseq, vs, kpool, vpool, table = paged_setup(lens, nkv, hd, page, dtype, seed=ks)
    ck = torch.zeros(kpool.shape[0], page // st, nkv * hd, dtype=dtype, device=DEV)
    # two steps: first the tokens up to 100 / 20, then the rest (compressed keys that straddle the cut
    # are completed by the second step)
    for a0, b0, a1, b1 in ((0, 100, 0, 20), (100, 150, 20, 37)):
        positions = list(range(a0, b0)) + list(range(a1, b1))
        slots = [0] * (b0 - a0) + [1] * (b1 - a1)
        ops.compress_keys(kpool, ck, nkv, table, page, torch.tensor(positions, dtype=torch.int32, device=DEV),
                          torch.tensor(slots, dtype=torch.int32, device=DEV), ks, st)
    for s, L in enumerate(lens):
        ref = F.avg_pool1d(kseq[s].reshape(L, -1).T[None], ks, st)[0].T        # [n_ck, nkv*hd]
        # a page of compressed keys lies [kv head][d / 8][row][d % 8]
        got = torch.stack([ck[int(table[s, (st * j) // page])].view(nkv, hd // 8, page // st, 8)
                           [:, :, ((st * j) % page) // st].reshape(nkv * hd) for j in range(ref.shape[0])])
        tol = 1e-6 if dtype == torch.float32 else 2 ** -8
        assert float((got.double().cpu() - ref).abs().max()) <= tol * float(ref.abs().max() + 1)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nh,nkv,hd", [(6, 2, 16), (32, 2, 128), (20, 1, 32), (8, 2, 48), (3, 1, 96)])
@pytest.mark.parametrize("ks,st,bs,init,topk,window,dense_len", [(8, 4, 16, 1, 4, 32, 64), (32, 16, 64, 1, 3, 128, 0),
                                                              (8, 8, 32, 2, 2, 32, 100), (16, 4, 16, 0, 5, 16, 0)])
def test_block_selection_equals_the_plain_selection(dtype, nh, nkv, hd, ks, st, bs, init, topk, window, dense_len):
    """Positions at block edges, window edges, just past dense_len and where compressed keys become visible."""
    import plain_minicpm as plain
    from cpmcu_amd import ops
    page = 64
    L = 460
    kseq, vs, kpool, vpool, table = paged_setup([L], nkv, hd, page, dtype, seed=bs + topk)
    ck = torch.zeros(kpool.shape[0], page // st, nkv * hd, dtype=dtype, device=DEV)
    allpos = torch.arange(L, dtype=torch.int32, device=DEV)
    ops.compress_keys(kpool, ck, nkv, table, page, allpos, torch.zeros(L, dtype=torch.int32, device=DEV), ks, st)
    sc = {"kernel_size": ks, "kernel_stride": st, "block_size": bs, "init_blocks": init, "topk": topk,
          "window_size": window, "dense_len": dense_len}
    positions = sorted(set([0, 1, ks - 1, ks, ks + 1, bs - 1, bs, bs + 1, window - 1, window, window + bs - 1, window + bs,
                            max(dense_len - 1, 0), dense_len, dense_len + 1, 255, 256, 257, 300, 399, 400, L - 1]))
    positions = [p for p in positions if 0 <= p < L]
    n = len(positions)
    q = rnd(n, nh, hd, seed=4, dtype=dtype)
    lb = window // bs
    sel_blocks = torch.full((n, nkv, topk + lb), -7, dtype=torch.int32, device=DEV)
    sel_count = torch.full((n, nkv), -7, dtype=torch.int32, device=DEV)
    # plain selection from the same (rounded) keys; compressed keys in the cache's own precision
    ck_ref = plain.compressed_keys(kseq[0], ks, st).to(dtype).double()
    # the matrix-core kernel, its forms for steps of few tokens (two kernels, or three when the last does not
    # normalise the scores itself), and the plain twin
    scratch = torch.full((ops.sparse_select_scratch(dtype, n, nh, nkv, hd, max(positions), ks, st, bs),), float("nan"), device=DEV)
    for force_plain, scr in (((False, None), (False, scratch), (2, scratch), (True, None)) if dtype == torch.bfloat16
                             else ((True, None),)):
        sel_blocks.fill_(-7)
        sel_count.fill_(-7)
        ops.sparse_select(q.view(n, -1), ck, nh, nkv, hd, hd ** -0.5, table, page,
                          torch.tensor(positions, dtype=torch.int32, device=DEV),
                          torch.zeros(n, dtype=torch.int32, device=DEV),
                          ks, st, bs, init, topk, lb, dense_len, max(positions), sel_blocks, sel_count, force_plain,
                          scratch=scr)
        for t, p in enumerate(positions):
            want = plain.infllm_select(q[t].double().cpu(), ck_ref, p, sc, nkv)
            for h in range(nkv):
                c = int(sel_count[t, h])
                if want is None:
                    assert c == -1, (p, h)
                else:
                    assert sel_blocks[t, h, :c].tolist() == want[h], (p, h, want[h], force_plain, scr is not None)


def test_block_selection_ties_and_forced_blocks():
    """All compressed keys equal: every score ties and the lowest blocks win; initial blocks count toward topk."""
    from cpmcu_amd import ops
    nh, nkv, hd, page, ks, st, bs = 2, 1, 16, 64, 8, 4, 16
    L = 208
    kpool = torch.ones(5, page, nkv * hd, device=DEV)
    table = torch.tensor([[3, 1, 4, 0]], dtype=torch.int32, device=DEV)
    ck = torch.zeros(5, page // st, nkv * hd, device=DEV)
    ops.compress_keys(kpool, ck, nkv, table, page, torch.arange(L, dtype=torch.int32, device=DEV),
                      torch.zeros(L, dtype=torch.int32, device=DEV), ks, st)
    q = torch.ones(1, nh * hd, device=DEV)
    for dtype in (torch.float32, torch.bfloat16):
        for init, topk, want in ((0, 3, [0, 1, 2, 11, 12]), (2, 2, [0, 1, 11, 12]), (1, 20, list(range(13)))):
            sb = torch.zeros(1, 1, topk + 2, dtype=torch.int32, device=DEV)
            cnt = torch.zeros(1, 1, dtype=torch.int32, device=DEV)
            for scr in ((None, torch.zeros(ops.sparse_select_scratch(dtype, 1, nh, nkv, hd, 200, ks, st, bs), device=DEV))
                        if dtype == torch.bfloat16 else (None,)):
                sb.zero_()
                cnt.zero_()
                ops.sparse_select(q.to(dtype), ck.to(dtype), nh, nkv, hd, 0.25, table, page,
                                  torch.tensor([200], dtype=torch.int32, device=DEV),
                                  torch.zeros(1, dtype=torch.int32, device=DEV), ks, st, bs, init, topk, 2, 0, 200, sb,
                                  cnt, scratch=scr)
                assert sb[0, 0, :int(cnt[0, 0])].tolist() == want, (dtype, scr is not None)
