"""The attention entry point that allocates nothing (cpmcu_attention_mfma_static), called through ctypes as a
caller without torch's allocator would: its output must equal that of cpmcu_attention_mfma with a workspace,
on two calls in a row (the second with a smaller input, so that what the first call left in the library's own
scratch lies beside and behind the second call's shares), and a call too large for that scratch is refused.
This file is collected last: a failure here must not hide the tests before it."""
import ctypes
from ctypes import c_char_p, c_float, c_int, c_void_p

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _entry_points():
    from cpmcu_amd.csrc import build
    lib = build.load("attention")
    new, old = lib.cpmcu_attention_mfma_static, lib.cpmcu_attention_mfma
    new.restype = old.restype = c_char_p
    return new, old


def _ptr(t):
    return c_void_p(0 if t is None else t.data_ptr())


def _call_pair(new, old, lens, n_tok, nh, nkv, hd, splits, seed):
    """Both entry points on the same inputs; returns (static, workspace) outputs."""
    from test_kernels_gpu import paged_setup, rnd
    page = 64
    ks, vs, kpool, vpool, table = paged_setup(lens, nkv, hd, page, torch.bfloat16, seed=seed)
    positions, slots = [], []
    for s, L in enumerate(lens):
        take = min(n_tok, L)
        positions += list(range(L - take, L))
        slots += [s] * take
    n = len(positions)
    q = rnd(n, nh * hd, seed=seed + 1, dtype=torch.bfloat16)
    pos_t = torch.tensor(positions, dtype=torch.int32, device=DEV)
    slot_t = torch.tensor(slots, dtype=torch.int32, device=DEV)
    out_new = torch.full((n, nh * hd), float("nan"), dtype=torch.bfloat16, device=DEV)
    out_old = torch.full((n, nh * hd), float("nan"), dtype=torch.bfloat16, device=DEV)
    po = torch.full((n, nh, splits, hd), float("nan"), device=DEV)
    pm = torch.full((n, nh, splits, 2), float("nan"), device=DEV)
    stream = c_void_p(torch.cuda.current_stream().cuda_stream)
    scale = c_float(hd ** -0.5)
    common = (c_int(n), c_int(nh), c_int(nkv), c_int(hd), scale, _ptr(kpool), _ptr(vpool), _ptr(table),
              c_int(table.shape[1]), c_int(page), _ptr(pos_t), _ptr(slot_t), _ptr(None), _ptr(None), c_int(0), c_int(0),
              c_int(splits), c_int(0), c_int(0))
    torch.cuda.synchronize()
    msg = new(_ptr(q), _ptr(out_new), *common, stream)
    assert msg is None, msg
    msg = old(_ptr(q), _ptr(out_old), _ptr(po), _ptr(pm), *common, stream)
    assert msg is None, msg
    torch.cuda.synchronize()
    return out_new, out_old


def test_static_scratch_attention_equals_workspace_attention_twice():
    new, old = _entry_points()
    # first call: 3 sequences x 4 tokens, 8 shares; second call: smaller in every size
    a_new, a_old = _call_pair(new, old, [900, 300, 70], 4, 8, 2, 64, 8, seed=11)
    assert not bool(a_old.isnan().any())
    assert torch.equal(a_new, a_old)
    b_new, b_old = _call_pair(new, old, [500], 1, 4, 1, 32, 3, seed=12)
    assert not bool(b_old.isnan().any())
    assert torch.equal(b_new, b_old)
    # and one share: no scratch at all
    c_new, c_old = _call_pair(new, old, [200, 64], 2, 6, 3, 48, 1, seed=13)
    assert torch.equal(c_new, c_old)


def test_static_scratch_attention_refuses_what_does_not_fit():
    new, _ = _entry_points()
    n, nh, nkv, hd, splits = 256, 64, 2, 128, 64        # 256 * 64 * 64 * 130 floats = 545 MB of shares
    q = torch.zeros(n, nh * hd, dtype=torch.bfloat16, device=DEV)
    out = torch.full_like(q, 3.0)
    pool = torch.zeros(2, 64, nkv * hd, dtype=torch.bfloat16, device=DEV)
    table = torch.zeros(1, 1, dtype=torch.int32, device=DEV)
    pos = torch.zeros(n, dtype=torch.int32, device=DEV)
    msg = new(_ptr(q), _ptr(out), c_int(n), c_int(nh), c_int(nkv), c_int(hd), c_float(0.1), _ptr(pool), _ptr(pool),
              _ptr(table), c_int(1), c_int(64), _ptr(pos), _ptr(pos), _ptr(None), _ptr(None), c_int(0), c_int(0),
              c_int(splits), c_int(0), c_int(0), c_void_p(torch.cuda.current_stream().cuda_stream))
    assert msg is not None and b"exceed the library's own scratch" in msg
    torch.cuda.synchronize()
    assert bool((out == 3.0).all())          # nothing was launched
