"""Python face of the HIP kernels: argument checks, then one launch each.

Tensors are torch tensors on the GPU, used as typed memory only; every function
launches on torch's current stream and allocates nothing.  Shapes are checked
here, on the host, before a pointer reaches a kernel; a size a kernel does not
take is refused with an error that names it.  There is no fallback: without a
GPU or without the built libraries these functions raise.
"""
from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_float, c_int, c_long, c_ulonglong, c_void_p
from typing import Optional, Sequence, Tuple

import torch

from .csrc import build as _build

F32, BF16 = 0, 1
_DT = {torch.float32: F32, torch.bfloat16: BF16}


class KernelError(RuntimeError):
    """A kernel entry point refused its arguments or failed to launch."""


def _code(t: torch.Tensor) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise KernelError(f"element type {t.dtype} is not supported (float32 or bfloat16)") from None


def _need(t: torch.Tensor, name: str, dtype=None, shape: Optional[Sequence[Optional[int]]] = None):
    if not isinstance(t, torch.Tensor) or t.device.type != "cuda":
        raise KernelError(f"{name}: a GPU tensor is needed (no CPU path exists), got "
                          f"{getattr(t, 'device', type(t).__name__)}")
    if not t.is_contiguous():
        raise KernelError(f"{name}: must be contiguous, strides {tuple(t.stride())} for shape {tuple(t.shape)}")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name}: dtype {t.dtype}, expected {dtype}")
    if shape is not None:
        if t.dim() != len(shape) or any(s is not None and s != d for s, d in zip(shape, t.shape)):
            raise KernelError(f"{name}: shape {tuple(t.shape)}, expected {tuple('*' if s is None else s for s in shape)}")


def _p(t: Optional[torch.Tensor]):
    return c_void_p(0 if t is None else t.data_ptr())


def _stream():
    return c_void_p(torch.cuda.current_stream().cuda_stream)


_fn_cache = {}


def _fn(module: str, name: str):
    key = (module, name)
    f = _fn_cache.get(key)
    if f is None:
        lib = _build.load(module)
        f = getattr(lib, name)
        f.restype = c_char_p
        _fn_cache[key] = f
    return f


def _check(msg):
    if msg:
        raise KernelError(msg.decode())


# ---------------------------------------------------------------------------
def embed(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor, scale: float):
    """out[r] = float(table[ids[r]]) * scale;  table [V,H], ids int32 [n], out float32 [n,H]."""
    _need(table, "embed table", shape=(None, None))
    V, H = table.shape
    _need(ids, "embed ids", torch.int32, (None,))
    n = ids.shape[0]
    _need(out, "embed out", torch.float32, (n, H))
    _check(_fn("core", "cpmcu_embed")(_p(table), c_int(_code(table)), _p(ids), _p(out), c_int(n), c_int(H), c_int(V),
                                      c_float(scale), _stream()))


def add_rms_norm(x: torch.Tensor, branch: Optional[torch.Tensor], branch_scale: float, weight: torch.Tensor,
                 eps: float, out: torch.Tensor, rows: Optional[torch.Tensor] = None):
    """x += branch_scale * branch (in place; summed over the leading axis if branch is [P,n,H]);
    out = rmsnorm(x) * weight.  With ``rows`` (int32 [R]) only those rows are normed, into out [R,H],
    and x is left as it was."""
    _need(x, "norm x", torch.float32, (None, None))
    n, H = x.shape
    _need(weight, "norm weight", torch.float32, (H,))
    nparts, stride, bcode = 1, 0, F32
    if branch is not None:
        if branch.dim() == 3:
            _need(branch, "norm branch", shape=(None, n, H))
            nparts, stride = branch.shape[0], n * H
        else:
            _need(branch, "norm branch", shape=(n, H))
        bcode = _code(branch)
    if rows is not None:
        _need(rows, "norm rows", torch.int32, (None,))
        n_out = rows.shape[0]
    else:
        n_out = n
    _need(out, "norm out", shape=(n_out, H))
    _check(_fn("core", "cpmcu_add_rms_norm")(_p(x), _p(branch), c_int(bcode), c_int(nparts), c_long(stride),
                                             c_float(branch_scale), _p(weight), c_float(eps), _p(out),
                                             c_int(_code(out)), _p(rows), c_int(n_out), c_int(H), _stream()))


NORM_SLICE = 64        # columns a slice of add_norm_columns (common.h)

# The kernels of decode steps that own a strip of output columns over all of K (qkv_rope, proj_add_norm) and
# the norm cut by columns (add_norm_columns) save kernels of the chain, but every workgroup reads all of x.
# Up to 16 rows they win at every width measured (MI355X, 4,096 columns: norm 4.7 against 6.6 us at 8 rows).
# qkv_rope (workgroups spread evenly over the CUs) wins up to 32 rows (4,096 columns, q/k/v + rotary: 11.7
# against 18.2 us at 16 rows, 15.6 against 19.7 at 24, 16.5 against 21.3 at 32; it loses beyond: 24.6 against
# 21.3 at 48, 27.2 against 23.2 at 64), and proj_add_norm wins beyond 16 rows only while a workgroup's copy of
# x stays small (1,024 columns, 64 rows: 8.6 against 8.9 + 4.2 us).
STRIP_ROWS = 16
STRIP_MAX_ROWS = 64
STRIP_X_BYTES = 160 * 1024
QKV_ROPE_MAX_ROWS = 32


def strip_kernels_ok(n: int, K: int) -> bool:
    """Whether proj_add_norm (and the norm cut by columns) take a step of n rows of K columns."""
    return n <= STRIP_ROWS or (n <= STRIP_MAX_ROWS and n * K * 2 <= STRIP_X_BYTES)



class RowScale:
    """What a product needs to finish a norm cut by columns: the rows' sums of squares by slices of columns,
    float32 [n, slices] (a slice for every NORM_SLICE columns after add_norm_columns, for every 16 after
    proj_add_norm), and eps.  The product multiplies its rows by rsqrt(sum of the row's slices / H + eps), H
    being its own input width."""
    __slots__ = ("sums", "eps")

    def __init__(self, sums: torch.Tensor, eps: float):
        self.sums, self.eps = sums, float(eps)


def norm_slices(H: int) -> int:
    return -(-H // NORM_SLICE)


def add_norm_columns(x: torch.Tensor, branch: Optional[torch.Tensor], branch_scale: float, weight: torch.Tensor,
                     out: torch.Tensor, sums: torch.Tensor):
    """The norm of a step of few rows without its row factor: x += branch_scale * branch (in place; summed over
    the leading axis if branch is [P,n,H]); out = bfloat16(x * weight); sums[r, s] = sum of x[r]^2 over slice s.
    rmsnorm(x) * weight = out * rsqrt(sums.sum(1) / H + eps) row by row, which the product that reads `out`
    applies to its result (gemm_skinny, qkv_rope: row_scale)."""
    _need(x, "norm x", torch.float32, (None, None))
    n, H = x.shape
    if H % 4:
        raise KernelError(f"add_norm_columns: a width of {H} is no multiple of 4")
    _need(weight, "norm weight", torch.float32, (H,))
    nparts, stride, bcode = 1, 0, F32
    if branch is not None:
        if branch.dim() == 3:
            _need(branch, "norm branch", shape=(None, n, H))
            nparts, stride = branch.shape[0], n * H
        else:
            _need(branch, "norm branch", shape=(n, H))
        bcode = _code(branch)
    _need(out, "norm out", torch.bfloat16, (n, H))
    _need(sums, "norm row sums", torch.float32, (n, norm_slices(H)))
    _check(_fn("core", "cpmcu_add_norm_columns")(_p(x), _p(branch), c_int(bcode), c_int(nparts), c_long(stride),
                                                 c_float(branch_scale), _p(weight), _p(out), _p(sums), c_int(n),
                                                 c_int(H), _stream()))


def silu_mul(gate_up: torch.Tensor, out: torch.Tensor):
    """out[r,c] = silu(gate_up[r,c]) * gate_up[r,c+I];  gate_up [n,2I], out [n,I]."""
    _need(gate_up, "silu_mul input", shape=(None, None))
    n, two_i = gate_up.shape
    if two_i % 2:
        raise KernelError(f"silu_mul: input width {two_i} is odd")
    _need(out, "silu_mul out", gate_up.dtype, (n, two_i // 2))
    _check(_fn("core", "cpmcu_silu_mul")(_p(gate_up), _p(out), c_int(_code(out)), c_int(n), c_int(two_i // 2), _stream()))


def rope_store(qkv: torch.Tensor, q_out: torch.Tensor, nh: int, nkv: int, hd: int, positions: torch.Tensor,
               tok_slot: torch.Tensor, inv_freq: Optional[torch.Tensor], mscale: float,
               kpool: Optional[torch.Tensor], vpool: Optional[torch.Tensor], page_table: Optional[torch.Tensor],
               page_size: int, write_kv: bool = True):
    """Rotate q (and k), write q to q_out [n, nh*hd] and k, v into the paged cache.
    qkv [n, W] or float32 partial sums [P, n, W] with W >= (nh + 2 nkv) hd (nh*hd if not write_kv)."""
    if qkv.dim() == 3:
        _need(qkv, "rope qkv", torch.float32, (None, None, None))
        nparts, n, width = qkv.shape
        stride = n * width
    else:
        _need(qkv, "rope qkv", shape=(None, None))
        n, width = qkv.shape
        nparts, stride = 1, 0
    _need(q_out, "rope q_out", shape=(n, nh * hd))
    _need(positions, "rope positions", torch.int32, (n,))
    _need(tok_slot, "rope token slots", torch.int32, (n,))
    if inv_freq is not None:
        _need(inv_freq, "rope inv_freq", torch.float32, (hd // 2,))
    tw = 0
    if write_kv:
        _need(page_table, "rope page table", torch.int32, (None, None))
        tw = page_table.shape[1]
        _need(kpool, "rope key pool", q_out.dtype, (None, page_size, nkv * hd))
        _need(vpool, "rope value pool", q_out.dtype, tuple(kpool.shape))
    _check(_fn("core", "cpmcu_rope_store")(_p(qkv), c_long(width), c_int(_code(qkv)), c_int(nparts), c_long(stride),
                                           _p(q_out), c_int(_code(q_out)), c_int(n), c_int(nh), c_int(nkv), c_int(hd),
                                           _p(positions), _p(tok_slot), _p(inv_freq), c_float(mscale), _p(kpool),
                                           _p(vpool), _p(page_table), c_int(tw), c_int(page_size),
                                           c_int(1 if write_kv else 0), _stream()))


def gemm_nt_plain(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, alpha: float = 1.0):
    """out[m,N] = alpha * x[m,K] . w[N,K]^T with scalar float FMAs (any size, both element types)."""
    _need(x, "gemm x", shape=(None, None))
    M, K = x.shape
    _need(w, "gemm weight", x.dtype, (None, K))
    N = w.shape[0]
    _need(out, "gemm out", shape=(M, N))
    _check(_fn("gemm", "cpmcu_gemm_nt_plain")(_p(x), c_long(K), _p(w), c_long(K), _p(out), c_long(N), c_int(_code(x)),
                                              c_int(_code(out)), c_int(M), c_int(N), c_int(K), c_float(alpha),
                                              _stream()))


def attention_plain(q: torch.Tensor, out: torch.Tensor, nh: int, nkv: int, hd: int, scale: float,
                    kpool: torch.Tensor, vpool: torch.Tensor, page_table: torch.Tensor, page_size: int,
                    positions: torch.Tensor, tok_slot: torch.Tensor,
                    sel_blocks: Optional[torch.Tensor] = None, sel_count: Optional[torch.Tensor] = None,
                    block_size: int = 0, head_slopes: Optional[torch.Tensor] = None):
    """Causal GQA attention of n query tokens over their sequences' cached keys (plain kernel).  head_slopes
    (float32 [nh]): the score of key j for the query at position p is lowered by head_slopes[h] * (p - j)."""
    _need(q, "attention q", shape=(None, nh * hd))
    n = q.shape[0]
    _need(out, "attention out", q.dtype, (n, nh * hd))
    _need(kpool, "attention key pool", q.dtype, (None, page_size, nkv * hd))
    _need(vpool, "attention value pool", q.dtype, tuple(kpool.shape))
    _need(page_table, "attention page table", torch.int32, (None, None))
    _need(positions, "attention positions", torch.int32, (n,))
    _need(tok_slot, "attention token slots", torch.int32, (n,))
    max_sel = 0
    if sel_count is not None:
        _need(sel_count, "attention block counts", torch.int32, (n, nkv))
        _need(sel_blocks, "attention block list", torch.int32, (n, nkv, None))
        max_sel = sel_blocks.shape[2]
    if head_slopes is not None:
        _need(head_slopes, "attention head slopes", torch.float32, (nh,))
    _check(_fn("attention", "cpmcu_attention_plain")(
        _p(q), _p(out), c_int(_code(q)), c_int(n), c_int(nh), c_int(nkv), c_int(hd), c_float(scale), _p(kpool),
        _p(vpool), _p(page_table), c_int(page_table.shape[1]), c_int(page_size), _p(positions), _p(tok_slot),
        _p(sel_blocks), _p(sel_count), c_int(max_sel), c_int(block_size), _p(head_slopes), _stream()))


MFMA_HEAD_DIMS = (16, 32, 48, 64, 80, 96, 112, 128)


def attention_mfma_ok(q: torch.Tensor, hd: int, page_size: int, block_size: int = 0) -> bool:
    return (q.dtype == torch.bfloat16 and hd in MFMA_HEAD_DIMS and page_size % 32 == 0
            and (block_size == 0 or block_size % 32 == 0))


def attention_mfma(q: torch.Tensor, out: torch.Tensor, nh: int, nkv: int, hd: int, scale: float,
                   kpool: torch.Tensor, vpool: torch.Tensor, page_table: torch.Tensor, page_size: int,
                   positions: torch.Tensor, tok_slot: torch.Tensor, n_splits: int = 1,
                   part_o: Optional[torch.Tensor] = None, part_ml: Optional[torch.Tensor] = None,
                   sel_blocks: Optional[torch.Tensor] = None, sel_count: Optional[torch.Tensor] = None,
                   block_size: int = 0, waves_per_group: int = 0, last_blocks_first: int = 0):
    """bf16 attention on the matrix cores (head_dim 16, 32, ... 128; pages and key blocks multiples of 32).
    With n_splits > 1 every token's keys are shared among n_splits wavefronts and merged afterwards;
    part_o float32 [n, nh, n_splits, hd] and part_ml float32 [n, nh, n_splits, 2] are its scratch.
    last_blocks_first: that many blocks at the end of every block list (the window that neighbouring tokens
    share) are visited before the others; it changes the order of the sums only."""
    _need(q, "attention q", torch.bfloat16, (None, nh * hd))
    n = q.shape[0]
    _need(out, "attention out", torch.bfloat16, (n, nh * hd))
    _need(kpool, "attention key pool", torch.bfloat16, (None, page_size, nkv * hd))
    _need(vpool, "attention value pool", torch.bfloat16, tuple(kpool.shape))
    _need(page_table, "attention page table", torch.int32, (None, None))
    _need(positions, "attention positions", torch.int32, (n,))
    _need(tok_slot, "attention token slots", torch.int32, (n,))
    max_sel = 0
    if sel_count is not None:
        _need(sel_count, "attention block counts", torch.int32, (n, nkv))
        _need(sel_blocks, "attention block list", torch.int32, (n, nkv, None))
        max_sel = sel_blocks.shape[2]
    if n_splits > 1:
        _need(part_o, "attention partial outputs", torch.float32, (n, nh, n_splits, hd))
        _need(part_ml, "attention partial max/sum", torch.float32, (n, nh, n_splits, 2))
    _check(_fn("attention", "cpmcu_attention_mfma")(
        _p(q), _p(out), _p(part_o), _p(part_ml), c_int(n), c_int(nh), c_int(nkv), c_int(hd), c_float(scale),
        _p(kpool), _p(vpool), _p(page_table), c_int(page_table.shape[1]), c_int(page_size), _p(positions),
        _p(tok_slot), _p(sel_blocks), _p(sel_count), c_int(max_sel), c_int(block_size), c_int(n_splits),
        c_int(waves_per_group), c_int(last_blocks_first), _stream()))


def attention_prefill_tokens_per_wave(nh: int, nkv: int, tiles_per_wave: int = 4) -> int:
    lib = _build.load("attention")
    lib.cpmcu_attention_prefill_tokens_per_wave.restype = c_int
    return int(lib.cpmcu_attention_prefill_tokens_per_wave(c_int(nh), c_int(nkv), c_int(tiles_per_wave)))


def attention_prefill_shape(n_tokens: int, nh: int, nkv: int, hd: int):
    """(tiles a wavefront, wavefronts a workgroup) for the prompt kernel.  Measured on the MI355X at head size
    128, 32 heads in 2 groups, one prompt of 512 / 2,048 / 8,192 / 32,768 tokens, in us:
      2 tiles, 1 / 2 / 4 wavefronts:  25 / 20 / 19    95 / 75 / 90    894 / 819 / 835   11.3 / 11.6 / 11.8 ms
      4 tiles, 1 / 2 / 4 wavefronts:  37 / 26 / 24   123 / 86 / 116   888 / 904 / 1058  13.7 / 13.4 / 14.1 ms
    Two tiles of 16 rows a wavefront leave room for two wavefronts a SIMD; wavefronts that share a group of
    tiles take the chunks of keys in turn, which evens out the causal triangle of short prompts."""
    if n_tokens <= 1024:
        return 2, 4
    return 2, (2 if n_tokens < 16384 else 1)


def attention_prefill_mfma(q: torch.Tensor, out: torch.Tensor, tiles: torch.Tensor, nh: int, nkv: int, hd: int,
                           scale: float, kpool: torch.Tensor, vpool: torch.Tensor, page_table: torch.Tensor,
                           page_size: int, positions: torch.Tensor, tok_slot: torch.Tensor, tiles_per_wave: int = 4,
                           waves_per_group: int = 1):
    """Dense causal bf16 attention for prompts: tiles int32 [T, 2] = (first packed token, tokens), each a run of
    consecutive tokens of one sequence, at most attention_prefill_tokens_per_wave(nh, nkv, tiles_per_wave) long."""
    _need(q, "attention q", torch.bfloat16, (None, nh * hd))
    n = q.shape[0]
    _need(out, "attention out", torch.bfloat16, (n, nh * hd))
    _need(tiles, "attention tiles", torch.int32, (None, 2))
    _need(kpool, "attention key pool", torch.bfloat16, (None, page_size, nkv * hd))
    _need(vpool, "attention value pool", torch.bfloat16, tuple(kpool.shape))
    _need(page_table, "attention page table", torch.int32, (None, None))
    _need(positions, "attention positions", torch.int32, (n,))
    _need(tok_slot, "attention token slots", torch.int32, (n,))
    _check(_fn("attention", "cpmcu_attention_prefill_mfma")(
        _p(q), _p(out), c_int(tiles.shape[0]), _p(tiles), c_int(tiles_per_wave), c_int(waves_per_group), c_int(nh),
        c_int(nkv), c_int(hd),
        c_float(scale),
        _p(kpool), _p(vpool), _p(page_table), c_int(page_table.shape[1]), c_int(page_size), _p(positions),
        _p(tok_slot), _stream()))


def prefill_tiles(q_lens: Sequence[int], tokens_per_wave: int, device) -> torch.Tensor:
    """Runs of at most tokens_per_wave consecutive tokens of one sequence, covering the packed batch."""
    tiles = []
    start = 0
    for q in q_lens:
        for a in range(0, q, tokens_per_wave):
            tiles.append((start + a, min(tokens_per_wave, q - a)))
        start += q
    return torch.tensor(tiles, dtype=torch.int32).to(device)


_cu_count = None


def compute_units() -> int:
    """CUs of the current GPU (256 on the MI355X, which is also what the heuristics below were measured on and
    what they assume when no GPU is visible)."""
    global _cu_count
    if _cu_count is None:
        _cu_count = (torch.cuda.get_device_properties(torch.cuda.current_device()).multi_processor_count
                     if torch.cuda.is_available() else 256)
    return _cu_count


def attention_splits(n_tokens: int, nkv: int, group: int, max_keys: int) -> int:
    """Shares of a token's keys for steps of few tokens.  Measured on the MI355X (head size 128, 2 kv heads,
    workgroups of 4 wavefronts, graph replay over keys that come from memory, attention + merge, in us for
    1/2/4/8/16/32 shares):
      8 sequences at 4,096 keys 38/24/17/13/12.5/14, at 16,384 keys 146/80/47/32/30/30, at 32,768 279/150/87/59/53/55;
      16 sequences at 4,096 keys 43/30/21/18/20/23; 24 sequences 44/34/24/27/27/31; 32 sequences 48/32/30/32/34/39;
      64 sequences 55/52/53/57/59/71;
      one sequence at 4,096 keys 22/15/11/8.8/7.9/7.6, at 16,384 keys 140/74/41/25/17/12.5, at 65,536 531/275/140/76/46/28;
      4 sequences at 32,768 keys 278/148/80/49/32/30.
    So: as many shares as give about 256 workgroups in all, one for every CU (a CU takes in ~30 GB/s however
    much it has in flight; the merge kernel costs ~3 us whatever the number of shares up to 32), a share of at
    least 128 keys, at most 32 shares (beyond 32 the merge kernel no longer holds every share's output in
    registers: one sequence at 32,000 keys, whole step, 3.89 ms with 64 shares against 3.60 with 32).  A step
    that has 128 workgroups or more by itself takes two shares from 4,096 keys on (they even out the
    workgroups' ends) and one below (no merge kernel: 64 sequences of the 0.5B shape)."""
    cus = compute_units()
    if n_tokens > cus:
        return 1
    groups = n_tokens * nkv * -(-group // 16)
    want = max(1, cus // max(groups, 1))
    if groups >= cus // 2:
        want = 2 if max_keys >= 4096 else 1
    return max(1, min(want, max_keys // 128, 32))


def compress_keys(kpool: torch.Tensor, ckpool: torch.Tensor, nkv: int, page_table: torch.Tensor, page_size: int,
                  positions: torch.Tensor, tok_slot: torch.Tensor, kernel_size: int, kernel_stride: int):
    """Write the compressed keys (means of kernel_size keys, every kernel_stride) that the step's tokens complete.
    The keys lie in their pages as rope_store writes them; a compressed key is a plain row [kv head][d]."""
    _need(kpool, "compress key pool", shape=(None, page_size, None))
    width = kpool.shape[2]
    if nkv <= 0 or width % nkv:
        raise KernelError(f"compress_keys: rows of {width} elements do not hold {nkv} kv heads")
    if kernel_stride <= 0 or page_size % kernel_stride:
        raise KernelError(f"compress_keys: kernel_stride {kernel_stride} must divide the cache page of {page_size} tokens")
    _need(ckpool, "compressed key pool", kpool.dtype, (kpool.shape[0], page_size // kernel_stride, width))
    _need(page_table, "compress page table", torch.int32, (None, None))
    _need(positions, "compress positions", torch.int32, (None,))
    n = positions.shape[0]
    _need(tok_slot, "compress token slots", torch.int32, (n,))
    _check(_fn("sparse", "cpmcu_compress_keys")(_p(kpool), _p(ckpool), c_int(_code(kpool)), c_int(n), c_int(nkv),
                                                c_int(width // nkv), _p(page_table), c_int(page_table.shape[1]), c_int(page_size),
                                                _p(positions), _p(tok_slot), c_int(kernel_size), c_int(kernel_stride),
                                                _stream()))


def sparse_select_scratch(dtype: torch.dtype, n: int, nh: int, nkv: int, hd: int, max_pos: int, kernel_size: int,
                          kernel_stride: int, block_size: int, force_plain=False) -> int:
    """Floats of scratch that sparse_select wants for a step of n tokens at positions up to max_pos (0: none).
    bf16 steps of few tokens run as three kernels of many small workgroups through it; contexts whose scores
    and ranking arrays exceed a workgroup's LDS keep them there instead (any step, both element types)."""
    lib = _build.load("sparse")
    f = lib.cpmcu_sparse_select_scratch
    f.restype = c_long
    return int(f(c_int(_DT[dtype]), c_int(n), c_int(nh), c_int(nkv), c_int(hd), c_int(kernel_size), c_int(kernel_stride),
                 c_int(block_size), c_int(max_pos), c_int(int(force_plain))))


def sparse_select(q: torch.Tensor, ckpool: torch.Tensor, nh: int, nkv: int, hd: int, scale: float,
                  page_table: torch.Tensor, page_size: int, positions: torch.Tensor, tok_slot: torch.Tensor,
                  kernel_size: int, kernel_stride: int, block_size: int, init_blocks: int, topk: int,
                  window_blocks: int, dense_len: int, max_pos: int, sel_blocks: torch.Tensor, sel_count: torch.Tensor,
                  force_plain=False, scratch: Optional[torch.Tensor] = None):
    """Block list per (token, kv head): sel_count -1 = dense, else the ascending blocks to attend to.
    scratch: float32 of at least sparse_select_scratch(...) elements, if that is not 0.
    force_plain: True = the plain kernel; 2 = steps of few tokens with the normalising kernel kept apart, as for
    contexts too long for the fused form (for tests)."""
    _need(q, "select q", shape=(None, nh * hd))
    n = q.shape[0]
    _need(ckpool, "select compressed keys", q.dtype, (None, page_size // max(kernel_stride, 1), nkv * hd))
    _need(page_table, "select page table", torch.int32, (None, None))
    _need(positions, "select positions", torch.int32, (n,))
    _need(tok_slot, "select token slots", torch.int32, (n,))
    _need(sel_count, "select counts", torch.int32, (n, nkv))
    _need(sel_blocks, "select block list", torch.int32, (n, nkv, None))
    if scratch is not None:
        _need(scratch, "select scratch", torch.float32, (None,))
    _check(_fn("sparse", "cpmcu_sparse_select")(
        _p(q), _p(ckpool), c_int(_code(q)), c_int(n), c_int(nh), c_int(nkv), c_int(hd), c_float(scale),
        _p(page_table), c_int(page_table.shape[1]), c_int(page_size), _p(positions), _p(tok_slot),
        c_int(kernel_size), c_int(kernel_stride), c_int(block_size), c_int(init_blocks), c_int(topk),
        c_int(window_blocks), c_int(dense_len), c_int(max_pos), _p(sel_blocks), _p(sel_count),
        c_int(sel_blocks.shape[2]), c_int(int(force_plain)), _p(scratch),
        c_long(scratch.numel() if scratch is not None else 0), _stream()))


def argmax(logits: torch.Tensor, out: torch.Tensor):
    """out[r] = index of the largest logits[r] (ties: the lowest index)."""
    _need(logits, "argmax logits", torch.float32, (None, None))
    R, V = logits.shape
    _need(out, "argmax out", torch.int32, (R,))
    _check(_fn("core", "cpmcu_argmax")(_p(logits), c_long(V), c_int(R), c_int(V), _p(out), _stream()))


def sample(logits: torch.Tensor, temperature: float, seed: int, request_ids: torch.Tensor, steps: torch.Tensor,
           out: torch.Tensor, u_out: Optional[torch.Tensor] = None):
    """out[r] ~ softmax(logits[r] / temperature), the uniform number keyed by (seed, request_ids[r], steps[r])."""
    _need(logits, "sample logits", torch.float32, (None, None))
    R, V = logits.shape
    _need(request_ids, "sample request ids", torch.int32, (R,))
    _need(steps, "sample steps", torch.int32, (R,))
    _need(out, "sample out", torch.int32, (R,))
    if u_out is not None:
        _need(u_out, "sample u_out", torch.float32, (R,))
    _check(_fn("core", "cpmcu_sample")(_p(logits), c_long(V), c_int(R), c_int(V), c_float(temperature),
                                       c_ulonglong(seed & 0xFFFFFFFFFFFFFFFF), _p(request_ids), _p(steps), _p(out),
                                       _p(u_out), _stream()))


def read_bandwidth(src: torch.Tensor, out: torch.Tensor):
    """Read all of ``src`` once with a kernel that does nothing else (out: int32 scratch of a few thousand
    words): what measurement compares the decode products' streaming with."""
    _need(src, "read source")
    _need(out, "read scratch", torch.int32, (None,))
    _check(_fn("core", "cpmcu_read_bandwidth")(_p(src), c_long(src.numel() * src.element_size()), _p(out),
                                               c_int(out.shape[0]), _stream()))


class TiledWeight:
    """A weight [N, K] re-laid for the skinny product: [strip of 16 rows][K-block of 128][MFMA i][lane][8],
    lane = 16*g + r holding row 16*strip + r, columns 128*block + 32*i + 8*g .. +8; zero padded."""

    def __init__(self, w: torch.Tensor):
        _need(w, "weight to tile", torch.bfloat16, (None, None))
        N, K = w.shape
        Np, Kp = -(-N // 16) * 16, -(-K // 128) * 128
        if (Np, Kp) != (N, K):
            wp = torch.zeros((Np, Kp), dtype=w.dtype, device=w.device)
            wp[:N, :K] = w
        else:
            wp = w
        self.data = wp.view(Np // 16, 16, Kp // 128, 4, 4, 8).permute(0, 2, 3, 4, 1, 5).contiguous()
        self.N, self.K = N, K

    def first_rows(self, n: int) -> "TiledWeight":
        """The same memory seen as the weight's first n rows (whole strips of 16, or all of it)."""
        if n == self.N:
            return self
        if n <= 0 or n > self.N or n % 16:
            raise KernelError(f"a tiled weight of {self.N} rows gives its first rows in whole strips of 16, not {n}")
        view = object.__new__(TiledWeight)
        view.data, view.N, view.K = self.data[:n // 16], n, self.K
        return view




class QKVRopeWeight:
    """The stacked [q heads; k heads; v heads] x hidden weight re-laid for qkv_rope:
    * the rows of every q and k head as rotation pairs side by side (c, c + hd/2, c + 1, c + 1 + hd/2, ...), v
      heads in their order;
    * cut into runs of R rows, one a workgroup (R from the kernel library: 16, or a few more where that spreads
      the workgroups evenly over the CUs);
    * per run and 128-column block: 16 rows as [MFMA i][lane = 16 g + row][8] (columns 32 i + 8 g ..), then the
      other R - 16 rows as [i][g][row][8]; rows and columns zero padded."""

    def __init__(self, w: torch.Tensor, nh: int, nkv: int, hd: int, rows_per_workgroup: Optional[int] = None):
        total = (nh + 2 * nkv) * hd
        _need(w, "qkv weight", torch.bfloat16, (total, None))
        if hd % 16:
            raise KernelError(f"qkv_rope: head_dim {hd} is no multiple of 16")
        if rows_per_workgroup is None:
            lib = _build.load("qkv")
            lib.cpmcu_qkv_rope_rows_per_workgroup.restype = c_int
            rows_per_workgroup = int(lib.cpmcu_qkv_rope_rows_per_workgroup(c_int(total)))
        R = int(rows_per_workgroup)
        if R < 16 or R > 32 or R % 2:
            raise KernelError(f"qkv_rope: {R} rows a workgroup (an even number from 16 to 32)")
        K = w.shape[1]
        c = torch.arange(hd // 2)
        order = torch.stack([c, c + hd // 2], dim=1).reshape(-1)
        rows = torch.arange(total).view(nh + 2 * nkv, hd).clone()
        rows[:nh + nkv] = rows[:nh + nkv, :1] + order
        n_wg, nkb = -(-total // R), -(-K // 128)
        padded = torch.zeros((n_wg * R, nkb * 128), dtype=w.dtype, device=w.device)
        padded[:total, :K] = w[rows.reshape(-1).to(w.device)]
        blk = padded.view(n_wg, R, nkb, 4, 4, 8)                 # run, row, block, i, g, element
        first = blk[:, :16].permute(0, 2, 3, 4, 1, 5).reshape(n_wg, nkb, 2048)
        rest = blk[:, 16:].permute(0, 2, 3, 4, 1, 5).reshape(n_wg, nkb, 128 * (R - 16))
        self.data = torch.cat([first, rest], dim=2).contiguous()
        self.N, self.K, self.rows_per_workgroup = total, K, R


def qkv_rope_weight(w: torch.Tensor, nh: int, nkv: int, hd: int, rows_per_workgroup: Optional[int] = None
                    ) -> QKVRopeWeight:
    """rows_per_workgroup: None lets the kernel library choose (what the engine does)."""
    return QKVRopeWeight(w, nh, nkv, hd, rows_per_workgroup)


def qkv_rope(x: torch.Tensor, w: QKVRopeWeight, q_out: torch.Tensor, nh: int, nkv: int, hd: int,
             positions: torch.Tensor, tok_slot: torch.Tensor, inv_freq: Optional[torch.Tensor], mscale: float,
             kpool: torch.Tensor, vpool: torch.Tensor, page_table: torch.Tensor, page_size: int,
             row_scale: Optional[RowScale] = None, compress: Optional[Tuple[torch.Tensor, int, int]] = None):
    """q, k, v = x . w^T for a step of at most 64 tokens, rotated (inv_freq None: not) and written: q to q_out
    [n, nh*hd], k and v into the paged cache.  w from qkv_rope_weight.  With row_scale, x is the x * w of
    add_norm_columns and the rows of the product are multiplied by the norm's factor before the rotation.
    With compress = (compressed key pool, kernel_size, kernel_stride) the compressed keys that the step's tokens
    complete are written too, as compress_keys would after this call."""
    _need(x, "qkv x", torch.bfloat16, (None, w.K))
    n = x.shape[0]
    if row_scale is not None:
        _need(row_scale.sums, "qkv row sums", torch.float32, (n, None))
    ckpool, ks, st = compress if compress is not None else (None, 0, 0)
    if ckpool is not None:
        # (compressed key pool, kernel_size, kernel_stride): the step's tokens also complete their compressed keys
        if st <= 0 or page_size % st:
            raise KernelError(f"qkv_rope: kernel_stride {st} must divide the cache page of {page_size} tokens")
        _need(ckpool, "qkv compressed key pool", torch.bfloat16, (kpool.shape[0], page_size // st, nkv * hd))
    if not isinstance(w, QKVRopeWeight) or w.N != (nh + 2 * nkv) * hd:
        raise KernelError(f"qkv_rope: the weight must come from qkv_rope_weight for {(nh + 2 * nkv) * hd} rows")
    _need(q_out, "qkv q_out", torch.bfloat16, (n, nh * hd))
    _need(positions, "qkv positions", torch.int32, (n,))
    _need(tok_slot, "qkv token slots", torch.int32, (n,))
    if inv_freq is not None:
        _need(inv_freq, "qkv inv_freq", torch.float32, (hd // 2,))
    _need(kpool, "qkv key pool", torch.bfloat16, (None, page_size, nkv * hd))
    _need(vpool, "qkv value pool", torch.bfloat16, tuple(kpool.shape))
    _need(page_table, "qkv page table", torch.int32, (None, None))
    _check(_fn("qkv", "cpmcu_qkv_rope")(_p(x), c_long(x.stride(0)), _p(w.data), c_int(w.rows_per_workgroup), c_int(n),
                                        c_int(w.K), _p(q_out),
                                        c_int(nh), c_int(nkv), c_int(hd), _p(positions), _p(tok_slot), _p(inv_freq),
                                        c_float(mscale), _p(kpool), _p(vpool), _p(page_table),
                                        c_int(page_table.shape[1]), c_int(page_size),
                                        _p(row_scale.sums if row_scale is not None else None),
                                        c_int(row_scale.sums.shape[1] if row_scale is not None else 0),
                                        c_float(row_scale.eps if row_scale is not None else 0.0),
                                        _p(ckpool), c_int(ks), c_int(st), _stream()))


def proj_add_norm(a: torch.Tensor, w: "TiledWeight", alpha: float, x: torch.Tensor, weight: torch.Tensor,
                  out: torch.Tensor, sums: torch.Tensor):
    """A branch's last product fused with the residual add and the column part of the norm that follows, for a
    step of at most 64 tokens: x += alpha * (a . w^T) in place (x float32 [n, N], a bfloat16 [n, K], w tiled
    [N, K]); out = bfloat16(x * weight); sums[r, s] = sum of x[r]^2 over the 16 columns of strip s (float32
    [n, ceil(N / 16)]).  As after add_norm_columns, the product that reads `out` applies the row factor."""
    _need(a, "proj a", torch.bfloat16, (None, None))
    n, K = a.shape
    if not isinstance(w, TiledWeight) or w.K != K:
        raise KernelError(f"proj_add_norm: the weight must be tiled for K = {K}")
    N = w.N
    if N % 4 or K % 8:
        raise KernelError(f"proj_add_norm: N={N} must be a multiple of 4 and K={K} of 8")
    _need(x, "proj residual", torch.float32, (n, N))
    _need(weight, "proj norm weight", torch.float32, (N,))
    _need(out, "proj out", torch.bfloat16, (n, N))
    _need(sums, "proj row sums", torch.float32, (n, -(-N // 16)))
    _check(_fn("qkv", "cpmcu_proj_add_norm")(_p(a), c_long(K), _p(w.data), c_int(n), c_int(N), c_int(K),
                                             c_float(alpha), _p(x), _p(weight), _p(out), _p(sums), _stream()))


def gated_strip(x: torch.Tensor, w: "TiledWeight", out: torch.Tensor, row_scale: Optional[RowScale] = None):
    """out = silu(x . Wg^T) * (x . Wu^T) for a step of at most 16 tokens, w tiled with the gate rows first (a
    multiple of 16 of them); out bfloat16 [n, N/2].  With row_scale as in gemm_skinny."""
    _need(x, "gated x", torch.bfloat16, (None, None))
    n, K = x.shape
    if not isinstance(w, TiledWeight) or w.K != K or w.N % 32:
        raise KernelError(f"gated_strip: the weight must be tiled for K = {K} with a multiple of 16 gate rows")
    _need(out, "gated out", torch.bfloat16, (n, w.N // 2))
    if row_scale is not None:
        _need(row_scale.sums, "gated row sums", torch.float32, (n, None))
    _check(_fn("qkv", "cpmcu_gated_strip")(_p(x), c_long(K), _p(w.data), c_int(n), c_int(w.N // 2), c_int(K), _p(out),
                                           _p(row_scale.sums if row_scale is not None else None),
                                           c_int(row_scale.sums.shape[1] if row_scale is not None else 0),
                                           c_float(row_scale.eps if row_scale is not None else 0.0), _stream()))


def gemm_skinny(x: torch.Tensor, w, out: torch.Tensor, alpha: float = 1.0, mode: str = "plain",
                row_scale: Optional[RowScale] = None):
    """bf16 product for at most 64 rows of x on the matrix cores, streaming w once; w is [N, K] as in the
    checkpoint or a TiledWeight.
    mode 'plain': out [m,N] float32 or bfloat16; 'partial': out float32 [S,m,N], S slices of K to be summed by
    the consumer; 'gated': w holds gate rows then up rows, out bfloat16 [m,N/2] = silu(gate) * up.
    With row_scale, x is the x * w of add_norm_columns: the rows of the product are multiplied by the norm's
    factor (before the gate's nonlinearity)."""
    _need(x, "gemm x", torch.bfloat16, (None, None))
    M, K = x.shape
    if row_scale is not None:
        _need(row_scale.sums, "gemm row sums", torch.float32, (M, None))
    tiled = isinstance(w, TiledWeight)
    if tiled:
        if w.K != K:
            raise KernelError(f"gemm weight: tiled for K={w.K}, x has {K} columns")
        N, wt = w.N, w.data
    else:
        _need(w, "gemm weight", torch.bfloat16, (None, K))
        N, wt = w.shape[0], w
    ksplit, omode = 1, 0
    if mode == "plain":
        _need(out, "gemm out", shape=(M, N))
        ldy = N
    elif mode == "partial":
        _need(out, "gemm partial sums", torch.float32, (None, M, N))
        ksplit, omode, ldy = out.shape[0], 1, N
    elif mode == "gated":
        _need(out, "gemm gated out", torch.bfloat16, (M, N // 2))
        omode, ldy = 2, N // 2
    else:
        raise KernelError(f"gemm_skinny: unknown mode '{mode}'")
    _check(_fn("gemm", "cpmcu_gemm_skinny")(_p(x), c_long(K), _p(wt), c_long(K), _p(out), c_long(ldy),
                                            c_int(_code(out)), c_int(omode), c_int(M), c_int(N), c_int(K),
                                            c_int(ksplit), c_float(alpha), c_int(1 if tiled else 0),
                                            _p(row_scale.sums if row_scale is not None else None),
                                            c_int(row_scale.sums.shape[1] if row_scale is not None else 0),
                                            c_float(row_scale.eps if row_scale is not None else 0.0), _stream()))


SKINNY_MAX_ROWS = 64


def skinny_ok(x: torch.Tensor, w=None) -> bool:
    return x.dtype == torch.bfloat16 and x.shape[0] <= SKINNY_MAX_ROWS and x.shape[1] % 8 == 0


def skinny_split(M: int, N: int, K: int) -> int:
    """Slices of K for a skinny product whose consumer sums partial results.  A workgroup streams 64 rows
    of the weight.  Up to 16 rows of x about 1024 small workgroups balance well over the 256 CUs; with more rows
    a workgroup holds 33 or 67 KB of LDS and a CU two or four of them, and a CU with one workgroup more than
    its neighbours ends late: at most one workgroup a CU then (MI355X, 64 rows, us for 2/4/8 slices: q/k/v
    4,608 x 4,096 16.6/19.1/17.7, o 15.7/11.4/13.8, down 51.0/30.5/31.3; 32 rows: 12.5/13.6/13.2, 11.9/9.5/10.6,
    37.8/24.6/25.7).  Every slice should still stream 512 columns, and more rows make the partial sums themselves
    cost traffic."""
    wgs = -(-N // 64)
    cap = 16 if M <= 16 else (8 if M <= 32 else 4)
    most = 5 * compute_units() if M <= 16 else compute_units()
    want = 1
    while want * 2 <= cap and wgs * want * 2 <= most and K // (want * 2) >= 512:
        want *= 2
    if want <= 1:
        return 1
    ks = -(-(-(-K // want)) // 128) * 128
    return -(-K // ks)


# ---------------------------------------------------------------------------
# dispatchers: choose the kernel for a shape and element type
# ---------------------------------------------------------------------------
def library_gemm_ok(x: torch.Tensor, out_dtype: torch.dtype) -> bool:
    """Many rows in bf16 with bf16 output: the library's matrix product (the reference calls its vendor's
    library for every linear layer, src/model/linear.cuh:9-37)."""
    return x.dtype == torch.bfloat16 and out_dtype == torch.bfloat16 and x.shape[0] > SKINNY_MAX_ROWS


def linear(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, alpha: float = 1.0, w_tiled=None):
    """out = alpha * x . w^T with the kernel that suits the element type and the number of rows."""
    M = x.shape[0]
    if w is None and (w_tiled is None or M > SKINNY_MAX_ROWS and out.dtype == torch.bfloat16 and alpha == 1.0):
        raise KernelError(f"linear: {M} rows need the weight in the checkpoint's layout, which this engine let go "
                          f"(it was built for forward passes of at most {SKINNY_MAX_ROWS} tokens)")
    if x.dtype == torch.bfloat16 and x.shape[1] % 8 == 0:
        if M <= SKINNY_MAX_ROWS:
            gemm_skinny(x, w_tiled if w_tiled is not None else w, out, alpha)
            return
        if out.dtype == torch.bfloat16 and alpha == 1.0:
            torch.mm(x, w.t(), out=out)
            return
        # float output for many rows (logits of many positions): the skinny kernel, 64 rows at a time
        for r in range(0, M, SKINNY_MAX_ROWS):
            gemm_skinny(x[r:r + SKINNY_MAX_ROWS], w_tiled if w_tiled is not None else w, out[r:r + SKINNY_MAX_ROWS], alpha)
        return
    gemm_nt_plain(x, w, out, alpha)


def attention(q, out, nh, nkv, hd, scale, kpool, vpool, page_table, page_size, ctx,
              sel_blocks=None, sel_count=None, block_size=0, window_blocks=0, head_slopes=None):
    """Attention of the step's queries over the cache, with the kernel that suits the step; writes ``out``.
    head_slopes (float32 [nh], a position encoding's bias of the scores by distance) is taken by the plain
    kernel only, in both element types."""
    if head_slopes is not None:
        attention_plain(q, out, nh, nkv, hd, scale, kpool, vpool, page_table, page_size, ctx.positions, ctx.tok_slot,
                        sel_blocks, sel_count, block_size, head_slopes)
        return
    if sel_count is None and not ctx.single_token and attention_mfma_ok(q, hd, page_size):
        r, nw = attention_prefill_shape(q.shape[0], nh, nkv, hd)
        tpw = attention_prefill_tokens_per_wave(nh, nkv, r)
        key = ("prefill_tiles", tpw)
        tiles = ctx.extras.get(key)
        if tiles is None:
            tiles = ctx.extras[key] = prefill_tiles(ctx.q_lens, tpw, q.device)
        attention_prefill_mfma(q, out, tiles, nh, nkv, hd, scale, kpool, vpool, page_table, page_size,
                               ctx.positions, ctx.tok_slot, r, nw)
        return
    if attention_mfma_ok(q, hd, page_size, block_size if sel_count is not None else 0):
        n = q.shape[0]
        keys = ctx.max_pos + 1
        if sel_count is not None:
            keys = min(keys, sel_blocks.shape[2] * block_size)
        splits = attention_splits(n, nkv, nh // nkv, keys)
        part_o = part_ml = None
        if splits > 1:
            part_o = ctx.ws.get("attn.part_o", (n, nh, splits, hd), torch.float32)
            part_ml = ctx.ws.get("attn.part_ml", (n, nh, splits, 2), torch.float32)
        attention_mfma(q, out, nh, nkv, hd, scale, kpool, vpool, page_table, page_size, ctx.positions, ctx.tok_slot,
                       splits, part_o, part_ml, sel_blocks, sel_count, block_size, last_blocks_first=window_blocks)
        return
    attention_plain(q, out, nh, nkv, hd, scale, kpool, vpool, page_table, page_size, ctx.positions, ctx.tok_slot,
                    sel_blocks, sel_count, block_size)
