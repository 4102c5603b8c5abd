"""Plain, slow MiniCPM4 (MiniCPMForCausalLM) forward pass: the oracle of the tests.

Whole sequences, no cache, one function per part, written from the formulas of
OpenBMB/CPM.cu (cited per function as path:line of that repository) and, where
that engine holds one sequence or leaves a choice open, from the engine's own
contract (block-sparse attention as a pure function of the prefix).  It shares
no code with the product package: it only needs torch on the CPU, a raw
config.json dict and a dict of tensors by their checkpoint names.

All arithmetic runs in ``dtype`` (float64 by default) so that the oracle's own
rounding is far below the engine's.
"""
import math

import torch

NEG_INF = float("-inf")


# ----------------------------------------------------------------------------
# configuration scalars
# ----------------------------------------------------------------------------
def head_dim_of(cfg):
    """head_dim defaults to hidden/heads (cpmcu/llm.py:62-66)."""
    return int(cfg.get("head_dim") or cfg["hidden_size"] // cfg["num_attention_heads"])


def mup_scalars(cfg):
    """(scale_emb, residual scale, head scale); cpmcu/llm.py:67-69.

    scale_emb (1 if absent); scale_depth/sqrt(L) (1 if absent);
    dim_model_base/hidden (1 if absent)."""
    s_e = float(cfg.get("scale_emb", 1.0))
    s_r = float(cfg["scale_depth"]) / math.sqrt(cfg["num_hidden_layers"]) if "scale_depth" in cfg else 1.0
    s_l = float(cfg["dim_model_base"]) / cfg["hidden_size"] if "dim_model_base" in cfg else 1.0
    return s_e, s_r, s_l


# ----------------------------------------------------------------------------
# parts
# ----------------------------------------------------------------------------
def embed(table, ids, scale_emb):
    """x[t] = E[id_t] * scale_emb (src/model/embedding.cuh:7-20, 49-52)."""
    return table[ids.long()] * scale_emb


def rms_norm(x, w, eps):
    """y = x * rsqrt(mean(x^2) + eps) * w; eps inside the root, weight after,
    no bias, no 1+w (src/model/norm.cuh:7-51, eps at :39, product at :46-49)."""
    ms = (x * x).sum(-1, keepdim=True) / x.shape[-1]
    return x * torch.rsqrt(ms + eps) * w


def rope_inv_freq(cfg, max_seq_len=None, dtype=torch.float64):
    """(inv_freq[hd/2], m): rotation frequencies and the cos/sin magnitude.

    The reference loads inv_freq once, computed for the engine's whole token
    budget (cpmcu/llm.py:181-191), so short or long LongRoPE factors are a
    static choice: long iff max_seq_len > original_max_position_embeddings.
    inv_freq[c] = 1 / (factor[c] * theta^(2c/hd)).  cos and sin are multiplied
    by m = sqrt(1 + ln(max_position/original_max)/ln(original_max)) when the
    model's position range was stretched, else 1 (the reference drops m,
    cpmcu/llm.py:190-192; ``rope_attention_scaling`` false reproduces that).
    """
    hd = head_dim_of(cfg)
    theta = float(cfg.get("rope_theta", 10000.0))
    c = torch.arange(0, hd, 2, dtype=dtype)
    base = theta ** (c / hd)
    rs = cfg.get("rope_scaling")
    if not rs:
        return 1.0 / base, 1.0
    kind = rs.get("rope_type", rs.get("type"))
    if kind in (None, "default"):
        return 1.0 / base, 1.0
    assert kind == "longrope", kind
    max_pos = int(cfg["max_position_embeddings"])
    orig = int(rs.get("original_max_position_embeddings",
                      cfg.get("original_max_position_embeddings", max_pos)))
    if max_seq_len is None:
        max_seq_len = max_pos
    factors = rs["long_factor"] if max_seq_len > orig else rs["short_factor"]
    f = torch.tensor(factors, dtype=dtype)
    assert f.numel() == hd // 2
    ratio = max_pos / orig
    m = math.sqrt(1.0 + math.log(ratio) / math.log(orig)) if ratio > 1.0 else 1.0
    if not cfg.get("rope_attention_scaling", True):
        m = 1.0
    return 1.0 / (f * base), m


def apply_rope(x, positions, inv_freq, m):
    """Rotate-half RoPE on x [T, heads, hd] at absolute positions [T].

    theta = p*inv_freq[c]; (x_c, x_{c+hd/2}) <- (x_c cos - x_{c+hd/2} sin,
    x_c sin + x_{c+hd/2} cos) (src/model/rotary.cuh:7-34)."""
    half = x.shape[-1] // 2
    ang = positions.to(inv_freq.dtype)[:, None] * inv_freq[None, :]
    cos = (torch.cos(ang) * m)[:, None, :]
    sin = (torch.sin(ang) * m)[:, None, :]
    a, b = x[..., :half], x[..., half:]
    return torch.cat([a * cos - b * sin, a * sin + b * cos], dim=-1)


def dense_attention(q, k, v, allowed=None):
    """Causal GQA attention of one whole sequence.

    q [T, nh, hd], k, v [T, nkv, hd]; score (q.k) * hd^-1/2, query i sees keys
    j <= i, softmax over keys, head h reads kv head h // (nh/nkv)
    (src/model/attn.cuh:200-227; src/flash_attn/flash_api.hpp:294-394; GQA
    index src/flash_attn/src/flash_fwd_kernel.h:1266-1267).  ``allowed``
    [T, nkv, T] bool further restricts the keys (block-sparse attention)."""
    T, nh, hd = q.shape
    nkv = k.shape[1]
    G = nh // nkv
    out = torch.empty_like(q)
    causal = torch.ones(T, T, dtype=torch.bool).tril()
    for h in range(nh):
        g = h // G
        s = (q[:, h] @ k[:, g].T) * hd ** -0.5
        mask = causal if allowed is None else (causal & allowed[:, g])
        s = s.masked_fill(~mask, NEG_INF)
        out[:, h] = torch.softmax(s, dim=-1) @ v[:, g]
    return out


def compressed_keys(k, ks, st):
    """ck[j] = mean(K[st*j : st*j+ks]) over rotated keys, per kv head
    (src/model/minicpm4/minicpm4_kvcache.cuh:6-62: kernel 32, stride 16 there,
    from sparse_config here).  k [T, nkv, hd] -> [n_ck, nkv, hd]."""
    T = k.shape[0]
    n_ck = (T - ks) // st + 1 if T >= ks else 0
    if n_ck <= 0:
        return k.new_zeros((0,) + k.shape[1:])
    return torch.stack([k[st * j: st * j + ks].mean(0) for j in range(n_ck)])


def infllm_select(q, ck, p, sc, nkv, pools=None):
    """Blocks of keys that the query at absolute position p attends to, for
    each kv head: list (per head) of sorted block indices, or None for dense.

    The reference scores compressed keys, max-pools them to blocks, takes the
    top-k and adds a sliding window (src/model/minicpm4/minicpm4_attn.cuh:107-202,
    minicpm4_kvcache.cuh:64-108, src/model/topk.cuh:6-213 with ties to the lower
    index at :17).  It does so per call, which makes its result depend on the
    chunking; here the same stages are a function of the prefix alone:
      1. dense iff p+1 <= dense_len;
      2. ck[j] is visible iff st*j + ks <= p;
      3. score[j] = sum over the heads of the group of softmax_j(q_h.ck[j] hd^-1/2);
      4. pool[b] = max score[j] over visible j whose span overlaps block b
         (-inf if none); +inf for b < init_blocks;
      5. candidates b <= floor(p/bs) - window_size/bs; the min(topk, #cand)
         largest, ties to the lower index;
      6. window: blocks floor(p/bs) - window_size/bs < b <= floor(p/bs).
    q [nh, hd] rotated query, ck [n_ck, nkv, hd].  ``pools``: a list that receives every kv head's
    pooled scores of the candidate blocks (a test asks how clear a choice was)."""
    ks, st, bs = sc["kernel_size"], sc["kernel_stride"], sc["block_size"]
    if p + 1 <= sc["dense_len"]:
        return None
    nh, hd = q.shape
    G = nh // nkv
    lb = sc["window_size"] // bs
    q_block = p // bs
    n_vis = 0 if p < ks else min((p - ks) // st + 1, ck.shape[0])
    n_cand = max(q_block - lb + 1, 0)
    window = list(range(max(q_block - lb + 1, 0), q_block + 1))
    out = []
    for g in range(nkv):
        pool = torch.full((n_cand,), NEG_INF, dtype=q.dtype)
        if n_vis > 0 and n_cand > 0:
            s = (q[g * G:(g + 1) * G] @ ck[:n_vis, g].T) * hd ** -0.5      # [G, n_vis]
            score = torch.softmax(s, dim=-1).sum(0)                       # [n_vis]
            for j in range(n_vis):
                b_lo = (st * j) // bs
                b_hi = (st * j + ks - 1) // bs
                for b in range(b_lo, min(b_hi, n_cand - 1) + 1):
                    pool[b] = max(pool[b], score[j])
        for b in range(min(sc["init_blocks"], n_cand)):
            pool[b] = float("inf")
        if pools is not None:
            pools.append(pool.clone())
        order = sorted(range(n_cand), key=lambda b: (-pool[b].item(), b))
        chosen = sorted(order[:min(sc["topk"], n_cand)])
        out.append(sorted(set(chosen) | set(window)))
    return out


def sparse_allowed(q, k, sc, pos0=0):
    """allowed[i, g, j]: may query i (position pos0+i) of kv head g see key j.
    Dense rows are all True (the causal mask is applied by the caller)."""
    T, nh, hd = q.shape
    nkv = k.shape[1]
    ck = compressed_keys(k, sc["kernel_size"], sc["kernel_stride"])
    bs = sc["block_size"]
    allowed = torch.ones(T, nkv, T, dtype=torch.bool)
    key_block = torch.arange(T) // bs
    for i in range(T):
        sel = infllm_select(q[i], ck, pos0 + i, sc, nkv)
        if sel is None:
            continue
        for g in range(nkv):
            allowed[i, g] = torch.isin(key_block, torch.tensor(sel[g], dtype=torch.long))
    return allowed


def gated_ffn(x, w_gate, w_up, w_down):
    """down( silu(x Wg^T) * (x Wu^T) ) (src/model/ffn.cuh:77-84,
    src/model/activation.cuh:6-18: g*sigmoid(g)*u)."""
    g = x @ w_gate.T
    u = x @ w_up.T
    return (g * torch.sigmoid(g) * u) @ w_down.T


# ----------------------------------------------------------------------------
# whole model
# ----------------------------------------------------------------------------
def attention_layer(cfg, w, prefix, a, positions, inv_freq, m, sparse=True):
    nh = cfg["num_attention_heads"]
    nkv = cfg.get("num_key_value_heads", nh)
    hd = head_dim_of(cfg)
    T = a.shape[0]
    q = (a @ w[prefix + "self_attn.q_proj.weight"].T).view(T, nh, hd)
    k = (a @ w[prefix + "self_attn.k_proj.weight"].T).view(T, nkv, hd)
    v = (a @ w[prefix + "self_attn.v_proj.weight"].T).view(T, nkv, hd)
    q = apply_rope(q, positions, inv_freq, m)
    k = apply_rope(k, positions, inv_freq, m)          # the cache holds rotated keys
    sc = cfg.get("sparse_config") if sparse else None
    allowed = sparse_allowed(q, k, sc) if sc else None
    o = dense_attention(q, k, v, allowed).reshape(T, nh * hd)
    return o @ w[prefix + "self_attn.o_proj.weight"].T


def forward(cfg, weights, tokens, max_seq_len=None, dtype=torch.float64, sparse=True):
    """Logits [T, V] of one whole sequence of token ids.

    Pre-norm decoder; each branch is scaled by scale_depth/sqrt(L) before it is
    added to the residual stream (src/model/minicpm4/minicpm4_layer.cuh:42-62,
    src/model/minicpm4/minicpm4_model.cuh:125-133); final norm, hidden divided
    by hidden/dim_model_base, lm_head (src/model/linear.cuh:86-105); tied
    embeddings reuse the unscaled table (cpmcu/llm.py:136-137)."""
    w = {k: v.to(dtype) for k, v in weights.items()}
    s_e, s_r, s_l = mup_scalars(cfg)
    eps = float(cfg["rms_norm_eps"])
    ids = torch.as_tensor(tokens)
    T = ids.numel()
    positions = torch.arange(T)
    inv_freq, m = rope_inv_freq(cfg, max_seq_len, dtype)
    x = embed(w["model.embed_tokens.weight"], ids, s_e)
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        a = rms_norm(x, w[p + "input_layernorm.weight"], eps)
        x = x + s_r * attention_layer(cfg, w, p, a, positions, inv_freq, m, sparse)
        f = rms_norm(x, w[p + "post_attention_layernorm.weight"], eps)
        x = x + s_r * gated_ffn(f, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"],
                                w[p + "mlp.down_proj.weight"])
    y = rms_norm(x, w["model.norm.weight"], eps) * s_l
    head = w["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings", "lm_head.weight" not in w) \
        else w["lm_head.weight"]
    return y @ head.T


def greedy(cfg, weights, prompt, n_new, stop=(), **kw):
    """Greedy continuation by re-running the whole sequence for each token;
    the stop token is returned and ends the sequence (cpmcu/llm.py:361-373)."""
    toks = list(prompt)
    out = []
    for _ in range(n_new):
        t = int(forward(cfg, weights, toks, **kw)[-1].argmax())
        out.append(t)
        toks.append(t)
        if t in stop:
            break
    return out
