"""Plain torch versions of every kernel in `simply_amd.kernels.ops`, with the same signatures.

Two uses, both in tests only: the reference that each HIP kernel is compared with on the GPU, and
(patched in by the `cpu_ops` fixture) a stand-in that lets the engine's host logic (step function,
cache manager, scheduler) run on a machine without a GPU.  Internal arithmetic is float32 (or
float64 when `PRECISE` is set) whatever the storage type is.
"""
from __future__ import annotations

import math

import torch

PRECISE = False

EPILOGUE_NONE, EPILOGUE_GATED_GELU, EPILOGUE_SOFT_CAP = 0, 1, 2
ALGO_AUTO, ALGO_GENERIC, ALGO_SKINNY, ALGO_TILED = 0, 1, 2, 3


def _f(t) -> torch.Tensor:
    if hasattr(t, "rows"):   # a tiled weight
        from simply_amd.kernels.packing import unpack_tiles
        t = unpack_tiles(t)
    return t.to(torch.float64 if PRECISE else torch.float32)


def embed(table, tokens, scale, out=None):
    r = (_f(table)[tokens.long()] * scale).to(torch.float32)
    if out is not None:
        out.copy_(r)
        return out
    return r


def rmsnorm(x, weight, eps, plus_one, out_dtype, out=None):
    xf = _f(x)
    y = xf * torch.rsqrt((xf * xf).mean(-1, keepdim=True) + eps) * (_f(weight) + (1.0 if plus_one else 0.0))
    y = y.to(out_dtype)
    if out is not None:
        out.copy_(y)
        return out
    return y


def add_rmsnorm(y, residual, *, post_weight=None, post_eps=0.0, post_plus_one=True, next_weight=None, next_eps=0.0,
                next_plus_one=True, out_dtype=None, out=None):
    v = _f(y)
    if post_weight is not None:
        v = v * torch.rsqrt((v * v).mean(-1, keepdim=True) + post_eps) * (_f(post_weight) + (1.0 if post_plus_one else 0.0))
    residual.copy_((_f(residual) + v).to(torch.float32))
    if next_weight is None:
        return None
    return rmsnorm(residual, next_weight, next_eps, next_plus_one, out_dtype or y.dtype, out)


def _rotate(x, positions, timescale, scale_factor):
    """x: [T, n, hd] float; half-split pairs."""
    half = x.shape[-1] // 2
    angle = _f(positions)[:, None, None] / _f(timescale)[None, None, :] / scale_factor
    s, c = torch.sin(angle), torch.cos(angle)
    x1, x2 = x[..., :half], x[..., half:]
    return torch.cat([x1 * c - x2 * s, x2 * c + x1 * s], -1)


def rope_cache_write(qkv, positions, timescale, scale_factor, q_div, num_heads, num_kv_heads, head_dim,
                     slot_mapping=None, k_pages=None, v_pages=None):
    T = qkv.shape[0]
    H, K, hd = num_heads, num_kv_heads, head_dim
    x = _f(qkv).reshape(T, H + 2 * K, hd)
    q, k, v = x[:, :H], x[:, H:H + K], x[:, H + K:]
    if timescale is not None:
        q = _rotate(q, positions, timescale, scale_factor)
        k = _rotate(k, positions, timescale, scale_factor)
    q = q / q_div
    qkv[:, :H * hd] = q.reshape(T, H * hd).to(qkv.dtype)
    if k_pages is not None:
        P = k_pages.shape[2]
        page, off = slot_mapping[:T] // P, slot_mapping[:T] % P
        # element d of the key goes where the layout of a stored page puts it (key_element_index below)
        at = key_element_index(P, hd, off[:, None], torch.arange(hd, device=off.device)[None, :])    # [T, hd]
        flat = k_pages.view(k_pages.shape[0], K, P * hd)
        flat[page[:, None, None], torch.arange(K, device=off.device)[None, :, None], at[:, None, :]] = k.to(k_pages.dtype)
        v_pages[page, :, :, off] = v.to(v_pages.dtype)     # value pages are [page, head, hd, page_size]
    return qkv


def rope(x, positions, timescale, scale_factor, div, num_heads, head_dim):
    T = x.shape[0]
    v = _f(x[:, :num_heads * head_dim]).reshape(T, num_heads, head_dim)
    v = _rotate(v, positions, timescale, scale_factor) / div
    x[:, :num_heads * head_dim] = v.reshape(T, -1).to(x.dtype)


def gather_rows(x, index, out_dtype=None, out=None):
    r = x[index.long()].to(out_dtype or x.dtype)
    if out is not None:
        out.copy_(r)
        return out
    return r


def fill_(t, value_bits=0):
    t.view(torch.int32).fill_(value_bits if value_bits < 2**31 else value_bits - 2**32)


def gelu_tanh(x):
    return 0.5 * x * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (x + 0.044715 * x ** 3)))


def silu(x):
    return x * torch.sigmoid(x)


def squared_relu(x):
    return torch.relu(x) ** 2


ACTIVATIONS = (gelu_tanh, silu, squared_relu)   # by the kernels' activation codes


def gemm(a, w, *, w2=None, soft_cap=None, out_dtype=None, out=None, algo=0, shape=0, activation=0, defer_sum=False):
    # (defer_sum: the kernels may leave a sum to the caller; this stand-in never cuts a product)
    out_dtype = out_dtype or a.dtype
    if getattr(w, "paired", False):
        from simply_amd.kernels.packing import unpack_gate_up
        w, w2 = unpack_gate_up(w)
    c = _f(a) @ _f(w).T
    if w2 is not None:
        up = _f(a) @ _f(w2).T
        c = ACTIVATIONS[activation](_f(c.to(out_dtype))) * _f(up.to(out_dtype))
    elif soft_cap:
        c = soft_cap * torch.tanh(c / soft_cap)
    c = c.to(out_dtype)
    if out is not None:
        out.copy_(c)
        return out
    return c


def key_element_index(P: int, hd: int, key: torch.Tensor, d: torch.Tensor) -> torch.Tensor:
    """Where element d of key `key` (its offset inside a page) lies in a stored page of keys, by the layout's own
    definition (simply_amd/csrc/api.h, sa_paged_attention): row-major [P][hd], unless P % 16 == 0 and hd % 32 == 0;
    then in blocks of 16 keys x 32 dimensions, block (key // 16, d // 32) a contiguous 512 elements holding element
    [(d % 32) // 8 * 16 + key % 16][d % 8] of a [64][8] array, the blocks of a group of 16 keys one after the other.
    (Index arithmetic of the test's own: the product's re-layout functions are not used.)"""
    if P % 16 or hd % 32:
        return key * hd + d
    block = (key // 16) * (hd // 32) + d // 32
    return block * 512 + ((d % 32) // 8 * 16 + key % 16) * 8 + d % 8


def stored_keys_as_rows(k_pages: torch.Tensor) -> torch.Tensor:
    """Pages of keys as the kernels store them [pages, heads, P, hd] -> row-major [pages, heads, P, hd]."""
    n, Kh, P, hd = k_pages.shape
    key = torch.arange(P, device=k_pages.device)[:, None].expand(P, hd)
    d = torch.arange(hd, device=k_pages.device)[None, :].expand(P, hd)
    index = key_element_index(P, hd, key, d).reshape(-1)
    return k_pages.reshape(n, Kh, P * hd)[:, :, index].reshape(n, Kh, P, hd)


def rows_as_stored_keys(rows: torch.Tensor) -> torch.Tensor:
    """Row-major pages of keys [pages, heads, P, hd] -> the kernels' storage order (same shape)."""
    n, Kh, P, hd = rows.shape
    key = torch.arange(P, device=rows.device)[:, None].expand(P, hd)
    d = torch.arange(hd, device=rows.device)[None, :].expand(P, hd)
    index = key_element_index(P, hd, key, d).reshape(-1)
    out = torch.empty_like(rows).reshape(n, Kh, P * hd)
    out[:, :, index] = rows.reshape(n, Kh, P * hd)
    return out.reshape(n, Kh, P, hd)


def paged_attention(q, k_pages, v_pages, block_table, token_seq, positions, num_heads, *, window, soft_cap, out=None,
                    algo=0):
    T = q.shape[0]
    _, Kh, P, hd = k_pages.shape
    k_pages = stored_keys_as_rows(k_pages)
    H = num_heads
    G = H // Kh
    res = torch.empty((T, H * hd), dtype=q.dtype, device=q.device)
    for t in range(T):
        pos = int(positions[t])
        lo = max(pos - window + 1, 0) if window else 0
        keys = torch.arange(lo, pos + 1, device=q.device)
        pages = block_table[int(token_seq[t]), keys // P].long()
        assert (pages >= 0).all(), "attention reads a key that has no page"
        k = _f(k_pages[pages, :, keys % P])          # [n, Kh, hd]
        v = _f(v_pages[pages, :, :, keys % P])       # [n, Kh, hd]
        qt = _f(q[t, :H * hd]).reshape(Kh, G, hd)
        s = torch.einsum("kgd,nkd->kgn", qt, k)
        if soft_cap:
            s = soft_cap * torch.tanh(s / soft_cap)
        p = torch.softmax(s, -1)
        res[t] = torch.einsum("kgn,nkd->kgd", p, v).reshape(H * hd).to(q.dtype)
    if out is not None:
        out.copy_(res)
        return out
    return res


def decode_attention_takes(q, k_pages, num_heads, max_q_len):
    return False


# ---- sampling: the same counter-based generator as the kernel, in integer arithmetic


def philox4x32_10(counter, key):
    M0, M1, W0, W1 = 0xD2511F53, 0xCD9E8D57, 0x9E3779B9, 0xBB67AE85
    c0, c1, c2, c3 = counter
    k0, k1 = key
    mask = 0xFFFFFFFF
    for _ in range(10):
        p0, p1 = M0 * c0, M1 * c2
        c0, c1, c2, c3 = ((p1 >> 32) ^ c1 ^ k0) & mask, p1 & mask, ((p0 >> 32) ^ c3 ^ k1) & mask, p0 & mask
        k0, k1 = (k0 + W0) & mask, (k1 + W1) & mask
    return c0, c1, c2, c3


def gumbel_noise(seed: int, counter: int, vocab: int) -> torch.Tensor:
    """float64 Gumbel noise for every vocabulary entry, from the kernel's random stream."""
    import numpy as np

    idx = np.arange(vocab, dtype=np.uint64)
    blocks = (vocab + 3) // 4
    M0, M1, W0, W1 = np.uint64(0xD2511F53), np.uint64(0xCD9E8D57), 0x9E3779B9, 0xBB67AE85
    m32 = np.uint64(0xFFFFFFFF)
    c0 = np.arange(blocks, dtype=np.uint64)
    c1 = np.full(blocks, counter & 0xFFFFFFFF, dtype=np.uint64)
    c2 = np.zeros(blocks, dtype=np.uint64)
    c3 = np.zeros(blocks, dtype=np.uint64)
    k0, k1 = seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF
    for _ in range(10):
        p0, p1 = M0 * c0, M1 * c2
        n0 = ((p1 >> np.uint64(32)) ^ c1 ^ np.uint64(k0)) & m32
        n1 = p1 & m32
        n2 = ((p0 >> np.uint64(32)) ^ c3 ^ np.uint64(k1)) & m32
        n3 = p0 & m32
        c0, c1, c2, c3 = n0, n1, n2, n3
        k0, k1 = (k0 + W0) & 0xFFFFFFFF, (k1 + W1) & 0xFFFFFFFF
    words = np.stack([c0, c1, c2, c3], axis=1).reshape(-1)[:vocab]
    u = ((words >> np.uint64(8)).astype(np.float64) + 0.5) / 16777216.0
    return torch.from_numpy(-np.log(-np.log(u)))


def sample(logits, temperature, top_k, top_p, seed, counter, tokens=None, logprobs=None, modes=7):
    import sys, os
    sys.path.insert(0, os.path.dirname(__file__))
    import plain_gemma2 as plain

    R, V = logits.shape
    toks = torch.empty(R, dtype=torch.int32)
    lps = torch.empty(R, dtype=torch.float32)
    for r in range(R):
        row = logits[r].double().cpu()
        t, k, p = float(temperature[r]), int(top_k[r]), float(top_p[r])
        if t == 0.0 or k == 1:
            toks[r], lps[r] = int(torch.argmax(row)), 0.0
            continue
        x = row / t
        keep = torch.ones(V, dtype=torch.bool)
        if k > 0:
            keep &= x >= torch.topk(x, min(k, V)).values[-1]
        if p < 1.0:
            xm = torch.where(keep, x, torch.full_like(x, -float("inf")))
            keep &= plain.top_p_mask(xm, p)
        xm = torch.where(keep, x, torch.full_like(x, -float("inf")))
        g = gumbel_noise(int(seed[r]) & (2**64 - 1), int(counter[r]), V)
        tok = int(torch.argmax(xm + g))
        toks[r] = tok
        lps[r] = float(torch.log_softmax(xm, -1)[tok])
    toks, lps = toks.to(logits.device), lps.to(logits.device)
    if tokens is not None:
        tokens[:R] = toks
        toks = tokens
    if logprobs is not None:
        logprobs[:R] = lps
        lps = logprobs
    return toks, lps


SCORE_MASKED = -0.5 * 3.4028234663852886e38


def score(logits, temperature, top_k, top_p, tokens, scores=None):
    """simply/utils/sampling_lib.py:540-601: the log-probability of a given token under temperature, top-k, top-p."""
    import sys, os
    sys.path.insert(0, os.path.dirname(__file__))
    import plain_gemma2 as plain

    R, V = logits.shape
    out = torch.empty(R, dtype=torch.float32)
    for r in range(R):
        row = logits[r].double().cpu()
        t, k, p, tok = float(temperature[r]), int(top_k[r]), float(top_p[r]), int(tokens[r])
        if t == 0.0 or k == 1:
            out[r] = 0.0 if int(torch.argmax(row)) == tok else SCORE_MASKED
            continue
        x = row / t
        keep = torch.ones(V, dtype=torch.bool)
        if k > 0:
            keep &= x >= torch.topk(x, min(k, V)).values[-1]
        if p < 1.0:
            xm = torch.where(keep, x, torch.full_like(x, -float("inf")))
            keep &= plain.top_p_mask(xm, p)
        xm = torch.where(keep, x, torch.full_like(x, -float("inf")))
        out[r] = float(torch.log_softmax(xm, -1)[tok]) if bool(keep[tok]) else SCORE_MASKED
    out = out.to(logits.device)
    if scores is not None:
        scores[:R] = out
        out = scores
    return out
