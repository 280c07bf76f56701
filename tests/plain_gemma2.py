"""A plain, slow Gemma 2 decoder: whole sequences, no cache, one function per part.

Written from the formulas of google-deepmind/simply (each function cites the file
and lines it follows). It shares no code with the `simply_amd` package: it reads
`config.json` and `model.safetensors` itself and computes with ordinary torch
operations on the CPU, in the dtype it is asked for (float32 or float64).

Tensor names and layouts are those of the model folder: linear weights are
`[out_features, in_features]`.
"""
from __future__ import annotations

import json
import math
import os

import torch


# --------------------------------------------------------------------------- parts


def rms_norm(x: torch.Tensor, scale: torch.Tensor, eps: float) -> torch.Tensor:
    """RMSNorm with a `(1 + scale)` gain.

    simply/model_lib.py:154-178 (LayerNorm.apply with use_bias=False,
    scale_plus_one=True): var = mean(x^2); x *= rsqrt(var + eps); x *= scale + 1.
    """
    var = torch.mean(x * x, dim=-1, keepdim=True)
    x = x * torch.rsqrt(var + eps)
    return x * (scale + 1.0)


def rope(x: torch.Tensor, positions: torch.Tensor, base: float) -> torch.Tensor:
    """Rotary position encoding, half-split pairing (i, i + hd/2).

    simply/utils/position_encoding.py:83-110: fraction = 2i/hd,
    timescale = base**fraction (min_timescale 1), angle = pos / timescale,
    out = concat(x1*cos - x2*sin, x2*cos + x1*sin).

    x: [T, heads, hd]; positions: [T].
    """
    hd = x.shape[-1]
    half = hd // 2
    fraction = 2.0 * torch.arange(0, half, dtype=x.dtype) / hd
    timescale = torch.as_tensor(base, dtype=x.dtype) ** fraction
    angle = positions.to(x.dtype)[:, None, None] / timescale[None, None, :]
    sin, cos = torch.sin(angle), torch.cos(angle)
    x1, x2 = x[..., :half], x[..., half:]
    return torch.cat([x1 * cos - x2 * sin, x2 * cos + x1 * sin], dim=-1)


def gelu_tanh(x: torch.Tensor) -> torch.Tensor:
    """simply/model_lib.py:94-96: 0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3)))."""
    return 0.5 * x * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (x + 0.044715 * x**3)))


def soft_cap(x: torch.Tensor, cap: float) -> torch.Tensor:
    """simply/model_lib.py:107-109: cap * tanh(x / cap)."""
    return cap * torch.tanh(x / cap)


def attention_mask(q_pos: torch.Tensor, k_pos: torch.Tensor, visible: int | None) -> torch.Tensor:
    """Boolean [Tq, Tk] mask: True where the query may look at the key.

    simply/model_lib.py:469-515 (create_mask): causal `q_pos >= k_pos`, and for a
    windowed layer `q_pos - k_pos <= window_size`. `visible` is the number of keys a
    query sees including itself, i.e. Simply's `window_size + 1`
    (simply/utils/ragged_paged_attention.py:922 passes sliding_window = window_size + 1;
    simply/kernels/ragged_paged_attention.py:237-241 masks q_span < k_span + sliding_window).
    """
    diff = q_pos[:, None] - k_pos[None, :]
    mask = diff >= 0
    if visible is not None:
        mask = mask & (diff < visible)
    return mask


def attention(q, k, v, mask, cap: float | None) -> torch.Tensor:
    """Scores -> cap -> mask -> softmax -> weighted values.

    simply/model_lib.py:611-638 (attn): logits = q.k (no further scaling: the query
    was already divided by query_scale), soft-capped if cap > 0, masked entries are
    *replaced* by the mask value, softmax over keys, output = probs . v.
    GQA: query head h reads key/value head h // G (simply/model_lib.py:2306-2310;
    simply/kernels/ragged_paged_attention.py:214-215 repeats each kv head G times).

    q: [T, H, hd]; k, v: [S, K, hd]; mask: [T, S].  Returns [T, H, hd].
    """
    H, K = q.shape[1], k.shape[1]
    G = H // K
    k = k.repeat_interleave(G, dim=1)
    v = v.repeat_interleave(G, dim=1)
    s = torch.einsum("thd,shd->hts", q, k)
    if cap is not None and cap > 0:
        s = soft_cap(s, cap)
    # simply/utils/common.py:543-551: mask value is -0.5 * float32 max.
    mask_value = -0.5 * torch.finfo(torch.float32).max
    s = torch.where(mask[None, :, :], s, torch.as_tensor(mask_value, dtype=s.dtype))
    p = torch.softmax(s, dim=-1)
    return torch.einsum("hts,shd->thd", p, v)


def attention_layer(x, positions, w, prefix, cfg, visible) -> torch.Tensor:
    """q/k/v projections -> RoPE on q and k -> query scale -> attention -> o projection.

    simply/model_lib.py:2106-2110 (projections), :1987-2020 (_scale_qk: RoPE first,
    then q / query_scale), :2362 (o projection).  query_scale is
    sqrt(query_pre_attn_scalar) (simply/config_lib.py:944: sqrt(4608/32) for 27B;
    default sqrt(per_head_dim), simply/model_lib.py:2017-2019).
    """
    T = x.shape[0]
    H, K, hd = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    q = (x @ w[prefix + "q_proj.weight"].T).reshape(T, H, hd)
    k = (x @ w[prefix + "k_proj.weight"].T).reshape(T, K, hd)
    v = (x @ w[prefix + "v_proj.weight"].T).reshape(T, K, hd)
    base = float(cfg.get("rope_theta", 10000.0))
    q = rope(q, positions, base)
    k = rope(k, positions, base)
    q = q / math.sqrt(float(cfg.get("query_pre_attn_scalar", hd)))
    mask = attention_mask(positions, positions, visible)
    o = attention(q, k, v, mask, cfg.get("attn_logit_softcapping"))
    return o.reshape(T, H * hd) @ w[prefix + "o_proj.weight"].T


def feed_forward(x, w, prefix) -> torch.Tensor:
    """Gated feed-forward: down(gelu(gate(x)) * up(x)).

    simply/model_lib.py:714-730: projected = ffn_0(x) (up), gate = ffn_0_gate(x),
    x = act(gate) * projected, out = ffn_1(x).
    """
    gate = x @ w[prefix + "gate_proj.weight"].T
    up = x @ w[prefix + "up_proj.weight"].T
    return (gelu_tanh(gate) * up) @ w[prefix + "down_proj.weight"].T


def block(x, positions, w, i, cfg, visible) -> torch.Tensor:
    """One decoder block with four norms.

    simply/model_lib.py:2669-2703: h = x; y = pre_ln_0(x); y = attn(y);
    y = post_ln_0(y); x = y + h; h = x; y = pre_ln_1(x); y = ffn(y);
    y = post_ln_1(y); x = y + h.
    """
    p = f"model.layers.{i}."
    eps = float(cfg.get("rms_norm_eps", 1e-6))
    h = x
    y = rms_norm(x, w[p + "input_layernorm.weight"], eps)
    y = attention_layer(y, positions, w, p + "self_attn.", cfg, visible)
    y = rms_norm(y, w[p + "post_attention_layernorm.weight"], eps)
    x = y + h
    h = x
    y = rms_norm(x, w[p + "pre_feedforward_layernorm.weight"], eps)
    y = feed_forward(y, w, p + "mlp.")
    y = rms_norm(y, w[p + "post_feedforward_layernorm.weight"], eps)
    return y + h


def layer_is_sliding(cfg: dict, i: int) -> bool:
    """simply/model_lib.py:2839-2844 with block_attn_pattern ('local', 'global')
    (simply/config_lib.py:876-879): even layers are windowed, odd layers global."""
    types = cfg.get("layer_types")
    if types is not None:
        return types[i] == "sliding_attention"
    return i % 2 == 0


def embed(tokens, w, cfg) -> torch.Tensor:
    """simply/utils/module.py:450-481: take(w, tokens) * sqrt(dim)."""
    table = w["model.embed_tokens.weight"]
    return table[tokens] * math.sqrt(cfg["hidden_size"])


def lm_head(x, w, cfg) -> torch.Tensor:
    """simply/model_lib.py:3184-3189: final norm, tied head ('vd,...d->...v' on the
    embedding table), then the final soft-cap if it is > 0."""
    x = rms_norm(x, w["model.norm.weight"], float(cfg.get("rms_norm_eps", 1e-6)))
    logits = x @ w["model.embed_tokens.weight"].T
    cap = cfg.get("final_logit_softcapping")
    if cap is not None and cap > 0:
        logits = soft_cap(logits, cap)
    return logits


# --------------------------------------------------------------------------- model


def forward(w: dict, cfg: dict, tokens, dtype=torch.float32, first_position: int = 0) -> torch.Tensor:
    """Logits [T, V] at every position of one whole sequence (simply/model_lib.py:2935-3189)."""
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    w = {k: v.to(dtype) for k, v in w.items()}
    positions = torch.arange(first_position, first_position + tokens.numel())
    x = embed(tokens, w, cfg)
    for i in range(cfg["num_hidden_layers"]):
        visible = cfg.get("sliding_window") if layer_is_sliding(cfg, i) else None
        x = block(x, positions, w, i, cfg, visible)
    return lm_head(x, w, cfg)


def load(model_dir: str):
    from safetensors.torch import load_file

    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    w = load_file(os.path.join(model_dir, "model.safetensors"))
    return w, cfg


def greedy(w, cfg, prompt, n, dtype=torch.float32) -> list[int]:
    """Greedy continuation by re-running the whole sequence for every new token
    (temperature 0 is argmax: simply/utils/sampling_lib.py:494-497, 532-537)."""
    seq = list(prompt)
    out = []
    for _ in range(n):
        logits = forward(w, cfg, seq, dtype)
        nxt = int(torch.argmax(logits[-1]))
        out.append(nxt)
        seq.append(nxt)
    return out


# --------------------------------------------------------------------------- sampling


def top_k_mask(logits: torch.Tensor, top_k: int) -> torch.Tensor:
    """simply/utils/sampling_lib.py:427-431: keep the k largest logits."""
    k = max(min(top_k, logits.shape[-1]), 1)
    idx = torch.topk(logits, k, dim=-1).indices
    mask = torch.zeros_like(logits, dtype=torch.bool)
    return mask.scatter(-1, idx, True)


def top_p_mask(logits: torch.Tensor, top_p: float) -> torch.Tensor:
    """simply/utils/sampling_lib.py:434-441: sort descending, cumulative sum that
    starts at 0; a token stays while the mass *before* it is < top_p (so the token
    that crosses top_p is kept)."""
    probs = torch.softmax(logits, dim=-1)
    sorted_probs, idx = torch.sort(probs, dim=-1, descending=True, stable=True)
    before = torch.cumsum(sorted_probs, dim=-1) - sorted_probs
    keep_sorted = before < top_p
    mask = torch.zeros_like(logits, dtype=torch.bool)
    return mask.scatter(-1, idx, keep_sorted)


def log_prob(logits: torch.Tensor, token: int, temperature: float) -> float:
    """simply/utils/sampling_lib.py:500-504 with simply/utils/distributions.py:73-74:
    log_softmax(logits / temperature)[token]."""
    return float(torch.log_softmax(logits.double() / temperature, dim=-1)[token])
