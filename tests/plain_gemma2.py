"""A plain, slow Gemma 2 decoder: whole sequences, no cache, one function per part.

Written from the formulas of google-deepmind/simply (each function cites the file
and lines it follows). It shares no code with the `simply_amd` package: it reads
`config.json` and `model.safetensors` itself and computes with ordinary torch
operations on the CPU, in the dtype it is asked for (float32 or float64).

Tensor names and layouts are those of the model folder: linear weights are
`[out_features, in_features]`.

Every part takes a `Rounding`: the places at which a run in a 16-bit activation type rounds its
intermediate results, so that the arithmetic of such a run can be followed on the CPU, place by
place, while everything between the places stays in the dtype asked for.  The default rounds nowhere.
"""
from __future__ import annotations

import json
import math
import os

import torch


# --------------------------------------------------------------------------- rounding


class Rounding:
    """Rounds to `dtype` (and back) at the named places, nowhere else.

    Places (what google-deepmind/simply rounds when `activation_dtype` is bfloat16):
      embed_scale  the factor sqrt(dim) (simply/utils/module.py:476-480)
      embed        the scaled embedding (same lines: the product is in the activation dtype)
      norm_inner   x * rsqrt(var + eps) before the gain, and the gain `scale + 1` itself
                   (simply/model_lib.py:166-173)
      norm_out     the norm's result (simply/model_lib.py:174)
      proj         results of the projections q, k, v, o, down (einsum in the activation dtype,
                   simply/utils/module.py:339-343)
      rope         rotated queries and keys, cast back from float32 (simply/utils/position_encoding.py:110);
                   the scaled query (simply/kernels/ragged_paged_attention.py:217-224)
      scores       q.k cast to the output dtype before the cap (simply/kernels/ragged_paged_attention.py:226-228;
                   the dense path keeps float32 here, simply/model_lib.py:623-625)
      probs        softmax cast to the values' dtype (simply/kernels/ragged_paged_attention.py:247;
                   simply/model_lib.py:634)
      attn_out     probs . v (simply/kernels/ragged_paged_attention.py:249)
      ffn_parts    gate and up each, and the activated gate (simply/model_lib.py:714-727)
      ffn_mid      act(gate) * up (simply/model_lib.py:727)
      residual     y + h (simply/model_lib.py:2683, 2700: `x += x_res` in the activation dtype)
      logits       the head's product and its soft-cap (simply/model_lib.py:3186-3188)
    """

    PLACES = ("embed_scale", "embed", "norm_inner", "norm_out", "proj", "rope", "scores", "probs", "attn_out",
              "ffn_parts", "ffn_mid", "residual", "logits")

    def __init__(self, dtype: torch.dtype | None = None, places=()):
        unknown = set(places) - set(self.PLACES)
        if unknown:
            raise ValueError(f"unknown rounding places {sorted(unknown)}")
        self.dtype, self.places = dtype, frozenset(places)

    def __call__(self, place: str, x: torch.Tensor) -> torch.Tensor:
        if self.dtype is None or place not in self.places:
            return x
        return x.to(self.dtype).to(x.dtype)


NO_ROUNDING = Rounding()


def rounding_like_simply(dtype=torch.bfloat16) -> Rounding:
    """Every place at which google-deepmind/simply rounds in a 16-bit activation dtype (paged serving path)."""
    return Rounding(dtype, Rounding.PLACES)


def rounding_of_fp32_residual_engine(dtype=torch.bfloat16) -> Rounding:
    """The places that are left when the residual stream, the norms' inner product, the scores and the logits are
    kept in 32-bit and the gated product is rounded once: what an engine that holds 16-bit activations only between
    its kernels does."""
    return Rounding(dtype, ("embed_scale", "norm_out", "proj", "rope", "probs", "attn_out", "ffn_mid"))


# --------------------------------------------------------------------------- parts


def rms_norm(x: torch.Tensor, scale: torch.Tensor, eps: float, rnd: Rounding = NO_ROUNDING) -> torch.Tensor:
    """RMSNorm with a `(1 + scale)` gain.

    simply/model_lib.py:154-178 (LayerNorm.apply with use_bias=False,
    scale_plus_one=True): var = mean(x^2); x *= rsqrt(var + eps); x *= scale + 1.
    """
    var = torch.mean(x * x, dim=-1, keepdim=True)
    x = rnd("norm_inner", x * torch.rsqrt(var + eps))
    return rnd("norm_out", x * rnd("norm_inner", scale + 1.0))


def rope(x: torch.Tensor, positions: torch.Tensor, base: float) -> torch.Tensor:
    """Rotary position encoding, half-split pairing (i, i + hd/2).

    simply/utils/position_encoding.py:83-110: fraction = 2i/hd,
    timescale = base**fraction (min_timescale 1), angle = pos / timescale,
    out = concat(x1*cos - x2*sin, x2*cos + x1*sin).

    x: [T, heads, hd]; positions: [T].
    """
    hd = x.shape[-1]
    half = hd // 2
    fraction = 2.0 * torch.arange(0, half, dtype=x.dtype, device=x.device) / hd
    timescale = torch.as_tensor(base, dtype=x.dtype, device=x.device) ** fraction
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


def attention(q, k, v, mask, cap: float | None, rnd: Rounding = NO_ROUNDING) -> torch.Tensor:
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
    s = rnd("scores", torch.einsum("thd,shd->hts", q, k))
    if cap is not None and cap > 0:
        s = soft_cap(s, cap)
    # simply/utils/common.py:543-551: mask value is -0.5 * float32 max.
    mask_value = -0.5 * torch.finfo(torch.float32).max
    s = torch.where(mask[None, :, :], s, torch.as_tensor(mask_value, dtype=s.dtype, device=s.device))
    p = rnd("probs", torch.softmax(s, dim=-1))
    return rnd("attn_out", torch.einsum("hts,shd->thd", p, v))


def attention_layer(x, positions, w, prefix, cfg, visible, rnd: Rounding = NO_ROUNDING) -> torch.Tensor:
    """q/k/v projections -> RoPE on q and k -> query scale -> attention -> o projection.

    simply/model_lib.py:2106-2110 (projections), :1987-2020 (_scale_qk: RoPE first,
    then q / query_scale), :2362 (o projection).  query_scale is
    sqrt(query_pre_attn_scalar) (simply/config_lib.py:944: sqrt(4608/32) for 27B;
    default sqrt(per_head_dim), simply/model_lib.py:2017-2019).
    """
    T = x.shape[0]
    H, K, hd = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    q = rnd("proj", x @ w[prefix + "q_proj.weight"].T).reshape(T, H, hd)
    k = rnd("proj", x @ w[prefix + "k_proj.weight"].T).reshape(T, K, hd)
    v = rnd("proj", x @ w[prefix + "v_proj.weight"].T).reshape(T, K, hd)
    base = float(cfg.get("rope_theta", 10000.0))
    q = rnd("rope", rope(q, positions, base))
    k = rnd("rope", rope(k, positions, base))
    q = rnd("rope", q / math.sqrt(float(cfg.get("query_pre_attn_scalar", hd))))
    mask = attention_mask(positions, positions, visible)
    o = attention(q, k, v, mask, cfg.get("attn_logit_softcapping"), rnd)
    return rnd("proj", o.reshape(T, H * hd) @ w[prefix + "o_proj.weight"].T)


def feed_forward(x, w, prefix, rnd: Rounding = NO_ROUNDING) -> torch.Tensor:
    """Gated feed-forward: down(gelu(gate(x)) * up(x)).

    simply/model_lib.py:714-730: projected = ffn_0(x) (up), gate = ffn_0_gate(x),
    x = act(gate) * projected, out = ffn_1(x).
    """
    gate = rnd("ffn_parts", x @ w[prefix + "gate_proj.weight"].T)
    up = rnd("ffn_parts", x @ w[prefix + "up_proj.weight"].T)
    mid = rnd("ffn_mid", rnd("ffn_parts", gelu_tanh(gate)) * up)
    return rnd("proj", mid @ w[prefix + "down_proj.weight"].T)


def block(x, positions, w, i, cfg, visible, rnd: Rounding = NO_ROUNDING) -> torch.Tensor:
    """One decoder block with four norms.

    simply/model_lib.py:2669-2703: h = x; y = pre_ln_0(x); y = attn(y);
    y = post_ln_0(y); x = y + h; h = x; y = pre_ln_1(x); y = ffn(y);
    y = post_ln_1(y); x = y + h.
    """
    p = f"model.layers.{i}."
    eps = float(cfg.get("rms_norm_eps", 1e-6))
    h = x
    y = rms_norm(x, w[p + "input_layernorm.weight"], eps, rnd)
    y = attention_layer(y, positions, w, p + "self_attn.", cfg, visible, rnd)
    y = rms_norm(y, w[p + "post_attention_layernorm.weight"], eps, rnd)
    x = rnd("residual", y + h)
    h = x
    y = rms_norm(x, w[p + "pre_feedforward_layernorm.weight"], eps, rnd)
    y = feed_forward(y, w, p + "mlp.", rnd)
    y = rms_norm(y, w[p + "post_feedforward_layernorm.weight"], eps, rnd)
    return rnd("residual", y + h)


def layer_is_sliding(cfg: dict, i: int) -> bool:
    """simply/model_lib.py:2839-2844 with block_attn_pattern ('local', 'global')
    (simply/config_lib.py:876-879): even layers are windowed, odd layers global."""
    types = cfg.get("layer_types")
    if types is not None:
        return types[i] == "sliding_attention"
    return i % 2 == 0


def embed(tokens, w, cfg, rnd: Rounding = NO_ROUNDING) -> torch.Tensor:
    """simply/utils/module.py:450-481: take(w, tokens) * sqrt(dim), the factor in the activation dtype."""
    table = w["model.embed_tokens.weight"]
    factor = rnd("embed_scale", torch.as_tensor(math.sqrt(cfg["hidden_size"]), dtype=table.dtype, device=table.device))
    return rnd("embed", table[tokens] * factor)


def lm_head(x, w, cfg, rnd: Rounding = NO_ROUNDING) -> torch.Tensor:
    """simply/model_lib.py:3184-3189: final norm, tied head ('vd,...d->...v' on the
    embedding table), then the final soft-cap if it is > 0."""
    x = rms_norm(x, w["model.norm.weight"], float(cfg.get("rms_norm_eps", 1e-6)), rnd)
    logits = rnd("logits", x @ head_table(w, cfg).T)
    cap = cfg.get("final_logit_softcapping")
    if cap is not None and cap > 0:
        logits = rnd("logits", soft_cap(logits, cap))
    return logits


def head_table(w, cfg) -> torch.Tensor:
    """The head's matrix: the embedding table when the two are tied (simply/utils/module.py:421-441,
    use_tied_embedding), else a tensor of its own."""
    if cfg.get("tie_word_embeddings", True):
        return w["model.embed_tokens.weight"]
    return w["lm_head.weight"]


# --------------------------------------------------------------------------- model


def forward(w: dict, cfg: dict, tokens, dtype=torch.float32, first_position: int = 0,
            rnd: Rounding = NO_ROUNDING, device=None) -> torch.Tensor:
    """Logits [T, V] at every position of one whole sequence (simply/model_lib.py:2935-3189).  `device`: where
    torch computes it (the CPU unless a long sequence at large sizes wants a faster place)."""
    tokens = torch.as_tensor(tokens, dtype=torch.long, device=device)
    w = {k: v.to(device=device, dtype=dtype) for k, v in w.items()}
    positions = torch.arange(first_position, first_position + tokens.numel(), device=device)
    x = embed(tokens, w, cfg, rnd)
    for i in range(cfg["num_hidden_layers"]):
        visible = cfg.get("sliding_window") if layer_is_sliding(cfg, i) else None
        x = block(x, positions, w, i, cfg, visible, rnd)
    return lm_head(x, w, cfg, rnd)


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
