"""Pins the plain implementation by what fixes it beside the reference's text: vectors that the
reference's own tests hold, special cases that reduce to a library routine, and invariants, each chosen
so that a plausible mistake (a wrong sign or pairing, a norm in the wrong place) fails it."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import plain_gemma2 as plain
import tiny

torch.manual_seed(0)


def weights(cfg, seed=0, std=0.3, norm_std=0.2, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    D, H, K, hd, Fd, V = (cfg[k] for k in ("hidden_size", "num_attention_heads", "num_key_value_heads", "head_dim",
                                           "intermediate_size", "vocab_size"))
    w = {"model.embed_tokens.weight": torch.randn(V, D, generator=g) * std,
         "model.norm.weight": torch.randn(D, generator=g) * norm_std}
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        for n, shape in (("self_attn.q_proj", (H * hd, D)), ("self_attn.k_proj", (K * hd, D)),
                         ("self_attn.v_proj", (K * hd, D)), ("self_attn.o_proj", (D, H * hd)),
                         ("mlp.gate_proj", (Fd, D)), ("mlp.up_proj", (Fd, D)), ("mlp.down_proj", (D, Fd))):
            w[p + n + ".weight"] = torch.randn(shape, generator=g) * std
        for n in ("input_layernorm", "post_attention_layernorm", "pre_feedforward_layernorm", "post_feedforward_layernorm"):
            w[p + n + ".weight"] = torch.randn(D, generator=g) * norm_std
    return {k: v.to(dtype) for k, v in w.items()}


# ------------------------------------------------------------------ norm
def test_rmsnorm_reduces_to_library_routine_and_has_one_plus_gain():
    x = torch.randn(5, 24, dtype=torch.float64) * 3
    zero = torch.zeros(24, dtype=torch.float64)
    torch.testing.assert_close(plain.rms_norm(x, zero, 1e-6), F.rms_norm(x, (24,), eps=1e-6))
    w = torch.randn(24, dtype=torch.float64) * 0.1
    torch.testing.assert_close(plain.rms_norm(x, w, 1e-6), F.rms_norm(x, (24,), weight=1 + w, eps=1e-6))
    # scale-equivariance: the norm forgets the input's scale (up to eps)
    torch.testing.assert_close(plain.rms_norm(7 * x, w, 1e-12), plain.rms_norm(x, w, 1e-12))
    # eps enters under the root: a zero row stays zero and finite
    assert torch.equal(plain.rms_norm(torch.zeros(1, 24, dtype=torch.float64), w, 1e-6), torch.zeros(1, 24, dtype=torch.float64))
    # a `w` gain instead of `1 + w` would make this small
    assert plain.rms_norm(x, w, 1e-6).abs().mean() > 0.5


# ------------------------------------------------------------------ rope
def test_rope_properties():
    hd = 16
    x = torch.randn(6, 3, hd, dtype=torch.float64)
    pos = torch.tensor([0, 1, 2, 3, 50, 51])
    y = plain.rope(x, pos, 10000.0)
    torch.testing.assert_close(y[0], x[0])                      # position 0 is the identity
    half = hd // 2                                              # each pair (i, i + hd/2) keeps its norm
    torch.testing.assert_close(y[..., :half] ** 2 + y[..., half:] ** 2, x[..., :half] ** 2 + x[..., half:] ** 2)
    # a one-hot at index 0 moves energy to index hd/2 (half-split pairs), not to index 1 (interleaved pairs)
    e = torch.zeros(1, 1, hd, dtype=torch.float64)
    e[0, 0, 0] = 1.0
    r = plain.rope(e, torch.tensor([1]), 10000.0)[0, 0]
    assert abs(r[0] - math.cos(1.0)) < 1e-12 and abs(r[half] - math.sin(1.0)) < 1e-12 and r[1] == 0
    # the slowest pair turns by pos / base**((hd-2)/hd)
    e = torch.zeros(1, 1, hd, dtype=torch.float64)
    e[0, 0, half - 1] = 1.0
    r = plain.rope(e, torch.tensor([100]), 10000.0)[0, 0]
    ang = 100 / 10000.0 ** ((hd - 2) / hd)
    assert abs(r[half - 1] - math.cos(ang)) < 1e-12 and abs(r[hd - 1] - math.sin(ang)) < 1e-12
    # <rope(q, m), rope(k, n)> depends on m - n only
    q, k = torch.randn(1, 1, hd, dtype=torch.float64), torch.randn(1, 1, hd, dtype=torch.float64)
    dots = [(plain.rope(q, torch.tensor([m]), 1e4) * plain.rope(k, torch.tensor([m - 7]), 1e4)).sum() for m in (7, 19, 300)]
    torch.testing.assert_close(dots[0], dots[1])
    torch.testing.assert_close(dots[0], dots[2])
    # the base matters (simply/utils/position_encoding_test.py:61-66)
    assert not torch.allclose(plain.rope(x, pos, 1e4), plain.rope(x, pos, 1e6))


# ------------------------------------------------------------------ masks (the reference's own vectors)
def test_mask_vectors_of_the_reference():
    # simply/model_lib_test.py:483-522: window_size=1 -> the query and one key before it
    pos = torch.arange(4)
    m = plain.attention_mask(pos, pos, visible=2)
    assert m.int().tolist() == [[1, 0, 0, 0], [1, 1, 0, 0], [0, 1, 1, 0], [0, 0, 1, 1]]
    # simply/model_lib_test.py:524-538: window_size=2 -> three visible
    m = plain.attention_mask(pos, pos, visible=3)
    assert m.int().tolist() == [[1, 0, 0, 0], [1, 1, 0, 0], [1, 1, 1, 0], [0, 1, 1, 1]]
    # simply/model_lib_test.py:540-551: one decoded query at position 7 over keys at 3..7
    m = plain.attention_mask(torch.tensor([7]), torch.tensor([3, 4, 5, 6, 7]), None)
    assert m.tolist() == [[True] * 5]
    # no window: plain causal
    assert plain.attention_mask(pos, pos, None).int().tolist() == torch.tril(torch.ones(4, 4)).int().tolist()


# ------------------------------------------------------------------ attention
def test_attention_reduces_to_library_routine():
    T, H, hd = 9, 3, 8
    q, k, v = (torch.randn(T, H, hd, dtype=torch.float64) for _ in range(3))
    pos = torch.arange(T)
    got = plain.attention(q, k, v, plain.attention_mask(pos, pos, None), None)
    # the library scales by 1/sqrt(hd); the plain function expects an already scaled query
    want = F.scaled_dot_product_attention((q * math.sqrt(hd)).transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1),
                                          is_causal=True).transpose(0, 1)
    torch.testing.assert_close(got, want)
    # one key only: the output is that key's value, whatever the scores are
    got1 = plain.attention(q[:1], k[:1], v[:1], torch.ones(1, 1, dtype=torch.bool), 50.0)
    torch.testing.assert_close(got1, v[:1])


def test_attention_cap_before_mask_and_grouping():
    T, H, K, hd = 5, 4, 2, 8
    q, k, v = torch.randn(T, H, hd, dtype=torch.float64) * 5, torch.randn(T, K, hd, dtype=torch.float64) * 5, None
    # kv heads hold distinct constants: query head h must read kv head h // G
    v = torch.stack([torch.full((T, hd), float(j + 1), dtype=torch.float64) for j in range(K)], dim=1)
    pos = torch.arange(T)
    out = plain.attention(q, k, v, plain.attention_mask(pos, pos, None), 50.0)
    for h in range(H):
        torch.testing.assert_close(out[:, h], torch.full((T, hd), float(h // 2 + 1), dtype=torch.float64))
    # the cap bounds the scores: with a tiny cap the softmax over visible keys is nearly uniform, and masked keys
    # (which are replaced after the cap, not capped) still get nothing
    v2 = torch.zeros(T, K, hd, dtype=torch.float64)
    v2[-1] = 1.0  # only the last key carries value
    out = plain.attention(q, k, v2, plain.attention_mask(pos, pos, None), 1e-6)
    torch.testing.assert_close(out[-1], torch.full((H, hd), 1.0 / T, dtype=torch.float64), rtol=1e-4, atol=1e-4)
    assert out[:-1].abs().max() == 0
    # cap formula
    s = torch.tensor([-100.0, -1.0, 0.0, 2.0, 1000.0], dtype=torch.float64)
    torch.testing.assert_close(plain.soft_cap(s, 30.0), 30 * torch.tanh(s / 30))
    assert plain.soft_cap(s, 30.0).abs().max() <= 30.0


def test_query_scale_is_applied_once_and_after_rope():
    cfg = dict(tiny.TINY_B, num_hidden_layers=1)
    w = weights(cfg)
    x = torch.randn(7, cfg["hidden_size"], dtype=torch.float64)
    pos = torch.arange(7)
    base = plain.attention_layer(x, pos, w, "model.layers.0.self_attn.", cfg, None)
    # scaling the query weights by c and query_pre_attn_scalar by c^2 changes nothing
    w2 = dict(w)
    w2["model.layers.0.self_attn.q_proj.weight"] = w["model.layers.0.self_attn.q_proj.weight"] * 3.0
    cfg2 = dict(cfg, query_pre_attn_scalar=cfg["query_pre_attn_scalar"] * 9.0)
    torch.testing.assert_close(plain.attention_layer(x, pos, w2, "model.layers.0.self_attn.", cfg2, None), base)
    # but the scalar alone does (it is not head_dim here: 24 != 32)
    cfg3 = dict(cfg, query_pre_attn_scalar=cfg["head_dim"])
    assert not torch.allclose(plain.attention_layer(x, pos, w, "model.layers.0.self_attn.", cfg3, None), base)


# ------------------------------------------------------------------ feed-forward
def test_gelu_and_gate():
    x = torch.linspace(-6, 6, 101, dtype=torch.float64)
    torch.testing.assert_close(plain.gelu_tanh(x), F.gelu(x, approximate="tanh"))
    cfg = dict(tiny.TINY_A, num_hidden_layers=1)
    w = weights(cfg)
    xs = torch.randn(3, cfg["hidden_size"], dtype=torch.float64)
    p = "model.layers.0.mlp."
    got = plain.feed_forward(xs, w, p)
    want = (F.gelu(xs @ w[p + "gate_proj.weight"].T, approximate="tanh") * (xs @ w[p + "up_proj.weight"].T)) @ w[p + "down_proj.weight"].T
    torch.testing.assert_close(got, want)
    swapped = dict(w)
    swapped[p + "gate_proj.weight"], swapped[p + "up_proj.weight"] = w[p + "up_proj.weight"], w[p + "gate_proj.weight"]
    assert not torch.allclose(plain.feed_forward(xs, swapped, p), got)   # the gate is the activated branch


# ------------------------------------------------------------------ block, embedding, head
def test_block_is_identity_when_post_norms_vanish():
    """x + post_ln(f(pre_ln(x))): post-norm gains of 1 + w = 0 leave the residual alone."""
    cfg = dict(tiny.TINY_A, num_hidden_layers=1)
    w = weights(cfg)
    x = torch.randn(6, cfg["hidden_size"], dtype=torch.float64)
    pos = torch.arange(6)
    assert not torch.allclose(plain.block(x, pos, w, 0, cfg, 8), x)
    for n in ("post_attention_layernorm", "post_feedforward_layernorm"):
        w[f"model.layers.0.{n}.weight"] = torch.full((cfg["hidden_size"],), -1.0, dtype=torch.float64)
    torch.testing.assert_close(plain.block(x, pos, w, 0, cfg, 8), x)
    # with only the feed-forward's post-norm at zero the block is x + post(attn(pre(x)))
    w = weights(cfg)
    w["model.layers.0.post_feedforward_layernorm.weight"] = torch.full((cfg["hidden_size"],), -1.0, dtype=torch.float64)
    eps = cfg["rms_norm_eps"]
    y = plain.rms_norm(x, w["model.layers.0.input_layernorm.weight"], eps)
    y = plain.attention_layer(y, pos, w, "model.layers.0.self_attn.", cfg, 8)
    y = plain.rms_norm(y, w["model.layers.0.post_attention_layernorm.weight"], eps)
    torch.testing.assert_close(plain.block(x, pos, w, 0, cfg, 8), x + y)


def test_embedding_and_head():
    cfg = dict(tiny.TINY_B)
    w = weights(cfg)
    # a table drawn N(0, 1 / D), the initialisation that simply/utils/module.py:470-474 names as the reason for the
    # factor, gives embeddings of variance 1: without the factor it would be 1 / D, with it twice D
    D = 4096
    table = torch.randn(1000, D, generator=torch.Generator().manual_seed(1), dtype=torch.float64) / math.sqrt(D)
    e = plain.embed(torch.arange(1000), {"model.embed_tokens.weight": table}, {"hidden_size": D})
    assert abs(e.var().item() - 1.0) < 0.01
    assert torch.equal(plain.embed(torch.tensor([3, 500, 3]), w, cfg)[0], plain.embed(torch.tensor([3]), w, cfg)[0])
    # the factor is on the input side only: the head is the plain product with the table
    x = torch.randn(4, 96, dtype=torch.float64) * 10
    logits = plain.lm_head(x, w, cfg)
    assert logits.shape == (4, 512) and logits.abs().max() < 15.0          # the final cap bounds the logits
    raw = plain.rms_norm(x, w["model.norm.weight"], 1e-5) @ w["model.embed_tokens.weight"].T  # tied: the same table
    torch.testing.assert_close(logits, 15 * torch.tanh(raw / 15))
    cfg_nocap = dict(cfg, final_logit_softcapping=None)
    torch.testing.assert_close(plain.lm_head(x, w, cfg_nocap), raw)


def test_layer_pattern():
    """Even layers are windowed, odd ones see everything (simply/config_lib.py:876-879 ('local', 'global')): with one
    layer a token beyond the window is invisible, with two it is seen, and only through the second layer."""
    cfg = dict(tiny.TINY_A, sliding_window=4)
    far, at = 3, 20
    tokens = tiny.random_tokens(24, cfg["vocab_size"], 6)
    changed = list(tokens)
    changed[far] = (changed[far] + 1) % cfg["vocab_size"]
    w = weights(dict(cfg, num_hidden_layers=2), seed=4)
    one = dict(cfg, num_hidden_layers=1)
    a, b = (plain.forward(w, one, t, torch.float64) for t in (tokens, changed))
    torch.testing.assert_close(a[far + 4:], b[far + 4:], rtol=0, atol=0)     # layer 0 is windowed
    two = dict(cfg, num_hidden_layers=2)
    a, b = (plain.forward(w, two, t, torch.float64) for t in (tokens, changed))
    assert not torch.allclose(a[at], b[at])                                  # layer 1 is not
    # ... and it is layer 1 that sees it: with layer 1's keys and values cut off from the far token's position
    # (its value projection zeroed) the difference is gone again
    both_windowed = dict(two, layer_types=["sliding_attention", "sliding_attention"])
    a, b = (plain.forward(w, both_windowed, t, torch.float64) for t in (tokens, changed))
    torch.testing.assert_close(a[at], b[at], rtol=0, atol=0)
    # an explicit list of layer types wins over the rule
    assert [plain.layer_is_sliding(tiny.TINY_C, i) for i in range(4)] == [False, True, True, False]


def test_untied_head_uses_its_own_table():
    cfg = dict(tiny.TINY_B, tie_word_embeddings=False)
    w = weights(cfg)
    w["lm_head.weight"] = torch.randn(512, 96, generator=torch.Generator().manual_seed(9), dtype=torch.float64)
    x = torch.randn(4, 96, dtype=torch.float64)
    raw = plain.rms_norm(x, w["model.norm.weight"], 1e-5) @ w["lm_head.weight"].T
    torch.testing.assert_close(plain.lm_head(x, w, cfg), 15 * torch.tanh(raw / 15))


# ------------------------------------------------------------------ whole model
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_only_distances_count(name):
    """Shifting all positions changes nothing: rotations and masks depend on distances only."""
    cfg = tiny.CONFIGS[name][0]
    w = weights(cfg, seed=3)
    tokens = tiny.random_tokens(30, cfg["vocab_size"], 5)
    a = plain.forward(w, cfg, tokens, torch.float64)
    b = plain.forward(w, cfg, tokens, torch.float64, first_position=1000)
    torch.testing.assert_close(a, b, rtol=1e-8, atol=1e-8)


def test_causality_and_window_reach():
    cfg = dict(tiny.TINY_A)  # window 8 on layer 0, global layer 1
    w = weights(cfg, seed=4)
    tokens = tiny.random_tokens(24, cfg["vocab_size"], 6)
    a = plain.forward(w, cfg, tokens, torch.float64)
    changed = list(tokens)
    changed[20] = (changed[20] + 1) % cfg["vocab_size"]
    b = plain.forward(w, cfg, changed, torch.float64)
    torch.testing.assert_close(a[:20], b[:20], rtol=0, atol=0)     # the future does not reach back
    assert not torch.allclose(a[20:], b[20:])
    # all layers windowed: a token further back than the layers' reach together is invisible
    cfg_w = dict(cfg, layer_types=["sliding_attention", "sliding_attention"], sliding_window=4)
    changed = list(tokens)
    changed[3] = (changed[3] + 1) % cfg["vocab_size"]
    a = plain.forward(w, cfg_w, tokens, torch.float64)
    b = plain.forward(w, cfg_w, changed, torch.float64)
    reach = 3 + 2 * (4 - 1)                                       # two layers, three keys back each
    assert not torch.allclose(a[reach], b[reach])
    torch.testing.assert_close(a[reach + 1:], b[reach + 1:], rtol=0, atol=0)


def test_greedy_and_sampling_helpers():
    cfg = dict(tiny.TINY_A)
    w = weights(cfg, seed=5)
    out = plain.greedy(w, cfg, [1, 2, 3], 4, torch.float64)
    assert len(out) == 4
    assert out[0] == int(plain.forward(w, cfg, [1, 2, 3], torch.float64)[-1].argmax())
    logits = torch.tensor([2.0, 1.0, 0.5, -1.0])
    assert plain.top_k_mask(logits, 2).tolist() == [True, True, False, False]
    # simply/utils/sampling_lib_test.py: the token that crosses top_p stays
    p = torch.softmax(logits, -1)
    assert plain.top_p_mask(logits, float(p[0]) + 1e-6).tolist() == [True, True, False, False]
    assert plain.top_p_mask(logits, float(p[0]) - 1e-6).tolist() == [True, False, False, False]
    assert abs(plain.log_prob(logits, 1, 0.5) - float(torch.log_softmax(logits.double() / 0.5, -1)[1])) < 1e-12


# ------------------------------------------------------------------ rounding places
def test_rounding_nowhere_changes_nothing_and_everywhere_is_bfloat16_arithmetic():
    cfg = dict(tiny.TINY_B)       # sqrt(96) is no bfloat16 number
    w = {k: v.to(torch.bfloat16).double() for k, v in weights(cfg, seed=6).items()}
    tokens = tiny.random_tokens(20, cfg["vocab_size"], 7)
    exact = plain.forward(w, cfg, tokens, torch.float64)
    assert torch.equal(plain.forward(w, cfg, tokens, torch.float64, rnd=plain.Rounding(torch.bfloat16, ())), exact)
    with pytest.raises(ValueError):
        plain.Rounding(torch.bfloat16, ("nowhere",))
    # every place rounds: each alone moves the logits, by no more than a few bfloat16 steps of the largest logit
    for place in plain.Rounding.PLACES:
        moved = plain.forward(w, cfg, tokens, torch.float64, rnd=plain.Rounding(torch.bfloat16, (place,)))
        err = (moved - exact).abs().max().item() / exact.abs().max().item()
        assert 0 < err < 2e-2, (place, err)
    # the norm's result rounded: the same as rounding by hand
    x = torch.randn(3, 96, dtype=torch.float64)
    scale = w["model.norm.weight"]
    by_hand = plain.rms_norm(x, scale, 1e-5).to(torch.bfloat16).double()
    assert torch.equal(plain.rms_norm(x, scale, 1e-5, plain.Rounding(torch.bfloat16, ("norm_out",))), by_hand)


def test_where_bfloat16_error_enters_a_sharp_model():
    """tiny.drawn_case(11): three global layers of one head of size 128, no soft-cap, weights N(0, 0.32): bfloat16
    logits are 5 to 10 % off, ten times the usual.  Rounding what feeds the scores (norm results, projections,
    rotated queries and keys) does it; rounding behind the softmax (probabilities, attention output, the gated
    product) costs a tenth of that.  With the scores themselves and the residual stream rounded too, as
    google-deepmind/simply does in bfloat16, the error is larger still.  A flat model (drawn_case(0): soft-cap 5) is
    at 0.3 %."""
    def errors(case, n):
        import tempfile

        with tempfile.TemporaryDirectory() as tmp:
            d, _, _ = tiny.write_drawn_case(case, tmp + "/m")
            w, cfg = plain.load(d)
        w = {k: v.to(torch.bfloat16) for k, v in w.items()}
        tokens = tiny.random_tokens(n, cfg["vocab_size"], case * 100)
        exact = plain.forward(w, cfg, tokens, torch.float64)
        err = lambda rnd: ((plain.forward(w, cfg, tokens, torch.float64, rnd=rnd) - exact).abs().max()
                           / exact.abs().max()).item()
        R = lambda *places: plain.Rounding(torch.bfloat16, places)
        return (err(R("norm_out", "proj", "rope")), err(R("probs", "attn_out", "ffn_mid")),
                err(plain.rounding_of_fp32_residual_engine()), err(plain.rounding_like_simply()))

    before, behind, engine, simply = errors(11, 82)
    assert before > 3e-2 and behind < before / 4
    assert engine > 3e-2 and simply > engine
    before, behind, engine, simply = errors(0, 130)
    assert engine < 6e-3 and simply < 1.2e-2
