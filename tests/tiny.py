"""Two tiny Gemma 2 configurations that differ in every size and option, and helpers that write them
as model folders with random weights (in a temporary folder, never committed)."""
from __future__ import annotations

import json
import os

import torch

TINY_A = dict(
    architectures=["Gemma2ForCausalLM"], hidden_size=64, num_hidden_layers=2, num_attention_heads=4,
    num_key_value_heads=2, head_dim=16, intermediate_size=128, vocab_size=256, rms_norm_eps=1e-6,
    rope_theta=10000.0, sliding_window=8, query_pre_attn_scalar=16, attn_logit_softcapping=50.0,
    final_logit_softcapping=30.0, tie_word_embeddings=True, max_position_embeddings=512,
    hidden_activation="gelu_pytorch_tanh", initializer_range=0.02,
)
TINY_B = dict(
    architectures=["Gemma2ForCausalLM"], hidden_size=96, num_hidden_layers=3, num_attention_heads=6,
    num_key_value_heads=1, head_dim=32, intermediate_size=320, vocab_size=512, rms_norm_eps=1e-5,
    rope_theta=1000000.0, sliding_window=16, query_pre_attn_scalar=24, attn_logit_softcapping=None,
    final_logit_softcapping=15.0, tie_word_embeddings=True, max_position_embeddings=512,
    hidden_activation="gelu_pytorch_tanh", initializer_range=0.05,
)
# a third one with sizes that are no power of two anywhere and a vocabulary that is no multiple of 64
TINY_C = dict(
    architectures=["Gemma2ForCausalLM"], hidden_size=120, num_hidden_layers=4, num_attention_heads=6,
    num_key_value_heads=3, head_dim=48, intermediate_size=200, vocab_size=333, rms_norm_eps=1e-6,
    rope_theta=5000.0, sliding_window=5, query_pre_attn_scalar=30, attn_logit_softcapping=20.0,
    final_logit_softcapping=None, tie_word_embeddings=True, max_position_embeddings=512,
    layer_types=["full_attention", "sliding_attention", "sliding_attention", "full_attention"],
    hidden_activation="gelu_pytorch_tanh", initializer_range=0.08,
)
# sizes that the bfloat16 MFMA kernels take (head size 64, pages of 16), still tiny
TINY_D = dict(
    architectures=["Gemma2ForCausalLM"], hidden_size=128, num_hidden_layers=3, num_attention_heads=4,
    num_key_value_heads=2, head_dim=64, intermediate_size=256, vocab_size=1000, rms_norm_eps=1e-6,
    rope_theta=10000.0, sliding_window=40, query_pre_attn_scalar=64, attn_logit_softcapping=50.0,
    final_logit_softcapping=30.0, tie_word_embeddings=True, max_position_embeddings=1024,
    hidden_activation="gelu_pytorch_tanh", initializer_range=0.05,
)
# the first one with a head of its own (a random head gives continuations that do not repeat one token)
TINY_U = dict(TINY_A, tie_word_embeddings=False)
CONFIGS = {"A": (TINY_A, 0, 0.1), "B": (TINY_B, 1, 0.2), "C": (TINY_C, 2, 0.3), "D": (TINY_D, 3, 0.1),
           "U": (TINY_U, 4, 0.1)}


def write_model(name: str, out_dir: str, dtype=torch.float32, std: float | None = None) -> str:
    """Writes configuration `name` with random weights through the framework's random-weights mode."""
    from simply_amd.config import config_from_dict
    from simply_amd.weights import write_random_model

    d, seed, norm_std = CONFIGS[name]
    cfg = config_from_dict(d)
    return write_random_model(cfg, out_dir, seed, dtype, std=std, norm_std=norm_std)


def write_config_model(d: dict, out_dir: str, seed: int, dtype=torch.float32, std: float | None = None,
                       norm_std: float = 0.2) -> str:
    """Writes the configuration `d` (config.json keys) with random weights."""
    from simply_amd.config import config_from_dict
    from simply_amd.weights import write_random_model

    return write_random_model(config_from_dict(d), out_dir, seed, dtype, std=std, norm_std=norm_std)


def odd_head_size_config(head_dim: int) -> dict:
    """A tiny configuration whose head size is even but no multiple of 16 (rotary pairs need no more:
    simply/utils/position_encoding.py:83-84 splits the head in halves)."""
    return dict(TINY_C, head_dim=head_dim, query_pre_attn_scalar=head_dim, num_hidden_layers=3,
                layer_types=["sliding_attention", "full_attention", "sliding_attention"], sliding_window=9)


def random_tokens(n: int, vocab: int, seed: int) -> list[int]:
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def random_config(seed: int) -> dict:
    """A tiny configuration drawn at random: head counts and groups, head sizes in steps of 16 up to 256, widths
    that are no multiple of 8, layer kinds in any order, caps present or not."""
    import numpy as np

    rng = np.random.default_rng(seed)
    kv, group = int(rng.choice([1, 2, 3, 4])), int(rng.choice([1, 2, 3, 4, 8]))
    hd = int(rng.choice([16, 32, 48, 64, 80, 96, 128, 256]))
    if hd >= 128:
        kv, group = min(kv, 2), min(group, 2)
    layers = int(rng.integers(1, 5))
    return dict(
        architectures=["Gemma2ForCausalLM"], hidden_size=int(rng.choice([64, 96, 120, 128, 136, 200, 100, 264])),
        num_hidden_layers=layers, num_attention_heads=kv * group, num_key_value_heads=kv, head_dim=hd,
        intermediate_size=int(rng.choice([128, 200, 320, 264, 72, 500])),
        vocab_size=int(rng.choice([256, 333, 512, 1000, 1001, 4099])), rms_norm_eps=float(rng.choice([1e-6, 1e-5])),
        rope_theta=float(rng.choice([10000.0, 1e6, 500.0])), sliding_window=int(rng.integers(3, 60)),
        query_pre_attn_scalar=int(rng.choice([hd, 24, 144])),
        attn_logit_softcapping=None if rng.random() < 0.3 else float(rng.choice([50.0, 20.0, 5.0])),
        final_logit_softcapping=None if rng.random() < 0.3 else float(rng.choice([30.0, 15.0])),
        tie_word_embeddings=True, max_position_embeddings=1024,
        layer_types=[str(rng.choice(["full_attention", "sliding_attention"])) for _ in range(layers)],
        hidden_activation="gelu_pytorch_tanh", initializer_range=0.05)


def write_random_config_model(seed: int, out_dir: str) -> str:
    from simply_amd.config import config_from_dict
    from simply_amd.weights import write_random_model

    d = random_config(seed)
    std = 0.15 * (64.0 / d["hidden_size"]) ** 0.5
    return write_random_model(config_from_dict(d), out_dir, seed, torch.float32, std=std, norm_std=0.2)


def drawn_case(case: int) -> tuple[dict, int, float, list[int]]:
    """Another family of configurations drawn at random, with larger weights: (config, page size, std of the
    weights, lengths of the requests).  Cases 4, 11, 21, 36, 94 and 135 are the ones whose bfloat16 logits lie
    furthest from the float64 ones (4 to 8 % of the largest logit: sharp softmaxes without a soft-cap, or four
    layers of head size 256 over a width of 136)."""
    import numpy as np

    rng = np.random.default_rng(case)
    kv, group = int(rng.choice([1, 2, 3, 4])), int(rng.choice([1, 2, 3, 4, 8]))
    hd = int(rng.choice([16, 32, 48, 64, 80, 96, 128, 256]))
    if hd >= 128:
        kv, group = min(kv, 2), min(group, 2)
    hidden = int(rng.choice([64, 96, 120, 128, 136, 200, 100, 264]))
    inter = int(rng.choice([128, 200, 320, 264, 72, 500]))
    layers = int(rng.integers(1, 5))
    vocab = int(rng.choice([256, 333, 512, 1000, 1001, 4099]))
    window = int(rng.integers(3, 60))
    types = [str(rng.choice(["full_attention", "sliding_attention"])) for _ in range(layers)]
    d = dict(
        architectures=["Gemma2ForCausalLM"], hidden_size=hidden, num_hidden_layers=layers,
        num_attention_heads=kv * group, num_key_value_heads=kv, head_dim=hd, intermediate_size=inter, vocab_size=vocab,
        rms_norm_eps=float(rng.choice([1e-6, 1e-5])), rope_theta=float(rng.choice([10000.0, 1e6, 500.0])),
        sliding_window=window, query_pre_attn_scalar=int(rng.choice([hd, 24, 144])),
        attn_logit_softcapping=None if rng.random() < 0.3 else float(rng.choice([50.0, 20.0, 5.0])),
        final_logit_softcapping=None if rng.random() < 0.3 else float(rng.choice([30.0, 15.0])),
        tie_word_embeddings=True, max_position_embeddings=1024, layer_types=types,
        hidden_activation="gelu_pytorch_tanh", initializer_range=0.05)
    page = int(rng.choice([4, 8, 16, 16, 32]))
    std = float(rng.choice([0.1, 0.2, 0.3])) * (64.0 / hidden) ** 0.5 * 1.5
    lens = [int(rng.integers(2, 160)) for _ in range(int(rng.integers(3, 7)))]
    return d, page, std, lens


# the smallest sizes anything takes, a window of one key: its bfloat16 logits were 8.7 % off on a 130-token request
SMALLEST = dict(
    architectures=["Gemma2ForCausalLM"], hidden_size=8, num_hidden_layers=3, num_attention_heads=1,
    num_key_value_heads=1, head_dim=16, intermediate_size=24, vocab_size=17, rms_norm_eps=1e-6, rope_theta=10000.0,
    sliding_window=1, query_pre_attn_scalar=16, attn_logit_softcapping=50.0, final_logit_softcapping=30.0,
    tie_word_embeddings=True, max_position_embeddings=1024,
    layer_types=["full_attention", "sliding_attention", "full_attention"], hidden_activation="gelu_pytorch_tanh",
    initializer_range=0.05)


def write_drawn_case(case, out_dir: str) -> tuple[str, int, list[int]]:
    """Writes `drawn_case(case)` (or, for case "smallest", SMALLEST) as a model folder; returns (folder, page size,
    request lengths)."""
    from simply_amd.config import config_from_dict
    from simply_amd.weights import write_random_model

    if case == "smallest":
        d, page, std, lens, seed = SMALLEST, 4, 0.3 * (64.0 / 8) ** 0.5 * 1.5, [19, 49, 67, 130], 2
    else:
        d, page, std, lens = drawn_case(case)
        seed = case
    return write_random_model(config_from_dict(d), out_dir, seed, torch.float32, std=std, norm_std=0.2), page, lens
