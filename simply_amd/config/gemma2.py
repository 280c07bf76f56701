"""Typed configuration of Gemma 2, read from the model folder's `config.json`.

The reference keeps these numbers in Python factories
(simply/config_lib.py:852-957: gemma2_2b, gemma2_9b, gemma2_27b over
BaseExperimentConfig simply/config_lib.py:241-343); the keys below are those of
the model folder, and the comments give the reference's field for each.
"""
from __future__ import annotations

import dataclasses
import math
from typing import Any, Mapping

from ..registry import ARCHITECTURES
from .spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

SLIDING = "sliding_attention"
FULL = "full_attention"
_TANH_GELU_NAMES = ("gelu_pytorch_tanh", "gelu_tanh", "gelu_new")


class ConfigError(ValueError):
    pass


def _need(d: Mapping[str, Any], key: str, typ):
    if key not in d or d[key] is None:
        raise ConfigError(f"config.json: required key {key!r} is missing")
    v = d[key]
    if typ is int and (isinstance(v, bool) or not isinstance(v, int)):
        raise ConfigError(f"config.json: {key!r} must be an integer, got {v!r}")
    return v


def _opt_cap(d: Mapping[str, Any], key: str, default: float) -> float | None:
    """A soft-cap: absent -> the architecture's default; null or <= 0 -> off
    (simply/model_lib.py:626 and :3187 apply a cap only when it is > 0)."""
    if key not in d:
        return default
    v = d[key]
    if v is None:
        return None
    v = float(v)
    return v if v > 0 else None


@dataclasses.dataclass(frozen=True)
class Gemma2Config:
    hidden_size: int                 # model_dim
    num_hidden_layers: int           # n_layers
    num_attention_heads: int         # n_heads
    num_key_value_heads: int         # n_kv_heads
    head_dim: int                    # per_head_dim
    intermediate_size: int           # ffn_expand_dim (expand_factor * model_dim)
    vocab_size: int
    rms_norm_eps: float              # rms_norm_epsilon
    rope_theta: float                # RoPE.max_timescale
    query_pre_attn_scalar: float     # query_scale ** 2
    sliding_window: int | None       # window_size + 1: keys a query sees, itself included
    attn_logit_softcapping: float | None   # attn_soft_cap
    final_logit_softcapping: float | None  # output_logits_soft_cap
    tie_word_embeddings: bool        # use_tied_embedding
    max_position_embeddings: int
    layer_types: tuple[str, ...]     # block_attn_pattern, spelled out per layer
    eos_token_ids: tuple[int, ...]
    bos_token_id: int | None
    pad_token_id: int | None
    initializer_range: float
    torch_dtype: str

    architecture = "Gemma2ForCausalLM"

    # ------------------------------------------------------------------ reading
    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "Gemma2Config":
        n_layers = _need(d, "num_hidden_layers", int)
        head_dim = _need(d, "head_dim", int)
        sliding_window = d.get("sliding_window", 4096)  # simply/config_lib.py:874: window_size 4095
        if sliding_window is not None:
            sliding_window = int(sliding_window)
        layer_types = d.get("layer_types")
        if layer_types is None:
            # simply/config_lib.py:876-879 with simply/model_lib.py:2839-2844:
            # pattern ('local', 'global') cycles, so even layers are windowed.
            layer_types = [SLIDING if i % 2 == 0 else FULL for i in range(n_layers)]
        if sliding_window is None:
            layer_types = [FULL] * n_layers
        act = d.get("hidden_activation", d.get("hidden_act", _TANH_GELU_NAMES[0]))
        if act not in _TANH_GELU_NAMES:
            raise ConfigError(
                f"config.json: hidden_activation {act!r} is not the tanh-approximate gelu "
                f"that Gemma 2 uses (simply/model_lib.py:94-96); accepted: {_TANH_GELU_NAMES}")
        if d.get("attention_bias"):
            raise ConfigError("config.json: attention_bias is set, Gemma 2 has no biases (simply/config_lib.py:881-882)")
        if d.get("rope_scaling"):
            raise ConfigError("config.json: rope_scaling is not supported for Gemma 2 (RoPE scale_factor is 1.0)")
        eos = d.get("eos_token_id")
        if eos is None:
            eos_ids: tuple[int, ...] = ()
        elif isinstance(eos, (list, tuple)):
            eos_ids = tuple(int(e) for e in eos)
        else:
            eos_ids = (int(eos),)
        cfg = cls(
            hidden_size=_need(d, "hidden_size", int),
            num_hidden_layers=n_layers,
            num_attention_heads=_need(d, "num_attention_heads", int),
            num_key_value_heads=_need(d, "num_key_value_heads", int),
            head_dim=head_dim,
            intermediate_size=_need(d, "intermediate_size", int),
            vocab_size=_need(d, "vocab_size", int),
            rms_norm_eps=float(d.get("rms_norm_eps", 1e-6)),   # simply/config_lib.py:300
            rope_theta=float(d.get("rope_theta", 10000.0)),    # simply/utils/position_encoding.py:65
            query_pre_attn_scalar=float(d.get("query_pre_attn_scalar", head_dim)),  # simply/model_lib.py:2017-2019
            sliding_window=sliding_window,
            attn_logit_softcapping=_opt_cap(d, "attn_logit_softcapping", 50.0),    # simply/config_lib.py:297
            final_logit_softcapping=_opt_cap(d, "final_logit_softcapping", 30.0),  # simply/config_lib.py:299
            tie_word_embeddings=bool(d.get("tie_word_embeddings", True)),
            max_position_embeddings=int(d.get("max_position_embeddings", 8192)),
            layer_types=tuple(layer_types),
            eos_token_ids=eos_ids,
            bos_token_id=d.get("bos_token_id"),
            pad_token_id=d.get("pad_token_id"),
            initializer_range=float(d.get("initializer_range", 0.02)),
            torch_dtype=str(d.get("torch_dtype", d.get("dtype", "bfloat16"))),
        )
        cfg.validate()
        return cfg

    def validate(self) -> None:
        for name in ("hidden_size", "num_hidden_layers", "num_attention_heads", "num_key_value_heads",
                     "head_dim", "intermediate_size", "vocab_size", "max_position_embeddings"):
            if getattr(self, name) <= 0:
                raise ConfigError(f"config.json: {name} must be positive, got {getattr(self, name)}")
        # simply/model_lib.py:2032-2036: query heads must split evenly over kv heads.
        if self.num_attention_heads % self.num_key_value_heads != 0:
            raise ConfigError(
                f"config.json: num_attention_heads {self.num_attention_heads} is not a multiple of "
                f"num_key_value_heads {self.num_key_value_heads}")
        if self.head_dim % 2 != 0:
            raise ConfigError(f"config.json: head_dim {self.head_dim} must be even for rotary pairs")
        if len(self.layer_types) != self.num_hidden_layers:
            raise ConfigError(
                f"config.json: layer_types has {len(self.layer_types)} entries for {self.num_hidden_layers} layers")
        for t in self.layer_types:
            if t not in (SLIDING, FULL):
                raise ConfigError(f"config.json: unknown layer type {t!r}; known: {SLIDING}, {FULL}")
        if SLIDING in self.layer_types and (self.sliding_window is None or self.sliding_window < 1):
            raise ConfigError("config.json: sliding layers need sliding_window >= 1")
        if self.query_pre_attn_scalar <= 0 or self.rms_norm_eps <= 0 or self.rope_theta <= 0:
            raise ConfigError("config.json: query_pre_attn_scalar, rms_norm_eps and rope_theta must be positive")

    def to_dict(self) -> dict[str, Any]:
        """The config.json that `from_dict` reads back to the same configuration."""
        d: dict[str, Any] = {"architectures": [self.architecture], "model_type": "gemma2"}
        for f in dataclasses.fields(self):
            v = getattr(self, f.name)
            if f.name == "eos_token_ids":
                d["eos_token_id"] = list(v) if len(v) != 1 else v[0]
            elif f.name == "layer_types":
                d[f.name] = list(v)
            else:
                d[f.name] = v
        d["hidden_activation"] = _TANH_GELU_NAMES[0]
        return d

    # ------------------------------------------------------------------ model spec
    def model_spec(self) -> ModelSpec:
        """The parts of Gemma 2 (simply/model_lib.py:2427 TransformerBlock, :1605 Attention,
        :643 FeedForward, :114 LayerNorm) as data."""
        D, H, K, hd = self.hidden_size, self.num_attention_heads, self.num_key_value_heads, self.head_dim

        def norm(name: str) -> PartSpec:
            # simply/config_lib.py:863 use_rmsnorm, :296 norm_scale_plus_one
            return PartSpec("rmsnorm", {"dim": D, "eps": self.rms_norm_eps, "scale_plus_one": True},
                            {"scale": name})

        layers = []
        for i, kind in enumerate(self.layer_types):
            p = f"model.layers.{i}."
            mixer = PartSpec(
                "paged_attention",
                {
                    "hidden_size": D, "num_heads": H, "num_kv_heads": K, "head_dim": hd,
                    # q / query_scale after RoPE (simply/model_lib.py:2014-2019)
                    "query_scale": math.sqrt(self.query_pre_attn_scalar),
                    "soft_cap": self.attn_logit_softcapping,
                    "window": self.sliding_window if kind == SLIDING else None,
                    "position_encoding": PartSpec("rope", {"head_dim": hd, "base": self.rope_theta,
                                                           "scale_factor": 1.0}),
                },
                {"q_proj": p + "self_attn.q_proj.weight", "k_proj": p + "self_attn.k_proj.weight",
                 "v_proj": p + "self_attn.v_proj.weight", "o_proj": p + "self_attn.o_proj.weight"},
            )
            ffn = PartSpec(
                "gated_dense",
                {"hidden_size": D, "intermediate_size": self.intermediate_size, "activation": "gelu_tanh"},
                {"gate_proj": p + "mlp.gate_proj.weight", "up_proj": p + "mlp.up_proj.weight",
                 "down_proj": p + "mlp.down_proj.weight"},
            )
            layers.append(LayerSpec(
                block=PartSpec("sandwich"),  # pre-norm, part, post-norm, then the residual (model_lib.py:2669-2703)
                mixer=mixer,
                feed_forward=ffn,
                norms={
                    "pre_mixer": norm(p + "input_layernorm.weight"),            # pre_ln_0
                    "post_mixer": norm(p + "post_attention_layernorm.weight"),  # post_ln_0
                    "pre_ffn": norm(p + "pre_feedforward_layernorm.weight"),    # pre_ln_1
                    "post_ffn": norm(p + "post_feedforward_layernorm.weight"),  # post_ln_1
                },
            ))
        head_tensor = "model.embed_tokens.weight" if self.tie_word_embeddings else "lm_head.weight"
        spec = ModelSpec(
            architecture=self.architecture,
            hidden_size=D,
            vocab_size=self.vocab_size,
            # simply/utils/module.py:472-481: lookup times sqrt(dim)
            embedding=PartSpec("scaled_embedding", {"vocab_size": self.vocab_size, "dim": D, "scale": math.sqrt(D)},
                               {"table": "model.embed_tokens.weight"}),
            layers=tuple(layers),
            schedule=tuple(ScheduleEntry(i) for i in range(self.num_hidden_layers)),
            final_norm=norm("model.norm.weight"),
            head=PartSpec("linear_head", {"vocab_size": self.vocab_size, "dim": D,
                                          "soft_cap": self.final_logit_softcapping},
                          {"weight": head_tensor}),
            max_position=self.max_position_embeddings,
            eos_token_ids=self.eos_token_ids,
            initializer_range=self.initializer_range,
            # a folder of a tied model may store the head once more under its own name
            copies={"lm_head.weight": "model.embed_tokens.weight"} if self.tie_word_embeddings else {},
        )
        spec.validate()
        return spec


ARCHITECTURES.register("Gemma2ForCausalLM", Gemma2Config)
