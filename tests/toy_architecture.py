"""A toy architecture that lives outside the package: its own config.json keys, a block arrangement and a norm of
its own, the package's attention and feed-forward with other constants.  Importing this module registers it; the
package never hears of it otherwise (`SIMPLY_AMD_PLUGINS=toy_architecture` lets a child process import it).  It is
no model of anyone's: pre-norm blocks with a mean-and-variance norm that has a bias, rotary attention without cap or
window, a SiLU-gated feed-forward, an embedding that is not scaled and a head of its own.

`plain_logits` is its plain version in float64, from the plain part functions of `plain_gemma2` where the parts are
the same.
"""
from __future__ import annotations

import dataclasses
import math
from typing import Any, Mapping

import torch

from simply_amd import registry
from simply_amd.config.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry
from simply_amd.parts.base import Block, Norm, ParamSpec, PendingNorm

NAME = "ToyDecoderForTests"


class MeanVarianceNorm(Norm):
    """y = (x - mean) * rsqrt(var + eps) * (1 + gain) + bias, in float32, with torch's own operators."""

    def __init__(self, dim: int, eps: float):
        self.dim, self.eps = int(dim), float(eps)
        self.gain = self.bias = None

    def param_specs(self):
        return {"gain": ParamSpec((self.dim,), role="vector", init="norm"),
                "bias": ParamSpec((self.dim,), role="vector", init="norm")}

    def forward(self, x, out_dtype):
        x = x.float()
        centred = x - x.mean(dim=-1, keepdim=True)
        var = (centred * centred).mean(dim=-1, keepdim=True)
        return (centred * torch.rsqrt(var + self.eps) * (1.0 + self.gain.float()) + self.bias.float()).to(out_dtype)


class PreNormBlock(Block):
    """h += mixer(norm_mixer(h)); h += feed_forward(norm_ffn(h)): no norm behind a part."""

    def first_norm(self):
        return self.norms["mixer"]

    def forward(self, h, ctx, cache, normed, next_norm):
        if isinstance(normed, PendingNorm):  # (a block before this one left its last sum to us)
            normed, h = normed.materialize(), normed.residual
        x = normed if normed is not None else self.norms["mixer"].forward(h, ctx.dtype)
        h.add_(self.mixer.forward(x, ctx, cache).float())
        h.add_(self.feed_forward.forward(self.norms["ffn"].forward(h, ctx.dtype), ctx).float())
        return h, (next_norm.forward(h, ctx.dtype) if next_norm is not None else None)


@dataclasses.dataclass(frozen=True)
class ToyConfig:
    width: int
    depth: int
    heads: int
    kv_heads: int
    head_size: int
    inner: int
    vocab: int
    norm_eps: float = 1e-5
    rope_base: float = 10000.0
    max_positions: int = 512
    architecture: str = NAME

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "ToyConfig":
        missing = [k for k in ("width", "depth", "heads", "kv_heads", "head_size", "inner", "vocab") if k not in d]
        if missing:
            raise ValueError(f"config.json of {NAME}: keys missing: {missing}")
        cfg = cls(**{f.name: d[f.name] for f in dataclasses.fields(cls) if f.name in d and f.name != "architecture"})
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if self.heads % self.kv_heads or self.head_size % 2:
            raise ValueError(f"{NAME}: heads must be a multiple of kv_heads and head_size even")

    def to_dict(self) -> dict[str, Any]:
        d = dataclasses.asdict(self)
        d.pop("architecture")
        return {"architectures": [NAME], **d}

    def model_spec(self) -> ModelSpec:
        D = self.width

        def norm(prefix):
            return PartSpec("toy_mean_variance", {"dim": D, "eps": self.norm_eps},
                            {"gain": prefix + ".gain", "bias": prefix + ".bias"})

        layers = []
        for i in range(self.depth):
            p = f"blk.{i}."
            mixer = PartSpec("paged_attention", {
                "hidden_size": D, "num_heads": self.heads, "num_kv_heads": self.kv_heads, "head_dim": self.head_size,
                "query_scale": math.sqrt(self.head_size), "soft_cap": None, "window": None,
                "position_encoding": PartSpec("rope", {"head_dim": self.head_size, "base": self.rope_base,
                                                       "scale_factor": 1.0})},
                {n: p + n[0] for n in ("q_proj", "k_proj", "v_proj", "o_proj")})
            ffn = PartSpec("gated_dense", {"hidden_size": D, "intermediate_size": self.inner, "activation": "silu"},
                           {"gate_proj": p + "gate", "up_proj": p + "up", "down_proj": p + "down"})
            layers.append(LayerSpec(PartSpec("toy_pre_norm"), mixer, ffn, {"mixer": norm(p + "n1"), "ffn": norm(p + "n2")}))
        spec = ModelSpec(
            architecture=NAME, hidden_size=D, vocab_size=self.vocab,
            embedding=PartSpec("scaled_embedding", {"vocab_size": self.vocab, "dim": D, "scale": 1.0}, {"table": "tok"}),
            layers=tuple(layers), schedule=tuple(ScheduleEntry(i) for i in range(self.depth)),
            final_norm=norm("last"),
            head=PartSpec("linear_head", {"vocab_size": self.vocab, "dim": D, "soft_cap": None}, {"weight": "out"}),
            max_position=self.max_positions, initializer_range=0.08)
        spec.validate()
        return spec


def register() -> None:
    registry.NORMS.register("toy_mean_variance", MeanVarianceNorm, overwrite=True)
    registry.BLOCKS.register("toy_pre_norm", PreNormBlock, overwrite=True)
    registry.ARCHITECTURES.register(NAME, ToyConfig, overwrite=True)


def unregister() -> None:
    registry.NORMS.unregister("toy_mean_variance")
    registry.BLOCKS.unregister("toy_pre_norm")
    registry.ARCHITECTURES.unregister(NAME)


register()


# ------------------------------------------------------------------------------------------ the plain version
def plain_logits(w: Mapping[str, torch.Tensor], cfg: ToyConfig, tokens) -> torch.Tensor:
    """Logits [T, vocab] in float64 for a whole sequence, no cache."""
    import plain_gemma2 as plain

    w = {k: v.double() for k, v in w.items()}
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    T = tokens.shape[0]
    positions = torch.arange(T)

    def norm(x, prefix):
        centred = x - x.mean(dim=-1, keepdim=True)
        var = (centred * centred).mean(dim=-1, keepdim=True)
        return centred * torch.rsqrt(var + cfg.norm_eps) * (1.0 + w[prefix + ".gain"]) + w[prefix + ".bias"]

    h = w["tok"][tokens]
    H, K, hd = cfg.heads, cfg.kv_heads, cfg.head_size
    mask = plain.attention_mask(positions, positions, None)
    for i in range(cfg.depth):
        p = f"blk.{i}."
        x = norm(h, p + "n1")
        q = plain.rope((x @ w[p + "q"].T).reshape(T, H, hd), positions, cfg.rope_base) / math.sqrt(hd)
        k = plain.rope((x @ w[p + "k"].T).reshape(T, K, hd), positions, cfg.rope_base)
        v = (x @ w[p + "v"].T).reshape(T, K, hd)
        h = h + plain.attention(q, k, v, mask, None).reshape(T, H * hd) @ w[p + "o"].T
        x = norm(h, p + "n2")
        h = h + (torch.nn.functional.silu(x @ w[p + "gate"].T) * (x @ w[p + "up"].T)) @ w[p + "down"].T
    return norm(h, "last") @ w["out"].T
