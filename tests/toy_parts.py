"""Toy parts that tests register to show what the framework takes without a change to its files.  They are
made for the tests and are nobody's model."""
from __future__ import annotations

import dataclasses

import torch

from simply_amd.config import LayerSpec, ModelSpec, PartSpec, ScheduleEntry
from simply_amd.parts.base import Mixer, ParamSpec


@dataclasses.dataclass(frozen=True)
class LatentNeed:
    """One latent vector per token, in pages of a layout of its own: [page, rank, page_size] float32, whatever the
    activation dtype is.  It is no subclass of anything in the framework: the cache manager takes any need that
    says `page_tensors`, `bytes_per_token` and `window`."""

    rank: int
    window: int | None = None

    def page_tensors(self, num_pages, page_size, dtype, device, fill):
        return {"latent": torch.full((num_pages, self.rank, page_size), fill, dtype=torch.float32, device=device)}

    def bytes_per_token(self, esize):
        return 4 * self.rank


class LatentMeanMixer(Mixer):
    """y_t = W_out . mean over the last `window` tokens s <= t of (W_in x_s): a mixer that pages something other than
    keys and values.  Written with torch on whatever device the step runs on."""

    def __init__(self, hidden_size: int, rank: int, window: int | None = None):
        self.hidden_size, self.rank, self.window = hidden_size, rank, window
        self.w_in = self.w_out = None

    def param_specs(self):
        return {"w_in": ParamSpec((self.rank, self.hidden_size)), "w_out": ParamSpec((self.hidden_size, self.rank))}

    def cache_need(self):
        return LatentNeed(self.rank, self.window)

    def forward(self, x, ctx, cache):
        group = ctx.groups[cache.group_id]
        pages = cache.pages["latent"]
        P = pages.shape[2]
        lat = x.float() @ self.w_in.float().T
        if cache.write:
            slots = group.slot_mapping
            pages[slots // P, :, slots % P] = lat
        out = torch.empty((x.shape[0], self.rank), dtype=torch.float32, device=x.device)
        for slot, a, b, start in zip(ctx.seq_slots, ctx.cu_q_lens[:-1], ctx.cu_q_lens[1:], ctx.seq_starts):
            n = start + b - a
            blocks = group.block_table[slot, :-(-n // P)].long().clamp(min=0)   # (holes are never read: below the window)
            keys = pages[blocks].permute(0, 2, 1).reshape(-1, self.rank)        # [blocks * P, rank] by position
            for t in range(a, b):
                pos = start + t - a
                lo = max(0, pos - self.window + 1) if self.window else 0
                out[t] = keys[lo:pos + 1].mean(dim=0)
        return (out @ self.w_out.float().T).to(x.dtype)


def latent_mean_reference(x: torch.Tensor, w_in: torch.Tensor, w_out: torch.Tensor, window: int | None) -> torch.Tensor:
    """The same mixer over a whole sequence x [T, D], no cache."""
    lat = x.double() @ w_in.double().T
    rows = []
    for t in range(x.shape[0]):
        lo = max(0, t - window + 1) if window else 0
        rows.append(lat[lo:t + 1].mean(dim=0))
    return torch.stack(rows) @ w_out.double().T


def latent_model_spec(D: int = 64, V: int = 128, window: int = 6) -> ModelSpec:
    """Three layers: the built-in attention (window 7), the toy mixer with pages of its own over a window, and the
    toy mixer over everything: three cache groups, two of them with a page layout that the framework has never seen."""
    norm = lambda name: PartSpec("rmsnorm", {"dim": D, "eps": 1e-6}, {"scale": name})
    norms = lambda p: {"pre_mixer": norm(p + "n0"), "post_mixer": norm(p + "n1"), "pre_ffn": norm(p + "n2"),
                       "post_ffn": norm(p + "n3")}
    dense = lambda p: PartSpec("gated_dense", {"hidden_size": D, "intermediate_size": 96},
                               {n: p + n for n in ("gate_proj", "up_proj", "down_proj")})
    attn = PartSpec("paged_attention", {"hidden_size": D, "num_heads": 4, "num_kv_heads": 2, "head_dim": 16,
                                        "query_scale": 4.0, "soft_cap": None, "window": 7,
                                        "position_encoding": PartSpec("rope", {"head_dim": 16, "base": 10000.0})},
                    {n: "l0." + n for n in ("q_proj", "k_proj", "v_proj", "o_proj")})
    latent = lambda p, w: PartSpec("toy_latent_mean", {"hidden_size": D, "rank": 12, "window": w},
                                   {"w_in": p + "w_in", "w_out": p + "w_out"})
    layers = (LayerSpec(PartSpec("sandwich"), attn, dense("l0."), norms("l0.")),
              LayerSpec(PartSpec("sandwich"), latent("l1.", window), dense("l1."), norms("l1.")),
              LayerSpec(PartSpec("sandwich"), latent("l2.", None), dense("l2."), norms("l2.")))
    return ModelSpec("ToyLatentModel", D, V,
                     PartSpec("scaled_embedding", {"vocab_size": V, "dim": D, "scale": 8.0}, {"table": "emb"}),
                     layers, tuple(ScheduleEntry(i) for i in range(3)), norm("final"),
                     PartSpec("linear_head", {"vocab_size": V, "dim": D, "soft_cap": None}, {"weight": "emb"}),
                     max_position=256)
