"""Grouped-query attention over a paged cache.

simply/model_lib.py:1605 (Attention): q/k/v projections, position encoding on q and k,
q / query_scale (:1987-2020), attention over the cache with soft-cap and window
(simply/utils/ragged_paged_attention.py:870-949), output projection (:2362).
"""
from __future__ import annotations

import functools

import torch

from ..config.spec import PartSpec
from ..kernels import ops
from ..registry import MIXERS, POSITION_ENCODINGS
from .base import Mixer, PagedKVNeed, ParamSpec, as_product_weight, pending_fits_product, pending_product, project


@MIXERS.register("paged_attention")
class PagedAttention(Mixer):
    accepts_pending = True
    defers_sum = True

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, query_scale: float,
                 soft_cap: float | None = None, window: int | None = None,
                 position_encoding: PartSpec | None = None):
        if num_heads % num_kv_heads:
            raise ValueError(f"paged_attention: {num_heads} heads do not split over {num_kv_heads} kv heads")
        self.hidden_size, self.num_heads, self.num_kv_heads, self.head_dim = hidden_size, num_heads, num_kv_heads, head_dim
        self.query_scale = float(query_scale)
        self.soft_cap = float(soft_cap) if soft_cap else None
        self.window = int(window) if window else None
        self.position_encoding = (POSITION_ENCODINGS.build(position_encoding.kind, **position_encoding.params)
                                  if position_encoding is not None else None)
        self.qkv_proj: torch.Tensor | None = None
        self.o_proj: torch.Tensor | None = None

    def param_specs(self):
        D, H, K, hd = self.hidden_size, self.num_heads, self.num_kv_heads, self.head_dim
        return {"q_proj": ParamSpec((H * hd, D)), "k_proj": ParamSpec((K * hd, D)),
                "v_proj": ParamSpec((K * hd, D)), "o_proj": ParamSpec((D, H * hd))}

    def load(self, tensors):
        # one product for q, k and v: rows [q heads | k heads | v heads]
        device = tensors["o_proj"].device
        self.qkv_proj = as_product_weight(torch.cat([tensors["q_proj"], tensors["k_proj"], tensors["v_proj"]], dim=0)
                                          .contiguous())
        self.o_proj = as_product_weight(tensors["o_proj"])
        if self.position_encoding is not None and hasattr(self.position_encoding, "to_device"):
            self.position_encoding.to_device(device)

    def cache_need(self):
        return PagedKVNeed(self.num_kv_heads, self.head_dim, self.window)

    def forward(self, x, ctx, cache, defer_sum=False):
        H, K, hd = self.num_heads, self.num_kv_heads, self.head_dim
        group = ctx.groups[cache.group_id]
        pe = self.position_encoding
        rotary = pe.rotary_table() if pe is not None else None
        write = cache.write
        pages = dict(slot_mapping=group.slot_mapping if write else None, k_pages=cache.k_pages if write else None,
                     v_pages=cache.v_pages if write else None)
        if (pe is None or rotary is not None) and hd % 32 == 0 and pending_fits_product(x, self.qkv_proj) \
                and cache.k_pages.dtype == torch.bfloat16:
            # a few tokens: the norms in front of the projection and the rotation, query scale and cache write
            # behind it run in the projection's kernel
            table, sf = rotary if rotary is not None else (None, 1.0)
            qkv = pending_product(x, functools.partial(
                ops.gemm_normed_rotary, w=self.qkv_proj, positions=ctx.positions, timescale=table, scale_factor=sf,
                query_scale=self.query_scale, num_heads=H, num_kv_heads=K, head_dim=hd, **pages))
        else:
            if pe is None or rotary is not None:
                # (the kernel behind the projection adds up its cuts of K, if it has any, on the way)
                table, sf = rotary if rotary is not None else (None, 1.0)
                qkv = ops.rope_cache_write(project(x, self.qkv_proj, defer_sum=True), ctx.positions, table, sf,
                                           self.query_scale, H, K, hd, **pages)
            else:
                qkv = project(x, self.qkv_proj)
                # another position encoding: applied by the part itself, then the plain scale-and-write kernel
                pe.apply(qkv, ctx.positions, H, hd, 1.0)
                pe.apply(qkv[:, H * hd:], ctx.positions, K, hd, 1.0)
                ops.rope_cache_write(qkv, ctx.positions, None, 1.0, self.query_scale, H, K, hd, **pages)
        o = torch.empty((qkv.shape[0], H * hd), dtype=qkv.dtype, device=qkv.device)
        if ops.decode_attention_takes(qkv, cache.k_pages, H, 1):
            # the MFMA kernels take up to 16 query rows (tokens x heads per key head) as a unit: a decoding request
            # is one unit and its keys are cut over workgroups; portions of prompts are cut into units of 16 / G
            # tokens, of which one workgroup takes four
            units, few, many, max_q = ctx.attention_units(16 // (H // K), ops.prefill_units_per_group())
            kw = dict(window=self.window, soft_cap=self.soft_cap, max_kv_len=ctx.max_kv_len, max_q_len=max_q, out=o)
            if few:
                ops.paged_attention_decode(qkv, cache.k_pages, cache.v_pages, group.block_table, units, 0, few, H, **kw)
            if many:
                ops.paged_attention_prefill(qkv, cache.k_pages, cache.v_pages, group.block_table, units, few, many, H,
                                            **kw)
        else:
            ops.paged_attention(qkv, cache.k_pages, cache.v_pages, group.block_table, ctx.token_seq, ctx.positions, H,
                                window=self.window, soft_cap=self.soft_cap, out=o)
        return ops.gemm(o, self.o_proj, defer_sum=defer_sum)
