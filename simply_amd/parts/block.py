"""Block arrangements.

'sandwich' is the block of simply/model_lib.py:2659-2708 with use_pre_ln and use_post_ln:
  h += post_mixer(mixer(pre_mixer(h)));  h += post_ffn(ffn(pre_ffn(h)))
The residual stream h is float32; each residual sum is fused with the norm before it and the
norm after it where those are RMSNorms.
"""
from __future__ import annotations

from ..registry import BLOCKS
from .base import Block


@BLOCKS.register("sandwich")
class SandwichBlock(Block):
    NORM_NAMES = ("pre_mixer", "post_mixer", "pre_ffn", "post_ffn")

    def __init__(self, mixer, feed_forward, norms):
        super().__init__(mixer, feed_forward, norms)
        missing = [n for n in self.NORM_NAMES if n not in self.norms]
        if missing:
            raise ValueError(f"sandwich block: norms missing: {missing}")

    def first_norm(self):
        return self.norms["pre_mixer"]

    def forward(self, h, ctx, cache, normed, next_norm):
        n = self.norms
        if normed is None:
            normed = n["pre_mixer"].forward(h, ctx.dtype)
        y = self.mixer.forward(normed, ctx, cache)
        normed = n["post_mixer"].add_into(h, y, n["pre_ffn"], ctx.dtype)
        y = self.feed_forward.forward(normed, ctx)
        normed_next = n["post_ffn"].add_into(h, y, next_norm, ctx.dtype)
        return h, normed_next
