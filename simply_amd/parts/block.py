"""Block arrangements.

'sandwich' is the block of simply/model_lib.py:2659-2708 with use_pre_ln and use_post_ln:
  h += post_mixer(mixer(pre_mixer(h)));  h += post_ffn(ffn(pre_ffn(h)))
The residual stream h is float32; each residual sum is fused with the norm before it and the
norm after it where those are RMSNorms.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from ..registry import BLOCKS
from .base import Block, PendingNorm


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
        if ctx.dtype == torch.bfloat16 and ctx.positions.is_cuda and ctx.num_tokens <= ops.few_rows_limit():
            return self._forward_few_rows(h, ctx, cache, normed, next_norm)
        if isinstance(normed, PendingNorm):
            normed, h = normed.materialize(), normed.residual
        if normed is None:
            normed = n["pre_mixer"].forward(h, ctx.dtype)
        # (a part's last product may leave the sum of its cuts of K to the norm behind it, where both can)
        def defer(part, norm):
            both = part.defers_sum and getattr(norm, "adds_partial_sums", False) and ctx.dtype == torch.bfloat16
            return {"defer_sum": True} if both else {}

        y = self.mixer.forward(normed, ctx, cache, **defer(self.mixer, n["post_mixer"]))
        normed = n["post_mixer"].add_into(h, y, n["pre_ffn"], ctx.dtype)
        y = self.feed_forward.forward(normed, ctx, **defer(self.feed_forward, n["post_ffn"]))
        normed_next = n["post_ffn"].add_into(h, y, next_norm, ctx.dtype)
        return h, normed_next

    def _forward_few_rows(self, h, ctx, cache, normed, next_norm):
        """The same block for a handful of rows (decoding): every "residual sum, norm" between two parts is handed
        on as a `PendingNorm`, which the next part's first product computes in its own kernel."""
        n = self.norms

        def give(part, x):
            if isinstance(x, PendingNorm) and not part.accepts_pending:
                return x.materialize()
            return x

        x = normed if normed is not None else PendingNorm(h, None, None, n["pre_mixer"], ctx.dtype)
        y = self.mixer.forward(give(self.mixer, x), ctx, cache)
        if isinstance(x, PendingNorm):
            h = x.settle()
        x = PendingNorm(h, y, n["post_mixer"], n["pre_ffn"], ctx.dtype)
        y = self.feed_forward.forward(give(self.feed_forward, x), ctx)
        h = x.settle()
        return h, PendingNorm(h, y, n["post_ffn"], next_norm, ctx.dtype)
