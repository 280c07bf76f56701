"""RMSNorm with an optional `(1 + scale)` gain (simply/model_lib.py:114-178, LayerNorm with
use_bias=False).  Statistics and the multiplication are in float32."""
from __future__ import annotations

import torch

from ..kernels import ops
from ..registry import NORMS
from .base import Norm, ParamSpec


@NORMS.register("rmsnorm")
class RMSNorm(Norm):
    #: the fused norm-and-product kernel computes exactly this norm from (scale, eps, scale_plus_one)
    fusable_rms = True
    #: add_into takes a product whose cuts of K are not added up yet (`ops.PartialSums`) in place of y
    adds_partial_sums = True

    def __init__(self, dim: int, eps: float, scale_plus_one: bool = True):
        self.dim = int(dim)
        self.eps = float(eps)
        self.scale_plus_one = bool(scale_plus_one)
        self.scale: torch.Tensor | None = None

    def param_specs(self):
        return {"scale": ParamSpec((self.dim,), role="vector", init="norm")}

    def forward(self, x, out_dtype):
        return ops.rmsnorm(x, self.scale, self.eps, self.scale_plus_one, out_dtype)

    def add_into(self, residual, y, next_norm, out_dtype):
        """residual += self(y) and, fused when the next norm is an RMSNorm too, next_norm(residual)."""
        if next_norm is None or isinstance(next_norm, RMSNorm):
            return ops.add_rmsnorm(
                y, residual, post_weight=self.scale, post_eps=self.eps, post_plus_one=self.scale_plus_one,
                next_weight=None if next_norm is None else next_norm.scale,
                next_eps=0.0 if next_norm is None else next_norm.eps,
                next_plus_one=True if next_norm is None else next_norm.scale_plus_one, out_dtype=out_dtype)
        ops.add_rmsnorm(y, residual, post_weight=self.scale, post_eps=self.eps, post_plus_one=self.scale_plus_one)
        return next_norm.forward(residual, out_dtype)
