"""Token embedding and the output head.

simply/utils/module.py:450-481: lookup, then times sqrt(dim) * embedding_scale, the factor
rounded to the activation dtype first.  simply/model_lib.py:3184-3189: logits are the product
with the (tied) table, then the final soft-cap if it is > 0.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from ..registry import EMBEDDINGS, HEADS
from .base import ParamSpec, Part, as_product_weight, project


@EMBEDDINGS.register("scaled_embedding")
class ScaledEmbedding(Part):
    def __init__(self, vocab_size: int, dim: int, scale: float):
        self.vocab_size, self.dim, self.scale = int(vocab_size), int(dim), float(scale)
        self.table: torch.Tensor | None = None

    def param_specs(self):
        return {"table": ParamSpec((self.vocab_size, self.dim), role="matrix", init="weight")}

    def load(self, tensors):
        # tiled like a product weight when it is bfloat16 on the GPU: a tied head reads the same storage
        self.table = as_product_weight(tensors["table"], shared=True)

    def forward(self, tokens: torch.Tensor) -> torch.Tensor:
        """tokens int32 [T] -> float32 residual stream [T, D]."""
        # the factor is rounded to the table's dtype (module.py:476-480), the product is kept in float32
        scale = float(torch.tensor(self.scale, dtype=self.table.dtype))
        return ops.embed(self.table, tokens, scale)


@HEADS.register("linear_head")
class LinearHead(Part):
    def __init__(self, vocab_size: int, dim: int, soft_cap: float | None):
        self.vocab_size, self.dim = int(vocab_size), int(dim)
        self.soft_cap = float(soft_cap) if soft_cap else None
        self.weight: torch.Tensor | None = None

    def param_specs(self):
        return {"weight": ParamSpec((self.vocab_size, self.dim), role="matrix", init="weight")}

    def load(self, tensors):
        self.weight = as_product_weight(tensors["weight"], shared=True)

    def forward(self, x: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
        """x [R, D] activations (or a `PendingNorm` of them) -> float32 logits [R, V] (written into `out` if given)."""
        return project(x, self.weight, soft_cap=self.soft_cap, out_dtype=torch.float32, out=out)

