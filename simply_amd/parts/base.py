"""Interfaces of the parts that a block is put together from.

A part is built from the `params` of its `PartSpec` (sizes and constants only: no
part knows which model it is in), declares the tensors it needs with
`param_specs()`, receives them with `load()`, and computes with `forward()`.
The residual stream that blocks pass along is float32 `[T, D]`; mixers and
feed-forwards take and return activations `[T, D]` in the activation dtype
(bfloat16 or float32).

Parts, per kind, and what each must provide:

* Norm:             forward(x, out_dtype) -> y;  add_into(residual, y, next_norm) (optional fusion)
* PositionEncoding: apply(x, positions, num_heads, head_dim, div); rotary_table() or None
* Mixer:            cache_need(); forward(x, ctx, cache) -> y
* FeedForward:      forward(x, ctx) -> y
* Block:            first_norm(); forward(h, ctx, cache, normed, next_norm) -> (h, normed_for_next)
"""
from __future__ import annotations

import dataclasses
from typing import Any, Mapping

import torch


@dataclasses.dataclass(frozen=True)
class ParamSpec:
    """One tensor that a part needs.

    role: 'matrix'  used in matrix products: held in the activation dtype;
          'vector'  a small tensor used in 32-bit arithmetic: a 16-bit stored one stays
                    16-bit, one stored in 32-bit stays 32-bit;
          'table'   integers: held as int32.
    init: how the random-weights mode draws it: 'weight' N(0, initializer_range),
          'norm' N(0, norm_std), 'zeros'.
    """

    shape: tuple[int, ...]
    role: str = "matrix"
    init: str = "weight"


@dataclasses.dataclass(frozen=True)
class PagedKVNeed:
    """A mixer that keeps keys and values of earlier tokens: per token `num_kv_heads * head_dim`
    keys and as many values; `window` None keeps all tokens, else only the last `window`."""

    num_kv_heads: int
    head_dim: int
    window: int | None = None


@dataclasses.dataclass(frozen=True)
class StateNeed:
    """A mixer that keeps a state of fixed size per request (zeroed when a request is admitted)."""

    shape: tuple[int, ...]
    dtype: torch.dtype = torch.float32


def as_product_weight(t: torch.Tensor, shared: bool = False):
    """A matrix in the form that the matrix-product kernels read fastest: bfloat16 matrices on the GPU are
    re-laid in tiles (simply_amd/kernels/packing.py), anything else stays row-major.  `shared`: parts that are
    handed the same tensor during one load (a tied table and head) get the same re-laid copy."""
    from ..kernels.packing import pack_tiles

    if t.dtype == torch.bfloat16 and t.is_cuda and t.dim() == 2:
        return pack_tiles(t, cached=shared)
    return t


class Part:
    """Common base: parameter declaration and loading."""

    def param_specs(self) -> dict[str, ParamSpec]:
        return {}

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        """`tensors` holds one device tensor per name of `param_specs()`, already in its final dtype."""
        for name, t in tensors.items():
            setattr(self, name, t)


class Norm(Part):
    def forward(self, x: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
        raise NotImplementedError

    def add_into(self, residual: torch.Tensor, y: torch.Tensor, next_norm: "Norm | None",
                 out_dtype: torch.dtype) -> torch.Tensor | None:
        """residual += self(y); returns next_norm(residual) if next_norm is given.
        The default does it in separate steps; a norm may fuse them."""
        from ..kernels import ops

        ops.add_rmsnorm(self.forward(y, torch.float32), residual)
        return next_norm.forward(residual, out_dtype) if next_norm is not None else None


class PositionEncoding(Part):
    def apply(self, x: torch.Tensor, positions: torch.Tensor, num_heads: int, head_dim: int, div: float = 1.0) -> None:
        """In place on x[t, h * head_dim : (h + 1) * head_dim] for h < num_heads, then x /= div."""
        raise NotImplementedError

    def rotary_table(self) -> tuple[torch.Tensor, float] | None:
        """(timescale [head_dim / 2] float32, scale_factor) if this encoding is the half-split rotation
        that the fused rotate-and-write kernel computes, else None."""
        return None


class Mixer(Part):
    def cache_need(self) -> PagedKVNeed | StateNeed | None:
        return None

    def forward(self, x: torch.Tensor, ctx: Any, cache: Any) -> torch.Tensor:
        """x: [T, D] activations of this step's tokens.  `ctx` is the step's `StepContext`; `cache` is
        this schedule entry's `CacheView` (None if cache_need() is None)."""
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, x: torch.Tensor, ctx: Any) -> torch.Tensor:
        raise NotImplementedError


class Block(Part):
    """An arrangement of a mixer, a feed-forward and norms around the residual stream."""

    def __init__(self, mixer: Mixer, feed_forward: FeedForward, norms: Mapping[str, Norm], **params):
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.norms = dict(norms)

    def first_norm(self) -> Norm | None:
        """The norm that this block applies to the residual stream first, if the block before may
        compute it together with its last residual sum."""
        return None

    def forward(self, h: torch.Tensor, ctx: Any, cache: Any, normed: torch.Tensor | None,
                next_norm: Norm | None) -> tuple[torch.Tensor, torch.Tensor | None]:
        """h: float32 residual stream [T, D], updated in place and returned.  `normed` is
        first_norm()(h) if the caller has it already.  Returns (h, next_norm(h) or None)."""
        raise NotImplementedError
