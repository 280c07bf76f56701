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

A mixer or feed-forward that sets `accepts_pending` may be handed a `PendingNorm` instead of x: the norm (and the
residual sum before it) that has not been computed yet, which `project` folds into the part's first product.
One that sets `defers_sum` takes `forward(..., defer_sum=True)` and may then return its last product with the
cuts of K not yet added up (`ops.PartialSums`); a block asks for that only when the norm that receives the result
says `adds_partial_sums`, and hands the result to that norm's `add_into` before anything else runs.
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


class PagedNeed:
    """What a mixer that keeps something for every earlier token asks of the cache manager.  The manager only
    counts pages (a page holds `page_size` consecutive tokens of one request; layers whose needs are equal share
    one pool, one free list and one block table); what a page holds and how it is laid out is the need's own
    business.  A need is hashable (a frozen dataclass) and provides

    window                     None: every token is kept; n: only the last n tokens (older pages are given back)
    page_tensors(num_pages, page_size, dtype, device, fill)
                               -> {name: tensor}, every tensor with num_pages as its first dimension, filled with
                               `fill`; one such set is made for every schedule entry that keeps a cache of its own
    bytes_per_token(esize)     bytes of storage that a token takes in one schedule entry

    Any class with these (a subclass of this one or not) is accepted."""

    window: "int | None" = None

    def page_tensors(self, num_pages: int, page_size: int, dtype: torch.dtype, device, fill: float) -> dict:
        raise NotImplementedError

    def bytes_per_token(self, esize: int) -> int:
        raise NotImplementedError


@dataclasses.dataclass(frozen=True)
class PagedKVNeed(PagedNeed):
    """A mixer that keeps keys and values of earlier tokens: per token `num_kv_heads * head_dim`
    keys and as many values; `window` None keeps all tokens, else only the last `window`.

    Pages in the layout that the attention kernels read: keys "k" [page, kv head, page_size, head_dim] (inside a
    page in 16-key x 32-dimension operand blocks when the sizes allow: simply_amd/kernels/packing.py), values "v"
    transposed [page, kv head, head_dim, page_size], so that the keys of a page are contiguous for each dimension."""

    num_kv_heads: int
    head_dim: int
    window: int | None = None

    def page_tensors(self, num_pages, page_size, dtype, device, fill):
        K, hd = self.num_kv_heads, self.head_dim
        return {"k": torch.full((num_pages, K, page_size, hd), fill, dtype=dtype, device=device),
                "v": torch.full((num_pages, K, hd, page_size), fill, dtype=dtype, device=device)}

    def bytes_per_token(self, esize):
        return 2 * self.num_kv_heads * self.head_dim * esize


@dataclasses.dataclass(frozen=True)
class StateNeed:
    """A mixer that keeps a state of fixed size per request (zeroed when a request is admitted).  The manager asks
    `slot_tensor(num_slots, device)` for the storage, one row per request slot; any class with that method is
    accepted in its place."""

    shape: tuple[int, ...]
    dtype: torch.dtype = torch.float32

    def slot_tensor(self, num_slots: int, device) -> torch.Tensor:
        return torch.zeros((num_slots, *self.shape), dtype=self.dtype, device=device)


def as_product_weight(t: torch.Tensor, shared: bool = False):
    """A matrix in the form that the matrix-product kernels read fastest: bfloat16 matrices on the GPU are
    re-laid in tiles (simply_amd/kernels/packing.py), anything else stays row-major.  `shared`: parts that are
    handed the same tensor during one load (a tied table and head) get the same re-laid copy."""
    from ..kernels.packing import pack_tiles

    if t.dtype == torch.bfloat16 and t.is_cuda and t.dim() == 2:
        return pack_tiles(t, cached=shared)
    return t


@dataclasses.dataclass
class PendingNorm:
    """Activations that are not computed yet: next_norm(residual + post_norm(y)), or next_norm(residual) if y is
    None.  A block hands this to a part that says `accepts_pending`, so that the part's first matrix product can do
    the residual sum and both norms in its own kernel (`project`); any other consumer calls `materialize()`.
    After either, `residual` is the updated residual stream (possibly another buffer) and `y` is None."""

    residual: torch.Tensor          # float32 [T, D]
    y: torch.Tensor | None          # [T, D] activations to be normed and added, or None
    post_norm: "Norm | None"        # applied to y before the sum (None: y is added as it is)
    next_norm: "Norm | None"        # applied to the sum (None: only the sum is wanted)
    dtype: torch.dtype

    def settle(self) -> torch.Tensor:
        """Does the residual sum if it is still pending; returns the updated residual stream."""
        if self.y is not None:
            from ..kernels import ops

            if self.post_norm is not None:
                self.post_norm.add_into(self.residual, self.y, None, self.dtype)
            else:
                ops.add_rmsnorm(self.y, self.residual)
            self.y = None
        return self.residual

    def rows_through(self, rows: torch.Tensor) -> torch.Tensor:
        """next_norm of the rows `rows` (int32 indices) of the pending sum, for a consumer that needs those rows only
        and nothing of the residual stream afterwards (the head at a model's end): one kernel over those rows where
        the norms can, else the sum, a gather and the norm."""
        from ..kernels import ops

        if self.next_norm is None:
            raise ValueError("a pending sum without a following norm has no activations")
        pn, nn = self.post_norm, self.next_norm
        if (self.y is not None and isinstance(self.y, torch.Tensor) and self.y.is_cuda and self.y.is_contiguous()
                and getattr(nn, "fusable_rms", False) and (pn is None or getattr(pn, "fusable_rms", False))):
            y, self.y = self.y, None
            return ops.add_rmsnorm_rows(y, self.residual, rows, post_weight=pn.scale if pn is not None else None,
                                        post_eps=pn.eps if pn is not None else 0.0,
                                        post_plus_one=pn.scale_plus_one if pn is not None else True,
                                        next_weight=nn.scale, next_eps=nn.eps, next_plus_one=nn.scale_plus_one,
                                        out_dtype=self.dtype)
        return nn.forward(ops.gather_rows(self.settle(), rows), self.dtype)

    def materialize(self) -> torch.Tensor:
        """The activations, computed with the separate kernels."""
        if self.next_norm is None:
            raise ValueError("a pending sum without a following norm has no activations")
        if self.y is not None and self.post_norm is not None:
            y, self.y = self.y, None
            return self.post_norm.add_into(self.residual, y, self.next_norm, self.dtype)
        return self.next_norm.forward(self.settle(), self.dtype)


def pending_fits_product(x, w) -> bool:
    """Whether the product kernel with the norms in front should take the pending norm `x` against the weight `w`:
    bfloat16 rows, RMSNorms with bfloat16 scales, and sizes for which the kernel library says that its fused
    kernel takes them and pays (`ops.gemm_normed_pays`)."""
    from ..kernels import ops

    if not isinstance(x, PendingNorm):
        return False
    pn, nn = x.post_norm, x.next_norm
    return (x.dtype == torch.bfloat16 and nn is not None and getattr(nn, "fusable_rms", False)
            and nn.scale.dtype == torch.bfloat16
            and (x.y is None or pn is None or (getattr(pn, "fusable_rms", False) and pn.scale.dtype == torch.bfloat16))
            and ops.gemm_normed_pays(x.residual.shape[0], w)
            and (x.y is None or (x.y.dtype == torch.bfloat16 and x.y.is_contiguous())))


def pending_product(x: PendingNorm, run) -> torch.Tensor:
    """Runs `run(y, h_in, h_out, **norm arguments)` (ops.gemm_normed or a relative of it) for a pending norm that
    `pending_fits_product`, and settles `x` with the residual that the kernel wrote."""
    pn, nn = x.post_norm, x.next_norm
    h_out = torch.empty_like(x.residual) if x.y is not None else None
    out = run(x.y, x.residual, h_out,
              post_weight=pn.scale if (pn is not None and x.y is not None) else None,
              post_eps=pn.eps if pn is not None else 0.0, post_plus_one=pn.scale_plus_one if pn is not None else True,
              next_weight=nn.scale, next_eps=nn.eps, next_plus_one=nn.scale_plus_one)
    if x.y is not None:
        x.residual, x.y = h_out, None
    return out


def project(x, w, *, soft_cap: float | None = None, out_dtype: torch.dtype | None = None,
            out: torch.Tensor | None = None, activation: int = 0, defer_sum: bool = False) -> torch.Tensor:
    """x . w^T (gated if w is a paired tiled weight) for activations x or a `PendingNorm`.  A pending norm is done
    inside the product's kernel when that kernel takes the sizes; otherwise it is materialized first.  `out`: where
    the result goes (a buffer of the caller's), else a new tensor.  `activation`: the gated product's (a code of
    the ACTIVATIONS registry).  `defer_sum`: the result may be an `ops.PartialSums` (see `ops.gemm`)."""
    import functools

    from ..kernels import ops

    if isinstance(x, PendingNorm):
        if pending_fits_product(x, w):
            return pending_product(x, functools.partial(ops.gemm_normed, w=w, soft_cap=soft_cap,
                                                        out_dtype=out_dtype or x.dtype, out=out,
                                                        activation=activation))
        x = x.materialize()
    return ops.gemm(x, w, soft_cap=soft_cap, out_dtype=out_dtype, out=out, activation=activation, defer_sum=defer_sum)


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
    #: True if forward() takes a `PendingNorm` in place of x (and consumes it with `project`)
    accepts_pending = False
    #: True if forward() takes defer_sum=True and may then return an `ops.PartialSums`
    defers_sum = False

    def cache_need(self) -> "PagedNeed | StateNeed | None":
        """What this mixer keeps between steps: a `PagedNeed` (something per token, in pages), a `StateNeed`
        (something of fixed size per request) or None."""
        return None

    def forward(self, x: torch.Tensor, ctx: Any, cache: Any) -> torch.Tensor:
        """x: [T, D] activations of this step's tokens.  `ctx` is the step's `StepContext`; `cache` is
        this schedule entry's `CacheView` (None if cache_need() is None)."""
        raise NotImplementedError


class FeedForward(Part):
    #: True if forward() takes a `PendingNorm` in place of x (and consumes it with `project`)
    accepts_pending = False
    #: True if forward() takes defer_sum=True and may then return an `ops.PartialSums`
    defers_sum = False

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

    def forward(self, h: torch.Tensor, ctx: Any, cache: Any, normed: "torch.Tensor | PendingNorm | None",
                next_norm: Norm | None) -> "tuple[torch.Tensor, torch.Tensor | PendingNorm | None]":
        """h: float32 residual stream [T, D].  `normed` is first_norm()(h) if the caller has it already, or a
        `PendingNorm` whose residual sum is still to be done (then h is the stream before that sum).  Returns
        (h, x) with x = next_norm(h), None, or a `PendingNorm` that carries the block's last sum."""
        raise NotImplementedError
