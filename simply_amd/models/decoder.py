"""A decoder put together from a `ModelSpec`: embedding, the layers run in the order of the
schedule, final norm, head (simply/model_lib.py:2750 TransformerLM, apply :2935-3189).

The model knows nothing of any one architecture: every part is built from its registry by
the kind that the spec names.
"""
from __future__ import annotations

import dataclasses
from typing import Callable, Mapping

import torch

from .. import parts as _parts  # noqa: F401  (registers the built-in parts)
from ..config.spec import LayerSpec, ModelSpec, PartSpec
from ..kernels import ops
from ..parts.base import Block, ParamSpec, Part, PendingNorm
from ..registry import BLOCKS, EMBEDDINGS, FEED_FORWARDS, HEADS, MIXERS, NORMS
from ..weights import binding


def _build_layer(spec: LayerSpec) -> Block:
    mixer = MIXERS.build(spec.mixer.kind, **spec.mixer.params)
    ffn = FEED_FORWARDS.build(spec.feed_forward.kind, **spec.feed_forward.params)
    norms = {name: NORMS.build(ns.kind, **ns.params) for name, ns in spec.norms.items()}
    return BLOCKS.build(spec.block.kind, mixer, ffn, norms, **spec.block.params)


class DecoderModel:
    def __init__(self, spec: ModelSpec):
        spec.validate()
        self.spec = spec
        self.embedding = EMBEDDINGS.build(spec.embedding.kind, **spec.embedding.params)
        self.head = HEADS.build(spec.head.kind, **spec.head.params)
        self.final_norm = NORMS.build(spec.final_norm.kind, **spec.final_norm.params)
        self.layers: list[Block] = [_build_layer(ls) for ls in spec.layers]
        self.loaded = False

    # ------------------------------------------------------------------ tensors
    def _bindings(self) -> list[tuple[Part, PartSpec]]:
        out: list[tuple[Part, PartSpec]] = [(self.embedding, self.spec.embedding)]
        for block, ls in zip(self.layers, self.spec.layers):
            out.append((block.mixer, ls.mixer))
            out.append((block.feed_forward, ls.feed_forward))
            for name, ns in ls.norms.items():
                out.append((block.norms[name], ns))
        out.append((self.final_norm, self.spec.final_norm))
        out.append((self.head, self.spec.head))
        return out

    def tensor_bindings(self) -> list[tuple[Part, str, ParamSpec, "binding.Binding"]]:
        """For every parameter of every part: (part, the part's name for it, what the part expects, how it is
        obtained from stored tensors).  A spec that names a plain tensor means that tensor as it is."""
        out = []
        for part, ps in self._bindings():
            for local, pspec in part.param_specs().items():
                if local not in ps.tensors:
                    raise ValueError(f"part {ps.kind!r} needs a tensor {local!r} that its spec does not name")
                b = binding.normalize(ps.tensors[local], pspec.shape)
                try:
                    got = binding.shape_of(b)
                except binding.BindingError as e:
                    raise ValueError(f"part {ps.kind!r}, tensor {local!r}: {e}") from None
                if tuple(got) != tuple(pspec.shape):
                    raise ValueError(f"part {ps.kind!r}, tensor {local!r}: the binding gives shape {list(got)}, the "
                                     f"part expects {list(pspec.shape)}")
                out.append((part, local, pspec, b))
        return out

    def expected_tensors(self) -> dict[str, ParamSpec]:
        """Stored tensor name in the model folder -> what is expected of it (its stored shape; role and random
        initialisation of the parameter that it feeds), in a fixed order."""
        expected: dict[str, ParamSpec] = {}
        for _, _, pspec, b in self.tensor_bindings():
            for leaf in binding.leaves(b):
                if leaf.name in expected and expected[leaf.name].shape != leaf.shape:
                    raise ValueError(f"tensor {leaf.name!r} is used with shapes {expected[leaf.name].shape} and "
                                     f"{leaf.shape}")
                expected.setdefault(leaf.name, dataclasses.replace(pspec, shape=leaf.shape))
        return expected

    def load_tensors(self, tensors: Mapping[str, torch.Tensor]) -> None:
        """`tensors`: stored name -> device tensor in its final dtype.  Every part receives its parameters as its
        spec's bindings make them from these."""
        from ..kernels import packing

        per_part: dict[int, tuple[Part, dict[str, torch.Tensor]]] = {}
        for part, local, _, b in self.tensor_bindings():
            per_part.setdefault(id(part), (part, {}))[1][local] = binding.evaluate(b, tensors.__getitem__)
        try:
            for part, _ in self._bindings():
                part.load(per_part.get(id(part), (part, {}))[1])
        finally:
            packing.clear_cache()   # sharing of re-laid tensors (tied table and head) ends with the load
        self.loaded = True

    # ------------------------------------------------------------------ cache
    def cache_needs(self):
        """For each schedule entry: (need of its mixer or None, cache_from)."""
        return [(self.layers[e.layer].mixer.cache_need(), e.cache_from) for e in self.spec.schedule]

    # ------------------------------------------------------------------ forward
    def forward(self, tokens: torch.Tensor, ctx, cache_views, logit_rows: torch.Tensor | None,
                logits_out: torch.Tensor | None = None) -> torch.Tensor | None:
        """Runs this step's tokens through the schedule.  Returns float32 logits [R, V] at the rows of
        the step that `logit_rows` (int32 [R]) names (in `logits_out` if that is given), or None if it is None or
        empty."""
        h = self.embedding.forward(tokens)
        schedule = self.spec.schedule
        normed = None
        for i, entry in enumerate(schedule):
            block = self.layers[entry.layer]
            nxt = self.layers[schedule[i + 1].layer].first_norm() if i + 1 < len(schedule) else None
            h, normed = block.forward(h, ctx, cache_views[i], normed, nxt)
        if logit_rows is None or logit_rows.numel() == 0:
            return None
        if isinstance(normed, PendingNorm):
            # the last block's residual sum is still pending: the final norm of the wanted rows comes out of the
            # same kernel (the residual stream itself is of no use to anyone after the last block)
            pending = PendingNorm(normed.residual, normed.y, normed.post_norm, self.final_norm, ctx.dtype)
            return self.head.forward(pending.rows_through(logit_rows), out=logits_out)
        rows = ops.gather_rows(h, logit_rows)
        return self.head.forward(PendingNorm(rows, None, None, self.final_norm, ctx.dtype), out=logits_out)
