"""How far the engine's logits may lie from the plain implementation in float64.

float32: 2e-5 of the largest logit (the reference's own bar for its cached against its uncached
logits is atol 1e-5, simply/model_lib_test.py:631; the plain implementation run in float32 differs from
itself in float64 by up to 1e-5 on the worst of the configurations used here).

bfloat16: no constant fits every configuration: a model whose softmax is sharp (no soft-cap, a small
query_pre_attn_scalar, large weights) amplifies the rounding of its activations ten times more than one
whose softmax is flat.  The bound is therefore derived per model and sequence: the plain implementation
is run once more with its intermediate results rounded to bfloat16 at the places where an engine with a
32-bit residual stream rounds (`plain.rounding_of_fp32_residual_engine`), and the engine may differ from
the float64 run by
    RMS_FACTOR x the root-mean-square error of that rounded run, and
    MAX_FACTOR x its largest error.
Measured over 53 configurations (two sequences each, whole and token by token) the engine's RMS error was
0.61 to 1.08 times the rounded run's and its largest error 0.49 to 1.66 times: both are samples of the same
rounding noise, so the factors leave room for the sampling alone and a kernel that loses a bit of
precision (x 1.4 in RMS) fails.  The reference's own rounding (every einsum result, the scores, the residual
stream: `plain.rounding_like_simply`) gives 1.3 to 2 times the error of the engine's places.
"""
from __future__ import annotations

import dataclasses

import torch

import plain_gemma2 as plain

FP32_TOL = 2e-5
RMS_FACTOR = 1.3
MAX_FACTOR = 2.5
# the RMS of two runs' rounding noise is compared over at least this many positions of at least this many logits
# together (the noise of one position's logits is correlated: it comes through one final activation vector)
RMS_MIN_ROWS = 16
RMS_MIN_VALUES = 8192


@dataclasses.dataclass
class Reference:
    want: torch.Tensor          # float64 logits [T, V] of the plain implementation
    rounded: torch.Tensor | None  # the same with bfloat16 rounding at the engine's places (bfloat16 only)
    dtype: str

    @property
    def scale(self) -> float:
        return self.want.abs().max().item()

    def max_bound(self) -> float:
        """Largest allowed difference, as a fraction of the largest logit."""
        if self.dtype == "float32":
            return FP32_TOL
        return MAX_FACTOR * (self.rounded - self.want).abs().max().item() / self.scale

    def check(self, got: torch.Tensor, rows=None, what="", rms: bool = True) -> float:
        """Asserts that `got` (logits at `rows` of the sequence, all rows if None) is within the bound.
        Returns the largest difference as a fraction of the largest logit.  rms=False: the largest error only (the
        caller pools the squared errors of several requests in a `Pooled` and checks their RMS together)."""
        got = got.double().cpu()
        assert torch.isfinite(got).all(), (what, "not finite")
        want = self.want if rows is None else self.want[rows]
        assert got.shape == want.shape, (what, got.shape, want.shape)
        diff = got - want
        err = diff.abs().max().item() / self.scale
        assert err <= self.max_bound(), (what, "largest error", err, "bound", self.max_bound())
        if rms and self.dtype != "float32" and diff.shape[0] >= RMS_MIN_ROWS and diff.numel() >= RMS_MIN_VALUES:
            rounded = self.rounded if rows is None else self.rounded[rows]
            rms = diff.pow(2).mean().sqrt().item()
            rms_ref = (rounded - want).pow(2).mean().sqrt().item()
            assert rms <= RMS_FACTOR * rms_ref, (what, "rms error", rms / self.scale, "rounded plain run",
                                                 rms_ref / self.scale)
        return err


class Pooled:
    """The RMS criterion over many short comparisons of one model (single decode steps, a few rows per request):
    each `add` contributes its squared errors, the engine's and the rounded plain run's, and `check` compares the
    two sums once enough rows and values have come together.  A step's rows alone are too few for the ratio of two
    samples of rounding noise to mean anything; pooled over the requests of a test they are not."""

    def __init__(self):
        self.engine = self.rounded = 0.0
        self.rows = self.values = 0
        self.scale = 0.0

    def add(self, ref: Reference, got: torch.Tensor, rows=None) -> None:
        if ref.dtype == "float32":
            return
        got = got.double().cpu()
        want = ref.want if rows is None else ref.want[rows]
        rounded = ref.rounded if rows is None else ref.rounded[rows]
        self.engine += (got - want).pow(2).sum().item()
        self.rounded += (rounded - want).pow(2).sum().item()
        self.rows += want.shape[0]
        self.values += want.numel()
        self.scale = max(self.scale, ref.scale)

    def check(self, what="") -> None:
        if self.rows >= RMS_MIN_ROWS and self.values >= RMS_MIN_VALUES:
            rms, rms_ref = (self.engine / self.values) ** 0.5, (self.rounded / self.values) ** 0.5
            assert rms <= RMS_FACTOR * rms_ref, (what, "pooled rms error", rms / self.scale, "rounded plain run",
                                                 rms_ref / self.scale, "rows", self.rows)


def reference(weights: dict, cfg: dict, tokens, dtype: str, device=None, rows=None) -> Reference:
    """weights: as stored (float32); for bfloat16 they are rounded first, as the engine holds them.  device: where
    torch computes the plain implementation (the CPU by default); rows: keep only these positions' logits (a slice
    or indices; `check` then counts its rows among them)."""
    if dtype == "bfloat16":
        weights = {k: v.to(torch.bfloat16) for k, v in weights.items()}
    keep = (lambda t: t.cpu()) if rows is None else (lambda t: t[rows].cpu())
    want = keep(plain.forward(weights, cfg, tokens, torch.float64, device=device))
    rounded = None
    if dtype == "bfloat16":
        rounded = keep(plain.forward(weights, cfg, tokens, torch.float64, rnd=plain.rounding_of_fp32_residual_engine(),
                                     device=device))
    return Reference(want, rounded, dtype)


def reference_of(model_dir: str, tokens, dtype: str) -> Reference:
    w, cfg = plain.load(model_dir)
    return reference(w, cfg, tokens, dtype)
