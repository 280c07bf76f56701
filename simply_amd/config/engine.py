"""Serving knobs.  Names follow simply/serving/common_flags.py:51-92 where the
reference has the knob (batch_size, page_size, max_seq_len, max_num_issue_tokens,
activation_dtype)."""
from __future__ import annotations

import dataclasses

import torch

_DTYPES = {
    "bfloat16": torch.bfloat16, "bf16": torch.bfloat16,
    "float32": torch.float32, "fp32": torch.float32, "f32": torch.float32,
}


def parse_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name not in (torch.bfloat16, torch.float32):
            raise ValueError(f"activation dtype must be bfloat16 or float32, not {name}")
        return name
    try:
        return _DTYPES[str(name)]
    except KeyError:
        raise ValueError(f"activation dtype must be bfloat16 or float32, not {name!r}") from None


@dataclasses.dataclass(frozen=True)
class EngineConfig:
    #: 'bfloat16' (serving kernels) or 'float32' (everything in true 32-bit).
    activation_dtype: str = "bfloat16"
    #: tokens per cache page (simply: --page_size, 128 on TPU; 16 suits CDNA4 gathers).
    page_size: int = 16
    #: live requests at most (simply: --batch_size).
    batch_size: int = 8
    #: longest sequence, prompt and generated tokens together (simply: --max_seq_len).
    max_seq_len: int = 8192
    #: most tokens in one step over all requests (simply: --max_num_issue_tokens; 0 = batch_size).
    max_num_issue_tokens: int = 2048
    #: pages of a cache group that keeps every token (simply: total_num_pages of the global layers' pool,
    #: simply/serving/page_server.py:180-196); None = from `memory_fraction` if that is set, else enough for
    #: batch_size sequences of max_seq_len.
    total_num_pages: int | None = None
    #: pages of a cache group that keeps a window only (simply: the local layers' pool); None = what batch_size
    #: requests can hold at once (a window and the step's tokens each).
    windowed_num_pages: int | None = None
    #: size the pools from the device memory that is free once the weights are loaded: this fraction of it goes to
    #: the cache (windowed groups get what their requests can hold, the groups that keep everything share the rest,
    #: never more than batch_size sequences of max_seq_len need).  Used when total_num_pages is None.
    memory_fraction: float | None = None
    #: decode steps that may run in a row without a new scheduling decision (simply: --intermediate_steps); the
    #: windowed pools leave room for that many tokens ahead of every request.
    intermediate_steps: int = 64
    #: fill freed pages with NaN so that a read of an unwritten key shows.
    poison_freed_pages: bool = False
    #: capture decode-only steps in HIP graphs.
    use_graphs: bool = True
    device: str = "cuda:0"

    @property
    def dtype(self) -> torch.dtype:
        return parse_dtype(self.activation_dtype)

    @property
    def issue_budget(self) -> int:
        return self.max_num_issue_tokens if self.max_num_issue_tokens > 0 else self.batch_size

    def validate(self) -> None:
        parse_dtype(self.activation_dtype)
        if self.page_size < 1:
            raise ValueError("page_size must be at least 1")
        if self.batch_size < 1:
            raise ValueError("batch_size must be at least 1")
        if self.max_seq_len < 2:
            raise ValueError("max_seq_len must be at least 2")
        if self.memory_fraction is not None and not 0.0 < self.memory_fraction <= 1.0:
            raise ValueError("memory_fraction must lie in (0, 1]")
        for name in ("total_num_pages", "windowed_num_pages"):
            if getattr(self, name) is not None and getattr(self, name) < 1:
                raise ValueError(f"{name} must be at least 1")
        if self.intermediate_steps < 1:
            raise ValueError("intermediate_steps must be at least 1")

    @property
    def max_step_tokens(self) -> int:
        """The most tokens for which one step reserves pages: a step's token budget, or every request's run of
        decode steps ahead."""
        return max(self.issue_budget, self.batch_size * self.intermediate_steps)
