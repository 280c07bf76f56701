"""Sampling parameters, with the names and meanings of simply/utils/sampling_lib.py:74-100."""
from __future__ import annotations

import dataclasses

INT32_MAX_HALF = (2**31 - 1) // 2


@dataclasses.dataclass(frozen=True)
class SamplingParams:
    #: 0 is greedy (argmax, log-probability 0): simply/utils/sampling_lib.py:532-537
    temperature: float = 1.0
    #: -1 is off; 1 is greedy
    top_k: int = -1
    #: 1.0 is off
    top_p: float = 1.0
    #: most tokens to generate
    max_decode_steps: int = 256
    #: prompt and generated tokens together stop here (the result is then marked truncated)
    max_seq_len: int = INT32_MAX_HALF
    #: longer prompts keep their trailing `max_input_len` tokens (simply/utils/sampling_lib.py:368-369)
    max_input_len: int | None = None
    #: seed of this request's own random stream; None: derived from the engine's seed and the request's index
    seed: int | None = None
    #: keep generating past an end-of-sequence token (for benchmarks)
    ignore_eos: bool = False

    def validate(self) -> None:
        if self.temperature < 0:
            raise ValueError("temperature must be >= 0")
        if self.top_k == 0 or self.top_k < -1:
            raise ValueError("top_k must be -1 (off) or positive")
        if not 0 < self.top_p <= 1:
            raise ValueError("top_p must be in (0, 1]")
        if self.max_decode_steps < 1:
            raise ValueError("max_decode_steps must be at least 1")

    @property
    def is_greedy(self) -> bool:
        return self.temperature == 0 or self.top_k == 1


@dataclasses.dataclass(frozen=True)
class ScoringParams:
    """What a token's score is computed under (simply/model_lib.py:4521-4533)."""

    temperature: float = 1.0
    top_k: int = -1
    top_p: float = 1.0

    @classmethod
    def from_sampling_params(cls, sampling_params: SamplingParams) -> "ScoringParams":
        return cls(temperature=sampling_params.temperature, top_k=sampling_params.top_k, top_p=sampling_params.top_p)

    def validate(self) -> None:
        SamplingParams(temperature=self.temperature, top_k=self.top_k, top_p=self.top_p).validate()
