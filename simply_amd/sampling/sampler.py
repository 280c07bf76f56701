"""Draws one token per row of logits with the HIP sampling kernel.

Every request has its own random stream, keyed by its seed and advanced by its own count of drawn
tokens, so its tokens do not depend on which other requests are in the batch (the reference splits
one key per step for the whole batch: simply/utils/ragged_paged_attention.py:2031).
"""
from __future__ import annotations

from typing import Sequence

import numpy as np
import torch

from ..kernels import ops
from .params import SamplingParams


def request_seed(engine_seed: int, request_index: int) -> int:
    """A 63-bit seed for a request that brought none (splitmix64 of the engine seed and the index)."""
    z = (engine_seed * 0x9E3779B97F4A7C15 + request_index + 1) & (2**64 - 1)
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & (2**64 - 1)
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & (2**64 - 1)
    return (z ^ (z >> 31)) & (2**63 - 1)


class Sampler:
    def __init__(self, device, max_rows: int):
        self.device = torch.device(device)
        self.max_rows = max_rows
        pin = self.device.type == "cuda"
        # [temperature | top_p] as float32 and [top_k | counter] as int32, seeds as int64: one staging buffer each
        self._f_host = torch.empty(2 * max_rows, dtype=torch.float32, pin_memory=pin)
        self._i_host = torch.empty(2 * max_rows, dtype=torch.int32, pin_memory=pin)
        self._s_host = torch.empty(max_rows, dtype=torch.int64, pin_memory=pin)
        self._f_dev = torch.empty(2 * max_rows, dtype=torch.float32, device=self.device)
        self._i_dev = torch.empty(2 * max_rows, dtype=torch.int32, device=self.device)
        self._s_dev = torch.empty(max_rows, dtype=torch.int64, device=self.device)
        # tokens and log-probabilities in one buffer, so that one copy brings both to the host
        self._out = torch.empty(2 * max_rows, dtype=torch.int32, device=self.device)
        self._out_host = torch.empty(2 * max_rows, dtype=torch.int32, pin_memory=pin)
        self._tokens = self._out[:max_rows]
        self._logprobs = self._out[max_rows:].view(torch.float32)
        #: what the staged rows ask for (ops.SAMPLE_*): `launch` leaves out the kernels that none of them needs, so
        #: a recorded launch serves only rows that ask for no more than these
        self.modes = 0

    def stage(self, params: Sequence[SamplingParams], seeds: Sequence[int], counters: Sequence[int]) -> None:
        """Puts the rows' parameters, seeds and draw counters where `launch` reads them (fixed device buffers)."""
        R = len(params)
        if not (len(seeds) == len(counters) == R):
            raise ValueError("sample: one params, seed and counter per row of logits")
        if R > self.max_rows:
            raise ValueError(f"sample: {R} rows, room for {self.max_rows}")
        n = self.max_rows
        self.modes = self.modes_of(params)
        f, i, sd = self._f_host.numpy(), self._i_host.numpy(), self._s_host.numpy()
        f[:R] = [p.temperature for p in params]
        f[n:n + R] = [p.top_p for p in params]
        i[:R] = [p.top_k for p in params]
        i[n:n + R] = counters
        sd[:R] = seeds
        self._f_dev.copy_(self._f_host, non_blocking=True)
        self._i_dev.copy_(self._i_host, non_blocking=True)
        self._s_dev.copy_(self._s_host, non_blocking=True)

    @staticmethod
    def modes_of(params: Sequence[SamplingParams]) -> int:
        """What these rows ask of the sampling kernels: a draw at all, top-k, top-p."""
        modes = 0
        for p in params:
            if p.temperature != 0.0 and p.top_k != 1:
                modes |= ops.SAMPLE_DRAWN
                if p.top_k > 0:
                    modes |= ops.SAMPLE_TOP_K
                if p.top_p < 1.0:
                    modes |= ops.SAMPLE_TOP_P
        return modes

    @property
    def draw_counters(self) -> torch.Tensor:
        """The rows' draw counters on the device (int32 [max_rows]); `launch` reads them."""
        return self._i_dev[self.max_rows:]

    def launch(self, logits: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
        """The sampling kernel on what `stage` left: returns the device buffers (tokens int32, log-probabilities
        float32, [max_rows], the same every time) without waiting for it."""
        n = self.max_rows
        return ops.sample(logits, self._f_dev[:n], self._i_dev[:n], self._f_dev[n:], self._s_dev, self._i_dev[n:],
                          self._tokens, self._logprobs, modes=self.modes)

    def sample(self, logits: torch.Tensor, params: Sequence[SamplingParams], seeds: Sequence[int],
               counters: Sequence[int]) -> tuple[list[int], list[float]]:
        """logits float32 [R, V]; one SamplingParams, seed and draw counter per row."""
        R = logits.shape[0]
        if len(params) != R:
            raise ValueError("sample: one params, seed and counter per row of logits")
        self.stage(params, seeds, counters)
        tokens, logprobs = self.launch(logits)
        # one synchronising copy back: the scheduler needs the tokens to go on
        n = self.max_rows
        self._out_host.copy_(self._out, non_blocking=True)
        if self.device.type == "cuda":
            torch.cuda.current_stream(self.device).synchronize()
        host = self._out_host.numpy()
        return host[:R].tolist(), host[n:n + R].view(np.float32).tolist()
