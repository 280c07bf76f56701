"""What every part is told about the step it runs in.

The batch is ragged: T tokens of S requests laid end to end, a portion of a prompt beside single
decoded tokens (simply/utils/ragged_paged_attention.py:1992-2019 builds the same flat batch, with
segment ids and absolute segment positions).  The description is independent of the kind of mixer.
"""
from __future__ import annotations

import dataclasses
from typing import Callable, Hashable

import numpy as np
import torch


@dataclasses.dataclass
class GroupStep:
    """Per cache group: where this step's tokens are stored and where each request's pages are."""

    block_table: torch.Tensor   # int32 [num_slots, max_blocks]: row = request's slot, column = position // page_size
    slot_mapping: torch.Tensor  # int64 [T]: page * page_size + offset of each token of the step


@dataclasses.dataclass
class StepContext:
    dtype: torch.dtype            # activation dtype
    num_tokens: int
    positions: torch.Tensor       # int32 [T] absolute position of each token in its request
    token_seq: torch.Tensor       # int32 [T] slot of each token's request (block-table row, state row)
    seq_meta: torch.Tensor        # int32 [S, 4] per request: slot, index of its first token, its tokens, position of the first
    groups: dict[int, GroupStep]
    # host-side description, in the order of the tokens: requests with fewer tokens come first
    request_ids: list[Hashable]
    seq_slots: list[int]          # slot of each request
    seq_starts: list[int]         # tokens of the request that earlier steps have run
    q_lens: list[int]             # tokens of the request in this step
    cu_q_lens: list[int]          # [S + 1] offsets of the requests in the flat batch
    _units: dict = dataclasses.field(default_factory=dict)
    #: set for a step whose launches are recorded and replayed for later steps: the most keys that any step that
    #: replays them may have (kernels size their plans by `max_kv_len`, which is then this bound)
    kv_bound: int = 0
    #: brings an integer array that a part makes for the step to the device without waiting for the device (the
    #: executor's pinned block); None: a plain copy
    to_device: Callable[[np.ndarray], torch.Tensor] | None = None

    @property
    def num_seqs(self) -> int:
        return len(self.q_lens)

    @property
    def max_q_len(self) -> int:
        return self.q_lens[-1] if self.q_lens else 0

    @property
    def max_kv_len(self) -> int:
        """The most keys that any request of the step may attend to (of any step that replays this one's launches,
        if it is recorded)."""
        return max(self.kv_bound, max(s + q for s, q in zip(self.seq_starts, self.q_lens)))

    def short_requests(self, max_tokens: int) -> tuple[int, int]:
        """(number of leading requests with at most max_tokens tokens, number of their tokens)."""
        n = 0
        while n < len(self.q_lens) and self.q_lens[n] <= max_tokens:
            n += 1
        return n, self.cu_q_lens[n]

    def attention_units(self, tokens_per_unit: int, group: int = 1) -> tuple[torch.Tensor, int, int, int]:
        """The step's tokens cut into units of at most `tokens_per_unit` consecutive tokens of one request, in
        the layout of `seq_meta` (slot, first token, tokens, first position): what an attention kernel that takes
        few query rows at a time is launched over.  Requests that fit into one unit come first, one unit each;
        then the units of the longer requests, each request's units filled up with empty ones to a multiple of
        `group`, so that a kernel that takes `group` units at a time never mixes requests.  Returns (units
        int32 [U, 4] on the device, number of one-unit requests, number of units after them, most tokens in a
        unit)."""
        if self.max_q_len <= tokens_per_unit:
            return self.seq_meta, self.num_seqs, 0, self.max_q_len
        key = (tokens_per_unit, group)
        cached = self._units.get(key)
        if cached is None:
            few, many = [], []
            for slot, first, start, q in zip(self.seq_slots, self.cu_q_lens, self.seq_starts, self.q_lens):
                if q <= tokens_per_unit:
                    few.append((slot, first, q, start))
                    continue
                count = -(-q // tokens_per_unit)
                at = np.minimum(np.arange(-(-count // group) * group) * tokens_per_unit, q)
                block = np.empty((len(at), 4), dtype=np.int32)
                block[:, 0], block[:, 1], block[:, 3] = slot, first + at, start + at
                block[:, 2] = np.minimum(q - at, tokens_per_unit)
                many.append(block)
            rows = np.concatenate([np.asarray(few, dtype=np.int32).reshape(-1, 4)] + many)
            units = self.to_device(rows) if self.to_device is not None else \
                torch.from_numpy(rows).to(self.positions.device)
            cached = (units, len(few), len(rows) - len(few), tokens_per_unit)
            self._units[key] = cached
        return cached
