"""The scheduler: admits requests, cuts prompts into portions under a token budget, decodes,
finishes and frees.

After `Batcher.loop` (simply/serving/page_batcher.py:701-895) and `SamplingState.issue_lens`
(simply/utils/ragged_paged_attention.py:1821-1859): decoding requests go first, oldest first, then
requests that are still in their prompt, oldest first; each gets all it wants until the budget
runs out, so one request gets a partial portion and the rest nothing.  The reference sizes its
page pool so that pages cannot run out (simply/serving/page_server.py:175-204); here they can, and
then:

* a request is admitted only when the free pages hold all the tokens it brings (its prompt, and what it
  had generated if it comes back after giving up its pages), and not in a step in which a request gave way;
* a later portion of a running request's prompt shrinks to the tokens that the free pages hold, and waits
  if that is none;
* a decoding request that cannot get a page makes the newest running request give up everything it
  holds; that request goes back to the front of the queue and later runs again from its first
  token, prompt and generated tokens together (its generated tokens are kept);
* a request that could not fit even with the whole cache to itself is finished at once, truncated.

The scheduler decides on the host from the cache manager's bookkeeping alone.
"""
from __future__ import annotations

import collections
import dataclasses
import enum
from typing import Hashable, Sequence

from ..cache import CacheManager
from ..sampling import SamplingParams


class Status(enum.Enum):
    WAITING = "waiting"
    RUNNING = "running"
    FINISHED = "finished"


@dataclasses.dataclass
class Request:
    request_id: Hashable
    prompt_token_ids: list[int]
    params: SamplingParams
    seed: int = 0
    arrival: int = 0
    eos_ids: tuple[int, ...] = ()
    status: Status = Status.WAITING
    output_token_ids: list[int] = dataclasses.field(default_factory=list)
    output_token_logprobs: list[float] = dataclasses.field(default_factory=list)
    num_computed: int = 0           # tokens whose keys are in the cache
    finish_reason: str | None = None  # 'eos', 'length' (max_decode_steps), 'max_seq_len', 'no_room'
    num_preemptions: int = 0

    @property
    def all_token_ids(self) -> list[int]:
        return self.prompt_token_ids + self.output_token_ids

    def tokens(self, start: int, count: int) -> list[int]:
        """Tokens start .. start + count - 1 of prompt and output together, without laying the two end to end."""
        p = len(self.prompt_token_ids)
        if start >= p:
            return self.output_token_ids[start - p:start - p + count]
        if start + count <= p:
            return self.prompt_token_ids[start:start + count]
        return self.prompt_token_ids[start:] + self.output_token_ids[:start + count - p]

    @property
    def num_tokens(self) -> int:
        return len(self.prompt_token_ids) + len(self.output_token_ids)

    @property
    def is_truncated(self) -> bool:
        """Ended before a natural end-of-sequence token (SamplingOutput.is_truncated, simply/model_lib.py:4472)."""
        return self.finish_reason != "eos"


@dataclasses.dataclass
class Scheduled:
    request: Request
    start: int          # position of the first token of the portion
    num_tokens: int
    samples: bool       # the portion ends at the request's last known token: its logits are sampled from


@dataclasses.dataclass
class SchedulerOutput:
    scheduled: list[Scheduled]
    preempted: list[Request]
    finished: list[Request]   # finished without running (no room)

    @property
    def num_tokens(self) -> int:
        return sum(s.num_tokens for s in self.scheduled)


class Scheduler:
    def __init__(self, cache: CacheManager, *, max_num_issue_tokens: int, max_seq_len: int):
        self.cache = cache
        self.budget = int(max_num_issue_tokens)
        # a request can never hold more tokens than one group's pages hold
        self.max_seq_len = min(int(max_seq_len), cache.num_pages * cache.page_size)
        self.waiting: collections.deque[Request] = collections.deque()
        self.running: list[Request] = []
        self._arrivals = 0

    # ------------------------------------------------------------------ queue
    def add(self, request: Request) -> None:
        if not request.prompt_token_ids:
            raise ValueError(f"request {request.request_id!r} has an empty prompt")
        request.params.validate()
        # simply/utils/ragged_paged_attention.py:1609-1613 refuses a prompt longer than max_seq_len;
        # the input processor keeps the trailing max_input_len tokens (simply/utils/sampling_lib.py:368-369)
        if request.params.max_input_len is not None and len(request.prompt_token_ids) > request.params.max_input_len:
            request.prompt_token_ids = request.prompt_token_ids[-request.params.max_input_len:]
        if len(request.prompt_token_ids) >= self._limit(request):
            raise ValueError(f"request {request.request_id!r}: a prompt of {len(request.prompt_token_ids)} tokens "
                             f"leaves no room to generate under max_seq_len {self._limit(request)}")
        request.arrival = self._arrivals
        self._arrivals += 1
        request.status = Status.WAITING
        self.waiting.append(request)

    def adopt(self, request: Request, num_computed: int) -> None:
        """Takes over a request whose first `num_computed` tokens already have their keys in the cache (written by
        the caller, for instance a benchmark that fills the pages instead of running a long prompt): the request is
        admitted and its pages are reserved and given back exactly as if those tokens had run in portions of the
        token budget, one request at a time, so a windowed group ends up holding its window only.  The request goes
        on from there like any running request.  Raises `OutOfPages` (and leaves nothing behind) if it does not fit."""
        if not request.prompt_token_ids:
            raise ValueError(f"request {request.request_id!r} has an empty prompt")
        request.params.validate()
        n = int(num_computed)
        if not 0 <= n < request.num_tokens:
            raise ValueError(f"request {request.request_id!r}: {n} computed tokens of {request.num_tokens}")
        if request.num_tokens >= self._limit(request):
            raise ValueError(f"request {request.request_id!r}: {request.num_tokens} tokens leave no room to generate "
                             f"under max_seq_len {self._limit(request)}")
        cache, rid = self.cache, request.request_id
        cache.admit(rid)
        try:
            for at in range(0, n, self.budget):
                q = min(self.budget, n - at)
                cache.reserve(rid, at, q)
                cache.mark_issued([(rid, at, q)])
        except Exception:
            cache.free(rid)
            raise
        request.arrival = self._arrivals
        self._arrivals += 1
        request.num_computed = n
        request.status = Status.RUNNING
        self.running.append(request)

    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    def _limit(self, r: Request) -> int:
        return min(self.max_seq_len, r.params.max_seq_len)

    # ------------------------------------------------------------------ one step's decisions
    def _fit(self, r: Request, start: int, want: int) -> int:
        """The most tokens <= want of r, from position start, that the free pages of every group hold."""
        if self.cache.can_reserve([(r.request_id, start, want)]):
            return want
        lo, hi = 0, want  # lo fits (0 tokens need no page), hi does not
        while hi - lo > 1:
            mid = (lo + hi) // 2
            if self.cache.can_reserve([(r.request_id, start, mid)]):
                lo = mid
            else:
                hi = mid
        return lo

    def _preempt(self, r: Request, out: SchedulerOutput) -> None:
        self.cache.free(r.request_id)
        self.running.remove(r)
        r.status = Status.WAITING
        r.num_computed = 0
        r.num_preemptions += 1
        self.waiting.appendleft(r)
        out.preempted.append(r)

    def schedule(self) -> SchedulerOutput:
        out = SchedulerOutput([], [], [])
        budget = self.budget
        # 1. decoding requests, oldest first; each needs room for one token
        decoding = sorted((r for r in self.running if r.num_computed == r.num_tokens - 1), key=lambda r: r.arrival)
        scheduled_ids = set()
        if decoding and budget >= len(decoding):
            # the usual case, all of them fit: one question to the cache instead of one per request (each costs
            # a pass over all live requests).  The requests one by one below decide the same when this holds.
            wants = [(r.request_id, r.num_computed, 1) for r in decoding]
            if self.cache.can_reserve(wants):
                self.cache.reserve_all(wants)
                for r in decoding:
                    out.scheduled.append(Scheduled(r, r.num_computed, 1, True))
                    scheduled_ids.add(r.request_id)
                budget -= len(decoding)
                decoding = []
        for r in decoding:
            if r.status is not Status.RUNNING or budget < 1:
                continue
            while not self.cache.can_reserve([(r.request_id, r.num_computed, 1)]):
                victims = [v for v in self.running if v.request_id not in scheduled_ids]
                victim = max(victims, key=lambda v: v.arrival)
                self._preempt(victim, out)
                if victim is r:
                    break
            if r.status is not Status.RUNNING:
                continue
            self.cache.reserve(r.request_id, r.num_computed, 1)
            out.scheduled.append(Scheduled(r, r.num_computed, 1, True))
            scheduled_ids.add(r.request_id)
            budget -= 1
        # 2. requests in their prompt (or recomputing after giving up their pages), oldest first
        for r in sorted((r for r in self.running if r.num_computed < r.num_tokens - 1), key=lambda r: r.arrival):
            if budget < 1:
                break
            n = self._fit(r, r.num_computed, min(r.num_tokens - r.num_computed, budget))
            if n < 1:
                continue
            self.cache.reserve(r.request_id, r.num_computed, n)
            out.scheduled.append(Scheduled(r, r.num_computed, n, r.num_computed + n == r.num_tokens))
            scheduled_ids.add(r.request_id)
            budget -= n
        # 3. admission, in order of arrival, while a slot is free and the free pages hold the whole request
        while self.waiting and budget >= 1 and self.cache.has_slot() and not out.preempted:
            r = self.waiting[0]
            if not self.cache.can_hold(r.num_tokens, self.budget):
                break
            self.cache.admit(r.request_id)
            n = min(r.num_tokens, budget)
            self.waiting.popleft()
            r.status = Status.RUNNING
            self.running.append(r)
            self.cache.reserve(r.request_id, 0, n)
            out.scheduled.append(Scheduled(r, 0, n, n == r.num_tokens))
            scheduled_ids.add(r.request_id)
            budget -= n
        # 4. nothing can move: the newest running request gives way to the oldest; with nothing running, the
        #    head of the queue does not fit even alone
        if not out.scheduled and not out.preempted:
            if len(self.running) > 1:
                self._preempt(max(self.running, key=lambda v: v.arrival), out)
                again = self.schedule()
                again.preempted = out.preempted + again.preempted
                return again
            if self.running or self.waiting:
                r = self.running[0] if self.running else self.waiting.popleft()
                if self.running:
                    self.cache.free(r.request_id)
                    self.running.remove(r)
                r.status = Status.FINISHED
                r.finish_reason = "no_room"
                out.finished.append(r)
        return out

    # ------------------------------------------------------------------ after the step
    def update(self, scheduled: Sequence[Scheduled], tokens: Sequence[int | None],
               logprobs: Sequence[float | None]) -> list[Request]:
        """Records the step: `tokens[i]` is the token drawn for scheduled[i] (None if it did not sample).
        Returns the requests that finished; what they held has been given back."""
        finished = []
        for s, tok, lp in zip(scheduled, tokens, logprobs):
            r = s.request
            r.num_computed = s.start + s.num_tokens
            if not s.samples:
                continue
            r.output_token_ids.append(int(tok))
            r.output_token_logprobs.append(float(lp))
            # simply/utils/ragged_paged_attention.py:1921-1944 (has_ended)
            if not r.params.ignore_eos and int(tok) in r.eos_ids:
                r.finish_reason = "eos"
            elif len(r.output_token_ids) >= r.params.max_decode_steps:
                r.finish_reason = "length"
            elif r.num_tokens >= self._limit(r):
                r.finish_reason = "max_seq_len"
            if r.finish_reason is not None:
                r.status = Status.FINISHED
                self.cache.free(r.request_id)
                self.running.remove(r)
                finished.append(r)
        return finished
