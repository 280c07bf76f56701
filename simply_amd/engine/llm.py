"""The Python entry point: token ids in, generated token ids out.

Shaped after `LMInterface.generate` (simply/model_lib.py:4579-4942) and its `SamplingOutput`
(simply/model_lib.py:4461-4480), but over the paged cache and continuous batching of
simply/serving/page_batcher.py.  The engine takes and returns token ids; text is out of its scope.
"""
from __future__ import annotations

import dataclasses
import time
from typing import Sequence

import torch

from ..config import EngineConfig, load_config
from ..sampling import Sampler, SamplingParams, ScoringParams, request_seed
from .executor import Executor, StepEntry
from .loading import load_model, random_model
from .scheduler import Request, Scheduled, Scheduler, Status


@dataclasses.dataclass(frozen=True)
class SamplingOutput:
    """simply/model_lib.py:4461-4480, the fields that exist without a tokenizer."""

    input_token_ids: list[int]
    output_token_ids: list[int]
    output_token_logprobs: list[float]
    is_truncated: bool
    finish_reason: str
    num_preemptions: int = 0

    @property
    def sum_output_logprob(self) -> float:
        return float(sum(self.output_token_logprobs))

    @property
    def avg_output_logprob(self) -> float:
        return self.sum_output_logprob / max(len(self.output_token_logprobs), 1)


RequestOutput = SamplingOutput


class LMInterface:
    """A model with weights, a cache, a scheduler and a sampler on one GPU.

    model: a model folder (config.json, model.safetensors); or `config` (a typed architecture
    configuration) together with `random_weights` (a seed) for weights drawn on the device.
    The other arguments are the serving knobs of simply/serving/common_flags.py by their names there.
    """

    def __init__(self, model: str | None = None, *, config=None, random_weights: int | None = None,
                 activation_dtype: str = "bfloat16", batch_size: int = 8, max_seq_len: int | None = None,
                 page_size: int = 16, max_num_issue_tokens: int = 2048, total_num_pages: int | None = None,
                 windowed_num_pages: int | None = None, memory_fraction: float | None = None, seed: int = 0, device: str = "cuda:0", poison_freed_pages: bool = False, use_graphs: bool = True,
                 intermediate_steps: int = 64, _model=None):
        from ..kernels import lib

        lib.load()  # fails here, loudly, if the kernel library is missing and cannot be built
        dtype = EngineConfig(activation_dtype=activation_dtype).dtype
        if _model is not None:       # a model that is already on the device (several engines over one set of weights)
            self.model, self.model_config = _model, config
        elif model is not None:
            self.model, self.model_config = load_model(model, dtype, torch.device(device))
        elif config is not None and random_weights is not None:
            self.model_config = config
            self.model = random_model(config, random_weights, dtype, torch.device(device))
        else:
            raise ValueError("give a model folder, or a configuration and a seed for random weights")
        if max_seq_len is None:
            max_seq_len = self.model.spec.max_position
        self.engine_config = EngineConfig(
            activation_dtype=activation_dtype, page_size=page_size, batch_size=batch_size, max_seq_len=max_seq_len,
            max_num_issue_tokens=max_num_issue_tokens, total_num_pages=total_num_pages,
            windowed_num_pages=windowed_num_pages, memory_fraction=memory_fraction,
            intermediate_steps=max(1, int(intermediate_steps)), device=device,
            poison_freed_pages=poison_freed_pages, use_graphs=use_graphs)
        self.executor = Executor(self.model, self.engine_config)
        self.scheduler = Scheduler(self.executor.cache, max_num_issue_tokens=self.engine_config.issue_budget,
                                   max_seq_len=max_seq_len)
        self.sampler = Sampler(device, max(batch_size, 1))
        # decode steps that may run in a row without a new scheduling decision (simply/serving/common_flags.py:84
        # --intermediate_steps, 1024 there, in a loop on the device that ends when a request has ended); here the
        # host reads every step's tokens a few steps behind the device and ends the run when a request has ended
        self.intermediate_steps = max(1, int(intermediate_steps))
        self.seed = int(seed)
        self._num_requests = 0
        self._num_scored = 0
        self.stats = {"steps": 0, "tokens": 0, "preemptions": 0, "seconds": 0.0}
        #: set to a list to have every call of `step` add (decode steps it ran or 0 for a step with a portion of a
        #: prompt, tokens, seconds): the host has the step's tokens when the call returns, so these are latencies
        self.step_log: list[tuple[int, int, float]] | None = None

    # ------------------------------------------------------------------ requests
    def adopt_request(self, request_id, prompt_token_ids: Sequence[int], num_computed: int,
                      params: SamplingParams | None = None) -> Request:
        """A request whose first `num_computed` tokens are taken as run already: the cache's pages are reserved as
        that run would have left them and hold whatever the caller has put there.  For measurements of decode steps
        over a long context without the prompts that would have written it; what is generated then depends on what
        the pages hold."""
        r = self._new_request(request_id, prompt_token_ids, params)
        self.scheduler.adopt(r, num_computed)
        self.executor.adopt(r.request_id, num_computed)
        return r

    def add_request(self, request_id, prompt_token_ids: Sequence[int], params: SamplingParams | None = None) -> Request:
        r = self._new_request(request_id, prompt_token_ids, params)
        self.scheduler.add(r)
        return r

    def _new_request(self, request_id, prompt_token_ids: Sequence[int], params: SamplingParams | None) -> Request:
        params = params or SamplingParams()
        seed = params.seed if params.seed is not None else request_seed(self.seed, self._num_requests)
        self._num_requests += 1
        vocab = self.model.spec.vocab_size
        ids = [int(t) for t in prompt_token_ids]
        if any(t < 0 or t >= vocab for t in ids):
            raise ValueError(f"request {request_id!r}: token id outside [0, {vocab})")
        return Request(request_id, ids, params, seed=seed, eos_ids=tuple(self.model.spec.eos_token_ids))

    def step(self, max_decode_steps: int | None = None) -> list[Request]:
        """One scheduling decision and one run of the step function; when every scheduled request is decoding and
        nothing waits for admission, up to `intermediate_steps` (and `max_decode_steps`) decode steps in a row
        without the host in between.  Returns the requests that finished."""
        t0 = time.perf_counter()
        out = self.scheduler.schedule()
        self.stats["preemptions"] += len(out.preempted)
        finished = list(out.finished)
        if not out.scheduled:
            return finished
        entries = []
        for s in out.scheduled:
            toks = s.request.tokens(s.start, s.num_tokens)
            entries.append(StepEntry(s.request.request_id, toks, [s.num_tokens - 1] if s.samples else [], s.start))
        n = self._decode_steps_ahead(out.scheduled, max_decode_steps)
        if n > 1:
            reqs = [s.request for s in out.scheduled]
            self.sampler.stage([r.params for r in reqs], [r.seed for r in reqs], [len(r.output_token_ids) for r in reqs])
            index = {id(s): i for i, s in enumerate(out.scheduled)}
            live = list(out.scheduled)
            ran = [0]

            def on_step(k, step_tokens, step_logprobs) -> bool:
                """A step's results have reached the host (later steps may be running already): the scheduler takes
                them; the steps in a row go on while nobody has finished."""
                nonlocal live
                if not live:
                    return False
                now = [Scheduled(s.request, s.start + k, 1, True) for s in live]
                done = self.scheduler.update(now, [step_tokens[index[id(s)]] for s in live],
                                             [step_logprobs[index[id(s)]] for s in live])
                finished.extend(done)
                live = [s for s in live if s.request.status is Status.RUNNING]
                self.stats["steps"] += 1
                self.stats["tokens"] += len(now)
                ran[0] += 1
                return bool(live) and not done

            self.executor.decode_many(entries, n, self.sampler, on_step=on_step)
            if self.step_log is not None:
                self.step_log.append((ran[0], ran[0] * len(entries), time.perf_counter() - t0))
            return finished
        logits = self.executor.step(entries)
        tokens: list = [None] * len(entries)
        logprobs: list = [None] * len(entries)
        rows = [i for i, s in enumerate(out.scheduled) if s.samples]
        if rows:
            reqs = [out.scheduled[i].request for i in rows]
            toks, lps = self.sampler.sample(logits, [r.params for r in reqs], [r.seed for r in reqs],
                                            [len(r.output_token_ids) for r in reqs])
            for i, t, lp in zip(rows, toks, lps):
                tokens[i], logprobs[i] = t, lp
        finished += self.scheduler.update(out.scheduled, tokens, logprobs)
        self.stats["steps"] += 1
        self.stats["tokens"] += out.num_tokens
        if self.step_log is not None:
            # a decode step: every token that went in is one that the model had generated
            decode_only = all(s.start >= len(s.request.prompt_token_ids) for s in out.scheduled)
            self.step_log.append((1 if decode_only else 0, out.num_tokens, time.perf_counter() - t0))
        return finished

    def _decode_steps_ahead(self, scheduled, max_decode_steps: int | None) -> int:
        """How many decode steps may run in a row now: more than one only if every scheduled request decodes, nothing
        waits, none of them would pass its own limits, and the free pages hold all of it."""
        n = self.intermediate_steps if max_decode_steps is None else min(self.intermediate_steps, max_decode_steps)
        if n <= 1 or self.scheduler.waiting or any(s.num_tokens != 1 or not s.samples for s in scheduled):
            return 1
        if len(scheduled) != len(self.scheduler.running):
            return 1   # someone is still in its prompt
        for s in scheduled:
            r = s.request
            n = min(n, r.params.max_decode_steps - len(r.output_token_ids), self.scheduler._limit(r) - r.num_tokens)
        while n > 1 and not self.executor.cache.can_reserve([(s.request.request_id, s.start, n) for s in scheduled]):
            n //= 2
        return max(n, 1)

    # ------------------------------------------------------------------ generate
    def generate(self, input_token_ids: Sequence[int] | Sequence[Sequence[int]], prng_key: int | None = None,
                 sampling_params: SamplingParams | Sequence[SamplingParams] | None = None) -> list[SamplingOutput]:
        """Generates a continuation for each input (a list of token ids, or a list of such lists).
        `prng_key`, if given, replaces the engine's seed for requests whose params carry none."""
        single = len(input_token_ids) > 0 and isinstance(input_token_ids[0], int)
        inputs = [input_token_ids] if single else list(input_token_ids)
        if isinstance(sampling_params, SamplingParams) or sampling_params is None:
            plist = [sampling_params or SamplingParams()] * len(inputs)
        else:
            plist = list(sampling_params)
            if len(plist) != len(inputs):
                raise ValueError("one SamplingParams per input, or one for all")
        if prng_key is not None:
            self.seed, self._num_requests = int(prng_key), 0
        t0 = time.perf_counter()
        requests = [self.add_request(("gen", id(inputs), i), ids, p) for i, (ids, p) in enumerate(zip(inputs, plist))]
        while self.scheduler.has_work():
            self.step()
        self.stats["seconds"] += time.perf_counter() - t0
        return [SamplingOutput(list(r.prompt_token_ids), list(r.output_token_ids), list(r.output_token_logprobs),
                               r.is_truncated, r.finish_reason or "", r.num_preemptions) for r in requests]


    # ------------------------------------------------------------------ score
    def score_tokens(self, tokens: Sequence[int], scoring_params: ScoringParams | None = None) -> list[float]:
        """The log-likelihood of tokens[1:], each given the tokens before it (simply/model_lib.py:4995-5036:
        the model runs on tokens[:-1], the scores are `compute_log_likelihood` of simply/utils/sampling_lib.py:540-601
        under the scoring parameters' temperature, top-k and top-p).  The tokens go through the step function in
        portions, as a request of their own beside whatever else is live; logits of a portion are scored on the
        device and only the scores come back."""
        from ..kernels import ops

        sp = scoring_params or ScoringParams()
        sp.validate()
        vocab = self.model.spec.vocab_size
        ids = [int(t) for t in tokens]
        if any(t < 0 or t >= vocab for t in ids):
            raise ValueError(f"score_tokens: token id outside [0, {vocab})")
        n = len(ids) - 1
        if n < 1:
            return []
        if n > self.engine_config.max_seq_len:
            raise ValueError(f"score_tokens: {n} tokens to run, max_seq_len is {self.engine_config.max_seq_len}")
        ex, dev = self.executor, self.executor.device
        # logits of a portion: float32 [rows, vocab], 256 MiB at most
        rows = max(1, min(self.engine_config.issue_budget, (64 << 20) // vocab))
        self._num_scored += 1
        rid = ("score", self._num_scored)
        out = []
        ex.add_request(rid)
        try:
            for i in range(0, n, rows):
                part = ids[i:min(i + rows, n)]
                logits = ex.step([StepEntry(rid, part, list(range(len(part))))])
                given = torch.tensor(ids[i + 1:i + 1 + len(part)], dtype=torch.int32, device=dev)
                full = lambda v, dt: torch.full((len(part),), v, dtype=dt, device=dev)
                out.append(ops.score(logits, full(sp.temperature, torch.float32), full(sp.top_k, torch.int32),
                                     full(sp.top_p, torch.float32), given))
        finally:
            ex.finish_request(rid)
        return torch.cat(out).tolist()


LLM = LMInterface
