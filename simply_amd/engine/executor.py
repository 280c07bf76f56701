"""The step function: one ragged batch through the model, from the cache.

`Executor.step` takes, for each request, its next tokens and the places among them whose logits
are wanted; it runs only those tokens, as one batch, and returns float32 logits at the wanted
places.  It corresponds to the forward half of `SamplingState.mixed_step`
(simply/utils/ragged_paged_attention.py:1954-2019); choosing which tokens to run is the
scheduler's job and sampling is the sampler's.
"""
from __future__ import annotations

import dataclasses
from typing import Hashable, Sequence

import numpy as np
import torch

from ..cache import CacheManager, pages_for_memory
from ..config import EngineConfig
from ..models import DecoderModel
from .context import GroupStep, StepContext


@dataclasses.dataclass
class StepEntry:
    request_id: Hashable
    tokens: Sequence[int]                 # the request's next tokens
    want: Sequence[int] = ()              # places among `tokens` whose logits are wanted
    start: int | None = None              # position of tokens[0]; None: right after the tokens run so far


class Executor:
    def __init__(self, model: DecoderModel, config: EngineConfig, *, num_pages: int | None = None):
        config.validate()
        if not model.loaded:
            raise RuntimeError("the model has no weights yet")
        self.model, self.config = model, config
        self.device = torch.device(config.device)
        self.dtype = config.dtype
        needs = model.cache_needs()
        pages = num_pages if num_pages is not None else config.total_num_pages
        if pages is None and config.memory_fraction is not None and self.device.type == "cuda":
            # what is free now, the weights being loaded; the kernels' workspace and a step's buffers come off first
            from ..kernels import ops

            free, _ = torch.cuda.mem_get_info(self.device)
            reserve = ops.WORKSPACE_BYTES + 8 * config.batch_size * model.spec.vocab_size + (256 << 20)
            pages = pages_for_memory(needs, page_size=config.page_size, num_slots=config.batch_size,
                                     max_seq_len=config.max_seq_len, max_step_tokens=config.max_step_tokens,
                                     esize=torch.empty((), dtype=self.dtype).element_size(),
                                     budget_bytes=int(free * config.memory_fraction) - reserve)
        if pages is None:
            pages = config.batch_size * -(-config.max_seq_len // config.page_size)
        windowed = config.windowed_num_pages
        self.cache = CacheManager(needs, page_size=config.page_size, num_pages=pages,
                                  num_slots=config.batch_size, max_seq_len=config.max_seq_len, dtype=self.dtype,
                                  device=self.device, poison=config.poison_freed_pages,
                                  max_step_tokens=config.max_step_tokens,
                                  group_pages=None if windowed is None else
                                  (lambda need, n: windowed if getattr(need, "window", None) is not None else n))
        self.num_computed: dict[Hashable, tuple[int, int]] = {}  # request -> (admission, tokens run)
        self.vocab_size = model.spec.vocab_size
        # one pinned staging buffer and one device buffer for all of a step's integers
        cap = max(config.issue_budget, config.batch_size)
        self._cap = cap
        ngroups = len(self.cache.groups)
        self._meta_at = cap * (4 + 2 * ngroups)          # [batch_size, 4] request descriptors after the token arrays
        self._words = self._meta_at + 4 * config.batch_size
        self._on_gpu = self.device.type == "cuda"
        self._host = torch.empty(self._words, dtype=torch.int32, pin_memory=self._on_gpu)
        self._dev = torch.empty(self._words, dtype=torch.int32, device=self.device)
        self._copied = torch.cuda.Event() if self._on_gpu else None
        # a second pinned block for integer arrays that parts make for a step (the units of an attention kernel):
        # a step's arrays lie one behind the other in it
        self._extra_words = 4 * (cap + 8 * config.batch_size)
        self._extra_host = torch.empty(self._extra_words, dtype=torch.int32, pin_memory=True) if self._on_gpu else None
        self._extra_dev = torch.empty(self._extra_words, dtype=torch.int32, device=self.device) if self._on_gpu else None
        self._extra_copied = torch.cuda.Event() if self._on_gpu else None
        self._extra_used = 0
        # decode-only steps (one token per request) are captured once per number of requests and order of magnitude
        # of the context (the attention kernels choose their cut of the keys when they are recorded) and replayed
        self._graphs: dict[tuple, torch.cuda.CUDAGraph] = {}
        self._graph_pool = None
        # where every recorded step writes its logits, [batch_size, vocab] float32: made at the first such step
        self._graph_logits: torch.Tensor | None = None
        # several decode steps in a row without the host (decode_many): what was drawn in each, and the step count
        self._records: tuple[torch.Tensor, ...] | None = None
        self._side_stream = None    # on which results of steps in a row travel to the host while later steps run

    # ------------------------------------------------------------------ requests
    def add_request(self, rid: Hashable) -> int:
        """Admits a request to the cache (a scheduler may do that itself on `self.cache`)."""
        return self.cache.admit(rid)

    def finish_request(self, rid: Hashable) -> None:
        self.cache.free(rid)

    def adopt(self, rid: Hashable, num_computed: int) -> None:
        """Records that the cache already holds the keys of the request's first `num_computed` tokens (the request
        is admitted and its pages are reserved: `Scheduler.adopt`); its next portion may start there."""
        if rid not in self.cache.requests:
            raise KeyError(f"request {rid!r} has not been admitted to the cache")
        self.num_computed[rid] = (self.cache.admission[rid], int(num_computed))

    def has_request(self, rid: Hashable) -> bool:
        return rid in self.cache.requests

    def _start_of(self, e: "StepEntry") -> int:
        admission, done = self.num_computed.get(e.request_id, (0, 0))
        if admission != self.cache.admission[e.request_id]:
            done = 0  # the request has given up its pages and come back since
        if e.start is None:
            return done
        if e.start > done:
            raise ValueError(f"request {e.request_id!r}: a portion starting at {e.start} would leave positions "
                             f"{done}..{e.start - 1} without keys")
        return e.start

    def _replay(self, T: int, ctx: StepContext, logit_rows: torch.Tensor) -> torch.Tensor:
        """A decode-only step through a captured HIP graph.  Everything that differs between two such steps
        with the same number of requests (tokens, positions, slots, block tables) lies in buffers at fixed
        addresses that the kernels read, so the launches can be recorded once.  The returned logits lie in a buffer
        that all recorded steps share: the next decode-only step overwrites them.  A step runs exactly once: the
        first step with a new key runs eagerly (kernels choose their plans, scratch buffers get allocated) and is
        this call's result; the recording that follows executes nothing (a mixer that keeps a state of its own would
        otherwise advance it twice)."""
        key = (T, self._context_bucket(ctx))
        ctx.kv_bound = 1 << key[1]
        out = self._shared_logits()[:T]
        graph = self._graphs.get(key)
        if graph is not None:
            graph.replay()
            return out
        logits = self.model.forward(self._dev[:T], ctx, self.cache.views, logit_rows, logits_out=out)
        self._graphs[key] = self._record(
            lambda: self.model.forward(self._dev[:T], ctx, self.cache.views, logit_rows, logits_out=out))
        return logits

    def _shared_logits(self) -> torch.Tensor:
        if self._graph_logits is None:
            self._graph_logits = torch.empty((self.config.batch_size, self.vocab_size), dtype=torch.float32,
                                             device=self.device)
        return self._graph_logits

    def _record(self, run) -> "torch.cuda.CUDAGraph":
        """Records the launches of `run()` in a HIP graph, executing none of them."""
        torch.cuda.synchronize(self.device)
        graph = torch.cuda.CUDAGraph()
        if self._graph_pool is None:
            self._graph_pool = torch.cuda.graph_pool_handle()
        with torch.cuda.graph(graph, pool=self._graph_pool):
            run()
        return graph

    @staticmethod
    def _context_bucket(ctx: StepContext, ahead: int = 0) -> int:
        """Recorded steps are kept per power of two of the longest context: a recording serves every step (and, with
        `ahead` further steps in a row, every run of steps) whose longest context stays within 2 ** bucket keys, and
        its kernels are planned for that many (`StepContext.kv_bound`)."""
        return max(ctx.max_kv_len + ahead - 1, 0).bit_length()

    # ------------------------------------------------------------------ the step
    def step(self, entries: Sequence[StepEntry]) -> torch.Tensor | None:
        """Runs the entries as one batch.  Returns float32 logits [wanted, vocab] in the order of the
        entries and of their `want`, or None if nothing is wanted."""
        prepared = self._prepare(entries)
        if prepared is None:
            return None
        T, R, ctx, logit_rows, wants, num_entries = prepared
        decode_only = (self._on_gpu and self.config.use_graphs and all(q == 1 for q in ctx.q_lens)
                       and R == num_entries)
        if decode_only:
            logits = self._replay(T, ctx, logit_rows)
        else:
            logits = self.model.forward(self._dev[:T], ctx, self.cache.views, logit_rows)
        for rid, start, q in wants:
            self.num_computed[rid] = (self.cache.admission[rid], start + q)
        self.cache.mark_issued(wants)
        return logits

    def decode_many(self, entries: Sequence[StepEntry], num_steps: int, sampler, on_step=None, lookahead: int = 8,
                    chunk: int = 4) -> tuple[list[list[int]], list[list[float]]]:
        """Up to `num_steps` decode steps in a row for requests that bring one token each (after
        `SamplingState.continue_decode`, simply/utils/ragged_paged_attention.py:2065-2103, which loops on the device
        until `until_fn` holds or `intermediate_steps` have run): every step's drawn tokens are the next step's
        input, on the device.  `sampler` has been staged (`Sampler.stage`) with one row per entry, in the entries'
        order.  Pages for all the steps are reserved first (`OutOfPages` if they do not fit).

        `on_step(k, tokens, logprobs) -> bool`, if given, is called for every step, in order, as its results reach
        the host, while up to `lookahead` later steps are already launched (results come out in chunks of `chunk`
        steps, copied on a stream of their own); once it returns False no further step is launched, and the steps
        already launched still finish and are delivered.  That is the device loop's `until_fn` with the host's
        view of the requests: a request that ends runs at most `lookahead + chunk` steps too many, all other rows of
        those steps are ordinary tokens.  Without `on_step` all steps run and the host comes back in once.
        Returns (tokens, logprobs) of the steps that ran, each [step][entry]."""
        entries = list(entries)
        if any(len(e.tokens) != 1 or list(e.want) != [0] for e in entries):
            raise ValueError("decode_many: every request brings one token whose logits are wanted")
        B = len(entries)
        if not (self._on_gpu and self.config.use_graphs) or num_steps == 1:
            # step by step through the host (no graphs: the CPU stand-in of the tests, or a single step)
            tokens, logprobs = [], []
            for k in range(num_steps):
                logits = self.step(entries)
                toks, lps = sampler.launch(logits)
                tokens.append(toks[:B].tolist())
                logprobs.append(lps[:B].tolist())
                sampler.draw_counters[:B] += 1
                if on_step is not None and not on_step(k, tokens[-1], logprobs[-1]):
                    break
                entries = [StepEntry(e.request_id, [t], [0]) for e, t in zip(entries, tokens[-1])]
            return tokens, logprobs
        prepared = self._prepare(entries, reserve_ahead=num_steps)
        T, R, ctx, logit_rows, wants, _ = prepared
        assert T == B == R and ctx.request_ids == [e.request_id for e in entries]  # rows, tokens and entries line up
        cap, dev = self._cap, self._dev
        if self._records is None or self._records[0].numel() < num_steps * cap:
            room = max(num_steps, 64)   # recorded graphs hold these addresses: made once for any usual run
            self._records = (torch.empty(room * cap, dtype=torch.int32, device=self.device),
                             torch.empty(room * cap, dtype=torch.float32, device=self.device),
                             torch.zeros(1, dtype=torch.int32, device=self.device),
                             torch.empty(room * cap, dtype=torch.int32, pin_memory=True),
                             torch.empty(room * cap, dtype=torch.float32, pin_memory=True))
            self._graphs = {k: v for k, v in self._graphs.items() if k[0] != "many"}  # they hold the old addresses
        rec_tok, rec_lp, counter, host_tok, host_lp = self._records
        max_steps = rec_tok.numel() // cap
        out_tok, out_lp = rec_tok[:max_steps * B].view(max_steps, B), rec_lp[:max_steps * B].view(max_steps, B)
        from ..kernels import ops

        shared = self._shared_logits()[:T]

        def one_step():
            logits = self.model.forward(dev[:T], ctx, self.cache.views, logit_rows, logits_out=shared)
            toks, lps = sampler.launch(logits)
            groups = [(ctx.groups[g.group_id].block_table, ctx.groups[g.group_id].slot_mapping) for g in self.cache.groups]
            # what was drawn becomes the next step's input, positions move on, and every cache group learns where
            # the next keys go: one launch for up to four groups
            ops.decode_advance(counter, toks, lps, dev[:T], dev[cap:cap + T], ctx.seq_meta, sampler.draw_counters,
                               out_tok, out_lp, token_seq=dev[2 * cap:2 * cap + T], page_size=self.cache.page_size,
                               groups=groups[:4])
            for table, slots in groups[4:]:
                ops.decode_slots(dev[cap:cap + T], dev[2 * cap:2 * cap + T], table, self.cache.page_size, slots)

        ops.fill_(counter, 0)
        key = ("many", B, self._context_bucket(ctx, num_steps - 1), max_steps, id(sampler), sampler.modes)
        ctx.kv_bound = 1 << key[2]
        graph = self._graphs.get(key)
        launched = 0
        if graph is None:
            one_step()   # once eagerly (it counts as the first step), then recorded
            launched = 1
            graph = self._graphs[key] = self._record(one_step)
        if on_step is None:
            lookahead = chunk = num_steps
        if self._side_stream is None:
            self._side_stream = torch.cuda.Stream(device=self.device)
        side = self._side_stream
        pending: list[tuple[int, int, torch.cuda.Event]] = []   # steps [a, b) on their way to the host
        copied = read = 0
        go = True
        tokens, logprobs = [], []

        def copy_out(upto: int) -> int:
            reached = torch.cuda.Event()
            reached.record()
            side.wait_event(reached)
            with torch.cuda.stream(side):
                host_tok[copied * B:upto * B].copy_(rec_tok[copied * B:upto * B], non_blocking=True)
                host_lp[copied * B:upto * B].copy_(rec_lp[copied * B:upto * B], non_blocking=True)
                arrived = torch.cuda.Event()
                arrived.record(side)
            pending.append((copied, upto, arrived))
            return upto

        while True:
            while go and launched < num_steps and launched - read < max(lookahead, 1):
                if launched - copied >= chunk:
                    copied = copy_out(launched)
                graph.replay()
                launched += 1
            if copied < launched and (launched - copied >= chunk or not go or launched == num_steps):
                copied = copy_out(launched)
            if not pending:
                break
            a, b, arrived = pending.pop(0)
            arrived.synchronize()
            toks, lps = host_tok[a * B:b * B].view(b - a, B).tolist(), host_lp[a * B:b * B].view(b - a, B).tolist()
            for k in range(a, b):
                tokens.append(toks[k - a])
                logprobs.append(lps[k - a])
                if on_step is not None and not on_step(k, tokens[-1], logprobs[-1]):
                    go = False
            read = b
        for rid, start, _ in wants:
            if rid in self.cache.requests:   # (not one that `on_step` has finished and freed meanwhile)
                self.num_computed[rid] = (self.cache.admission[rid], start + launched)
        self.cache.mark_issued([(rid, start, launched) for rid, start, _ in wants if rid in self.cache.requests])
        return tokens, logprobs

    def _to_device(self, array: np.ndarray) -> torch.Tensor:
        """An int32 array of the step on the device, through the pinned block if it still fits: the copy does not
        wait for the device, so the stream keeps its lead over the launches."""
        words = array.size
        if not self._on_gpu or array.dtype != np.int32 or self._extra_used + words > self._extra_words:
            return torch.from_numpy(np.ascontiguousarray(array)).to(self.device)
        at = self._extra_used
        if at == 0:
            self._extra_copied.synchronize()  # the last step's copies out of the block have finished
        self._extra_used = at + words
        self._extra_host.numpy()[at:at + words] = array.reshape(-1)
        dev = self._extra_dev[at:at + words]
        dev.copy_(self._extra_host[at:at + words], non_blocking=True)
        self._extra_copied.record()
        return dev.view(array.shape)

    def _prepare(self, entries: Sequence[StepEntry], reserve_ahead: int = 1):
        """Checks the entries, reserves their pages (for `reserve_ahead` tokens where an entry brings one token
        and more steps follow without the host), lays the step out in the staging buffer and copies it to the
        device.  Returns (tokens, wanted rows, context, wanted-row indices on the device, [(request, start,
        tokens reserved)], number of entries), or None for an empty step."""
        entries = [e for e in entries if len(e.tokens) > 0]
        T = sum(len(e.tokens) for e in entries)
        if T == 0:
            return None
        if T > self._cap:
            raise ValueError(f"a step of {T} tokens exceeds max_num_issue_tokens {self._cap}")
        seen = set()
        for e in entries:
            if e.request_id in seen:
                raise ValueError(f"request {e.request_id!r} appears twice in one step")
            seen.add(e.request_id)
            if e.request_id not in self.cache.requests:
                raise KeyError(f"request {e.request_id!r} has not been admitted to the cache")
        cache, cap = self.cache, self._cap
        # forget what is known of requests that have left the cache since (finished or preempted elsewhere)
        for rid in [r for r in self.num_computed if r not in self.cache.requests]:
            del self.num_computed[rid]
        # requests with few tokens first (the attention kernels take them as one range); `order` remembers
        # where each entry went so that the logits come back in the callers' order
        order = sorted(range(len(entries)), key=lambda i: len(entries[i].tokens))
        if len(entries) > self.config.batch_size:
            raise ValueError(f"{len(entries)} requests in one step, batch_size is {self.config.batch_size}")
        # make room for every entry first: nothing is reserved unless all of it fits
        wants = [(e.request_id, self._start_of(e), max(len(e.tokens), reserve_ahead)) for e in entries]
        cache.reserve_all(wants)

        if self._copied is not None:
            self._copied.synchronize()  # the last step's copy out of the staging buffer has finished
        host = self._host.numpy()
        tok, pos, seq, rows = (host[i * cap:(i + 1) * cap] for i in range(4))
        slot_maps = [host[(4 + 2 * g) * cap:(6 + 2 * g) * cap].view(np.int64) for g in range(len(cache.groups))]
        meta = host[self._meta_at:self._meta_at + 4 * len(entries)].reshape(len(entries), 4)
        ctx_ids, ctx_slots, ctx_starts, ctx_q, cu = [], [], [], [], [0]
        first_token = [0] * len(entries)
        t0 = 0
        for j, i in enumerate(order):
            e, (rid, start, reserved) = entries[i], wants[i]
            q = len(e.tokens)
            slot = cache.slot_of(rid)
            if q == 1:  # a decoded token: no arrays
                ids = int(e.tokens[0])
                bad = not 0 <= ids < self.vocab_size
                pos[t0] = start
            else:
                ids = np.asarray(e.tokens, dtype=np.int64)
                bad = ids.min() < 0 or ids.max() >= self.vocab_size
                pos[t0:t0 + q] = np.arange(start, start + q)
            if bad:
                raise ValueError(f"request {rid!r}: token id outside [0, {self.vocab_size})")
            tok[t0:t0 + q] = ids
            seq[t0:t0 + q] = slot
            meta[j] = (slot, t0, q, start)
            for g in cache.groups:
                slot_maps[g.group_id][t0:t0 + q] = cache.slot_mapping(g.group_id, rid, start, q)
                cache.check_readable(g.group_id, rid, start, reserved)
            first_token[i] = t0
            ctx_ids.append(rid); ctx_slots.append(slot); ctx_starts.append(start); ctx_q.append(q)
            t0 += q
            cu.append(t0)
        R = 0
        for i, e in enumerate(entries):
            q = len(e.tokens)
            for w in e.want:
                if not 0 <= w < q:
                    raise ValueError(f"request {e.request_id!r}: wanted place {w} is outside its {q} tokens")
                rows[R] = first_token[i] + w
                R += 1
        tables = cache.sync_tables()
        self._dev.copy_(self._host, non_blocking=True)
        if self._copied is not None:
            self._copied.record()
        dev = self._dev
        groups = {g.group_id: GroupStep(tables[g.group_id],
                                        dev[(4 + 2 * g.group_id) * cap:(6 + 2 * g.group_id) * cap].view(torch.int64)[:T])
                  for g in cache.groups}
        ctx = StepContext(dtype=self.dtype, num_tokens=T, positions=dev[cap:cap + T], token_seq=dev[2 * cap:2 * cap + T],
                          seq_meta=dev[self._meta_at:self._meta_at + 4 * len(entries)].view(len(entries), 4),
                          groups=groups, request_ids=ctx_ids, seq_slots=ctx_slots, seq_starts=ctx_starts, q_lens=ctx_q,
                          cu_q_lens=cu, to_device=self._to_device)
        self._extra_used = 0
        logit_rows = dev[3 * cap:3 * cap + R] if R else None
        return T, R, ctx, logit_rows, [(rid, start, len(e.tokens)) for (rid, start, _), e in zip(wants, entries)], \
            len(entries)
