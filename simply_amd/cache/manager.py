"""The cache manager: pages of keys and values with a block table per request, in groups of
layers with the same needs, and slots for per-request state of fixed size.

After simply/utils/ragged_paged_attention.py: `DecodeState` keeps a page pool, a free stack and
`page_indices` per layer (:142-173); `allocate` (:475-518) pops pages from the front of the free
stack, `release` (:521-541) and `release_for_window` (:437-472) push pages back at its end; layers
with the same (pages, page size, window) share the bookkeeping (:865-917).  Differences: the
bookkeeping lives on the host, a block table is indexed by the absolute block number of a key
(position // page_size) so that a windowed group leaves holes instead of shifting its table, and
running out of pages is reported to the caller instead of being excluded by construction.
Every group has a pool of its own size: a windowed group's holds what its requests can hold at
once (`windowed_pool_pages`), as the reference sizes its local pool by the window (:95-110,
simply/serving/page_server.py:180-196).

Bookkeeping is separate from storage: `CacheManager(device=None)` keeps no tensors and runs
anywhere.  The manager counts pages and slots only; what a page or a slot holds, and in which layout, is
said by the need that a mixer declares (simply_amd/parts/base.py: `PagedNeed.page_tensors`,
`StateNeed.slot_tensor`), as the reference keys its groups by what a layer needs
(simply/utils/ragged_paged_attention.py:865-867) and leaves the tensors to the layer.
"""
from __future__ import annotations

import collections
import dataclasses
from typing import Hashable, Sequence

import numpy as np
import torch


class CacheError(RuntimeError):
    pass


class OutOfPages(CacheError):
    """Raised by `reserve` when a group cannot hold the tokens; nothing has been changed."""


def ceil_div(a: int, b: int) -> int:
    return -(-a // b)


def windowed_pool_pages(window: int, page_size: int, num_slots: int, max_step_tokens: int) -> int:
    """The most pages that `num_slots` requests of a group with this window hold at once.  A request that has run
    c tokens and brings q more holds blocks floor((c - window + 1) / P) .. ceil((c + q) / P) - 1, at most
    (window - 1 + q) / P + 2 of them; the q of one step add up to max_step_tokens at most.  (The reference,
    whose steps never hold more than the window, has ceil(window / P) + 1 per request:
    simply/utils/ragged_paged_attention.py:95-110.)"""
    return num_slots * (ceil_div(max(window - 1, 0), page_size) + 2) + ceil_div(max_step_tokens, page_size)


def pages_for_memory(needs, *, page_size: int, num_slots: int, max_seq_len: int, max_step_tokens: int, esize: int,
                     budget_bytes: int) -> int:
    """How many pages a group that keeps every token gets when `budget_bytes` of device memory go to the cache:
    the windowed groups take what their requests can hold at once, the others share the rest page for page; never
    more than `num_slots` sequences of `max_seq_len` need, at least one sequence's worth of one page.  `needs` as
    `CacheManager` takes them."""
    per_page_full = per_page_windowed_total = 0
    for need, cache_from in needs:
        if cache_from is not None or not callable(getattr(need, "page_tensors", None)):
            continue
        page_bytes = need.bytes_per_token(esize) * page_size
        window = getattr(need, "window", None)
        if window is None:
            per_page_full += page_bytes
        else:
            per_page_windowed_total += page_bytes * windowed_pool_pages(window, page_size, num_slots, max_step_tokens)
    most = num_slots * ceil_div(max_seq_len, page_size)
    if per_page_full == 0:
        return most
    return int(max(1, min(most, (int(budget_bytes) - per_page_windowed_total) // per_page_full)))


class PagePool:
    """Free pages of one group, handed out from the front and taken back at the end
    (simply/utils/ragged_paged_attention.py:495-511, 530-535)."""

    def __init__(self, num_pages: int):
        self.num_pages = int(num_pages)
        self._free = collections.deque(range(self.num_pages))
        self._is_free = np.ones(self.num_pages, dtype=bool)

    @property
    def num_free(self) -> int:
        return len(self._free)

    def free_list(self) -> list[int]:
        return list(self._free)

    def take(self, n: int) -> list[int]:
        if n > len(self._free):
            raise OutOfPages(f"{n} pages wanted, {len(self._free)} free")
        out = [self._free.popleft() for _ in range(n)]
        self._is_free[out] = False
        return out

    def give_back(self, pages: Sequence[int]) -> None:
        for p in pages:
            if not 0 <= p < self.num_pages:
                raise CacheError(f"page {p} does not exist")
            if self._is_free[p]:
                raise CacheError(f"page {p} freed twice")
            self._is_free[p] = True
            self._free.append(p)


@dataclasses.dataclass
class _Sequence:
    slot: int
    num_tokens: int = 0       # tokens whose keys have a place (prompt and generated)
    first_block: int = 0      # blocks below this one have been given back (windowed groups)


class CacheGroup:
    """Pages and block tables of the layers whose paged needs are equal."""

    def __init__(self, group_id: int, need, page_size: int, num_pages: int, num_slots: int,
                 max_blocks_per_seq: int):
        self.group_id, self.need = group_id, need
        #: None: every token's page is kept; n: pages that lie wholly before the last n tokens are given back
        self.window = getattr(need, "window", None)
        self.page_size, self.num_slots, self.max_blocks = int(page_size), int(num_slots), int(max_blocks_per_seq)
        self.pool = PagePool(num_pages)
        #: table[slot, absolute block] = page, -1 where no page is held
        self.table = np.full((self.num_slots, self.max_blocks), -1, dtype=np.int32)
        self.seqs: dict[Hashable, _Sequence] = {}
        self.dirty_slots: set[int] = set()

    # -- what a step would need
    def dead_blocks(self, num_computed: int) -> int:
        """Blocks that no query at position >= num_computed can see (windowed groups only):
        the first visible key is num_computed - window + 1
        (simply/utils/ragged_paged_attention.py:441-445 with window_size = window - 1)."""
        if self.window is None:
            return 0
        return max(num_computed - self.window + 1, 0) // self.page_size

    def pages_needed(self, rid: Hashable, num_computed: int, q_len: int) -> int:
        """New pages for tokens [num_computed, num_computed + q_len), net of those that become free first."""
        s = self.seqs[rid]
        have_to = ceil_div(s.num_tokens, self.page_size)
        need_to = ceil_div(num_computed + q_len, self.page_size)
        released = max(min(self.dead_blocks(num_computed), have_to) - s.first_block, 0)
        return max(need_to - have_to, 0) - released

    # -- changes
    def add(self, rid: Hashable, slot: int) -> None:
        if rid in self.seqs:
            raise CacheError(f"request {rid!r} is already in group {self.group_id}")
        self.seqs[rid] = _Sequence(slot)

    def new_blocks(self, rid: Hashable, new_num_tokens: int) -> int:
        """Pages that `extend(rid, new_num_tokens)` would take."""
        s = self.seqs[rid]
        return max(ceil_div(new_num_tokens, self.page_size) - ceil_div(s.num_tokens, self.page_size), 0)

    def releasable(self, rid: Hashable, num_computed: int | None) -> int:
        """Pages that `release_window(rid, num_computed)` would give back."""
        s = self.seqs[rid]
        return max(min(self.dead_blocks(num_computed), ceil_div(s.num_tokens, self.page_size)) - s.first_block, 0)

    def release_window(self, rid: Hashable, num_computed: int) -> list[int]:
        s = self.seqs[rid]
        dead = min(self.dead_blocks(num_computed), ceil_div(s.num_tokens, self.page_size))
        if dead <= s.first_block:
            return []
        pages = [int(p) for p in self.table[s.slot, s.first_block:dead]]
        self.table[s.slot, s.first_block:dead] = -1
        s.first_block = dead
        self.pool.give_back(pages)
        self.dirty_slots.add(s.slot)
        return pages

    def extend(self, rid: Hashable, new_num_tokens: int) -> list[int]:
        s = self.seqs[rid]
        have_to = ceil_div(s.num_tokens, self.page_size)
        need_to = ceil_div(new_num_tokens, self.page_size)
        if need_to > self.max_blocks:
            raise CacheError(f"request {rid!r}: {new_num_tokens} tokens need {need_to} blocks, the table has "
                             f"{self.max_blocks}")
        pages = self.pool.take(max(need_to - have_to, 0))
        if pages:
            self.table[s.slot, have_to:need_to] = pages
            self.dirty_slots.add(s.slot)
        s.num_tokens = max(s.num_tokens, new_num_tokens)
        return pages

    def remove(self, rid: Hashable) -> list[int]:
        s = self.seqs.pop(rid)
        row = self.table[s.slot]
        pages = [int(p) for p in row[row >= 0]]
        row[:] = -1
        self.pool.give_back(pages)
        self.dirty_slots.add(s.slot)
        return pages

    def pages_of(self, rid: Hashable) -> list[int]:
        s = self.seqs[rid]
        row = self.table[s.slot]
        return [int(p) for p in row[row >= 0]]

    def check(self) -> None:
        """Invariants: every page is free or held by exactly one request, never both or twice."""
        held = self.table[self.table >= 0]
        if len(np.unique(held)) != len(held):
            raise CacheError(f"group {self.group_id}: a page is held twice")
        free = self.pool.free_list()
        if len(set(free)) != len(free):
            raise CacheError(f"group {self.group_id}: a page is in the free list twice")
        if set(free) & set(int(p) for p in held):
            raise CacheError(f"group {self.group_id}: a page is both free and held")
        if len(free) + len(held) != self.pool.num_pages:
            raise CacheError(f"group {self.group_id}: {self.pool.num_pages - len(free) - len(held)} pages lost")
        live_slots = {s.slot for s in self.seqs.values()}
        for slot in range(self.num_slots):
            if slot not in live_slots and (self.table[slot] >= 0).any():
                raise CacheError(f"group {self.group_id}: slot {slot} has pages but no request")


class StateSlots:
    """Slots for per-request state of fixed size; the slot also selects the request's block-table row
    (the batch slot of simply/utils/ragged_paged_attention.py:1448-1462)."""

    def __init__(self, num_slots: int):
        self.num_slots = int(num_slots)
        self._free = list(range(self.num_slots - 1, -1, -1))
        self.owner: dict[int, Hashable] = {}

    @property
    def num_free(self) -> int:
        return len(self._free)

    def take(self, rid: Hashable) -> int:
        if not self._free:
            raise CacheError("no free state slot")
        slot = self._free.pop()
        self.owner[slot] = rid
        return slot

    def give_back(self, slot: int) -> None:
        if slot not in self.owner:
            raise CacheError(f"state slot {slot} freed twice")
        del self.owner[slot]
        self._free.append(slot)
        self._free.sort(reverse=True)


@dataclasses.dataclass
class CacheView:
    """What one schedule entry's mixer is handed: its own storage (or that of the entry it reads)."""

    need: object | None
    group_id: int | None = None
    #: the page tensors that the need asked for, by the need's own names (first dimension: pages of the group's pool)
    pages: dict = dataclasses.field(default_factory=dict)
    state: torch.Tensor | None = None     # [num_slots, ...] as the need's `slot_tensor` made it
    write: bool = True                    # False: this entry reads the cache of another entry

    @property
    def k_pages(self) -> torch.Tensor | None:
        """Key pages of a `PagedKVNeed`: [num_pages, kv heads, page_size, head_dim]."""
        return self.pages.get("k")

    @property
    def v_pages(self) -> torch.Tensor | None:
        """Value pages of a `PagedKVNeed`: [num_pages, kv heads, head_dim, page_size]."""
        return self.pages.get("v")


class CacheManager:
    """All groups, the state slots and (if `device` is given) the storage.

    needs: one `(need, cache_from)` per schedule entry, as `DecoderModel.cache_needs()` returns.
    """

    def __init__(self, needs, *, page_size: int, num_pages: int, num_slots: int, max_seq_len: int,
                 dtype: torch.dtype = torch.float32, device=None, poison: bool = False,
                 max_step_tokens: int | None = None, group_pages=None):
        """num_pages: pages of a group that keeps every key.  A windowed group gets the fewer pages that its
        requests can hold at once when a step brings at most `max_step_tokens` tokens (None: as many as the
        others).  group_pages: a function (need, default number) -> number, for a group with a pool of another
        size."""
        self.page_size, self.num_pages, self.num_slots = int(page_size), int(num_pages), int(num_slots)
        self.max_seq_len, self.dtype, self.device, self.poison = int(max_seq_len), dtype, device, bool(poison)
        self.slots = StateSlots(num_slots)
        self.groups: list[CacheGroup] = []
        self.requests: dict[Hashable, int] = {}
        #: a number that is new for every admission (a request that comes back after giving up its pages gets another)
        self.admission: dict[Hashable, int] = {}
        self._admissions = 0
        #: per request the number of its tokens whose step has been handed to the GPU (`mark_issued`): the queries
        #: still to come start there, so a window's pages below what they see can go
        self.issued: dict[Hashable, int] = {}
        self.views: list[CacheView] = []
        self._group_entries: dict[int, list[int]] = {}
        self._device_tables: dict[int, torch.Tensor] = {}
        self._stage_host = self._stage_dev = self._stage_done = None  # what `sync_tables` sends its rows through
        by_need: dict[object, CacheGroup] = {}
        max_blocks = ceil_div(self.max_seq_len, self.page_size)
        for i, (need, cache_from) in enumerate(needs):
            if cache_from is not None:
                src = self.views[cache_from]
                if type(src.need) is not type(need) or src.need != need:
                    raise CacheError(f"schedule entry {i} reads the cache of entry {cache_from}, whose need differs: "
                                     f"{need} vs {src.need}")
                self.views.append(dataclasses.replace(src, write=False))
                continue
            if need is None:
                self.views.append(CacheView(None))
            elif callable(getattr(need, "page_tensors", None)):
                # something per token, in pages: layers with equal needs share pool, free list and block table
                group = by_need.get(need)
                if group is None:
                    pages = self.num_pages
                    window = getattr(need, "window", None)
                    if window is not None and max_step_tokens is not None:
                        pages = min(pages, windowed_pool_pages(window, self.page_size, self.num_slots,
                                                               int(max_step_tokens)))
                    if group_pages is not None:
                        pages = int(group_pages(need, pages))
                    group = CacheGroup(len(self.groups), need, self.page_size, pages, self.num_slots, max_blocks)
                    by_need[need] = group
                    self.groups.append(group)
                    self._group_entries[group.group_id] = []
                view = CacheView(need, group.group_id)
                if device is not None:
                    n = group.pool.num_pages
                    view.pages = dict(need.page_tensors(n, self.page_size, dtype, device,
                                                        float("nan") if poison else 0.0))
                    for name, t in view.pages.items():
                        if t.dim() < 1 or t.shape[0] != n:
                            raise CacheError(f"schedule entry {i}: page tensor {name!r} of {need!r} has shape "
                                             f"{tuple(t.shape)}; its first dimension must be the {n} pages")
                self._group_entries[group.group_id].append(i)
                self.views.append(view)
            elif callable(getattr(need, "slot_tensor", None)):
                # something of fixed size per request: a row per request slot
                view = CacheView(need)
                if device is not None:
                    view.state = need.slot_tensor(self.num_slots, device)
                    if view.state.dim() < 1 or view.state.shape[0] != self.num_slots:
                        raise CacheError(f"schedule entry {i}: the state of {need!r} has shape "
                                         f"{tuple(view.state.shape)}; its first dimension must be the {self.num_slots} slots")
                self.views.append(view)
            else:
                raise CacheError(f"schedule entry {i}: cache need {need!r} says neither page_tensors(...) (something "
                                 f"per token) nor slot_tensor(...) (something of fixed size per request)")
        if device is not None:
            for g in self.groups:
                self._device_tables[g.group_id] = torch.full((self.num_slots, g.max_blocks), -1, dtype=torch.int32,
                                                             device=device)

    # ------------------------------------------------------------------ requests
    def has_slot(self) -> bool:
        return self.slots.num_free > 0

    def admit(self, rid: Hashable) -> int:
        """Takes a state slot and an empty block-table row in every group; zeroes the request's state."""
        if rid in self.requests:
            raise CacheError(f"request {rid!r} is already admitted")
        slot = self.slots.take(rid)
        self.requests[rid] = slot
        self._admissions += 1
        self.admission[rid] = self._admissions
        self.issued[rid] = 0
        for g in self.groups:
            g.add(rid, slot)
        for v in self.views:
            if v.state is not None and v.write:
                v.state[slot].zero_()
        return slot

    def slot_of(self, rid: Hashable) -> int:
        return self.requests[rid]

    def pages_needed(self, rid: Hashable, num_computed: int, q_len: int) -> dict[int, int]:
        return {g.group_id: g.pages_needed(rid, num_computed, q_len) for g in self.groups}

    def _release_points(self, wants: Sequence[tuple[Hashable, int, int]]) -> dict[Hashable, int]:
        """For every live request the position from which its next queries look back: where its tokens of this
        step begin, or, for a request that this step leaves out, the end of what has been handed to the GPU."""
        points = dict(self.issued)
        for rid, nc, _ in wants:
            points[rid] = nc
        return points

    def mark_issued(self, wants: Sequence[tuple[Hashable, int, int]]) -> None:
        """The step that `reserve_all(wants)` made room for has been handed to the GPU (in stream order before
        anything that a later step writes): the requests' next queries begin behind it."""
        for rid, nc, q in wants:
            if rid in self.issued:
                self.issued[rid] = nc + q

    def can_reserve(self, wants: Sequence[tuple[Hashable, int, int]]) -> bool:
        """Whether every group can hold all of `wants` = (request, num_computed, q_len) together, once every live
        request, in the step or not, has given back the pages that its window has passed (`reserve_all` does it in
        that order)."""
        points = self._release_points(wants)
        for g in self.groups:
            free = g.pool.num_free
            if g.window is not None:
                free += sum(g.releasable(rid, at) for rid, at in points.items())
            if sum(g.new_blocks(rid, nc + q) for rid, nc, q in wants) > free:
                return False
        return True

    def can_hold(self, num_tokens: int, max_step_tokens: int) -> bool:
        """Whether the free pages of every group hold a new request of `num_tokens` tokens that runs in steps of at
        most `max_step_tokens`: all of its pages in a group that keeps every key, the most it ever holds at once
        in a windowed one."""
        points = self._release_points(())
        for g in self.groups:
            peak = ceil_div(num_tokens, self.page_size)
            free = g.pool.num_free
            if g.window is not None:
                step = min(num_tokens, max(int(max_step_tokens), 1))
                peak = min(peak, ceil_div(g.window - 1 + step, self.page_size) + 1)
                free += sum(g.releasable(rid, at) for rid, at in points.items())
            if peak > free:
                return False
        return True

    def reserve_all(self, wants: Sequence[tuple[Hashable, int, int]]) -> None:
        """Makes room for the tokens [num_computed, num_computed + q_len) of every (request, num_computed, q_len) in
        every group: all of it or, with OutOfPages, nothing.  The pages that windows have passed are given back
        first, by every live request (also those that the step leaves out: what they hold beyond their window
        is of no use to anyone), then the new ones are taken: a request whose window frees pages makes room for
        another wherever the two stand in `wants`."""
        for rid, nc, q in wants:
            if nc + q > self.max_seq_len:
                raise CacheError(f"request {rid!r}: {nc + q} tokens exceed max_seq_len {self.max_seq_len}")
        if not self.can_reserve(wants):
            raise OutOfPages("the cache cannot hold this step's tokens: " + ", ".join(
                f"{rid!r}+{q}" for rid, _, q in wants) + "; free pages per group: " + ", ".join(
                str(g.pool.num_free) for g in self.groups))
        points = self._release_points(wants)
        for rid, nc, _ in wants:
            self.issued[rid] = min(self.issued[rid], nc)    # its queries from nc on are still to come
        for g in self.groups:
            if g.window is not None:
                for rid, at in points.items():
                    self._poison(g, g.release_window(rid, at))
            for rid, nc, q in wants:
                g.extend(rid, nc + q)

    def reserve(self, rid: Hashable, num_computed: int, q_len: int) -> None:
        """`reserve_all` for one request."""
        self.reserve_all([(rid, num_computed, q_len)])

    def free(self, rid: Hashable) -> None:
        """Gives back everything the request holds."""
        slot = self.requests.pop(rid)
        del self.admission[rid]
        del self.issued[rid]
        for g in self.groups:
            self._poison(g, g.remove(rid))
        self.slots.give_back(slot)

    def _poison(self, g: CacheGroup, pages: Sequence[int]) -> None:
        """Fills pages that were just given back with NaN (in stream order: after the steps that read
        them, before the step that writes them again), so that a read of an unwritten key shows."""
        if not (self.poison and self.device is not None and pages):
            return
        idx = torch.as_tensor(list(pages), dtype=torch.long, device=self.device)
        for e in self._group_entries[g.group_id]:
            for t in self.views[e].pages.values():
                if t.is_floating_point():
                    t[idx] = float("nan")

    def check(self) -> None:
        for g in self.groups:
            g.check()
            if set(g.seqs) != set(self.requests):
                raise CacheError(f"group {g.group_id} and the manager disagree on the live requests")
        if set(self.slots.owner.values()) != set(self.requests):
            raise CacheError("state slots and the manager disagree on the live requests")

    # ------------------------------------------------------------------ what a step reads
    def slot_mapping(self, group_id: int, rid: Hashable, start: int, q_len: int) -> np.ndarray:
        """Storage slot (page * page_size + offset) of positions [start, start + q_len)."""
        g = self.groups[group_id]
        if q_len == 1:  # a decoded token: plain integers
            page = int(g.table[g.seqs[rid].slot, start // g.page_size])
            if page < 0:
                raise CacheError(f"request {rid!r}: position {start} has no page in group {group_id}")
            return np.array([page * g.page_size + start % g.page_size], dtype=np.int64)
        pos = np.arange(start, start + q_len, dtype=np.int64)
        pages = g.table[g.seqs[rid].slot, pos // g.page_size].astype(np.int64)
        if (pages < 0).any():
            raise CacheError(f"request {rid!r}: a position in [{start}, {start + q_len}) has no page in group {group_id}")
        return pages * g.page_size + pos % g.page_size

    def check_readable(self, group_id: int, rid: Hashable, start: int, q_len: int) -> None:
        """Every key that the queries at [start, start + q_len) may read has a page."""
        g = self.groups[group_id]
        lo = 0 if g.window is None else max(start - g.window + 1, 0)
        blocks = g.table[g.seqs[rid].slot, lo // g.page_size: ceil_div(start + q_len, g.page_size)]
        if (blocks < 0).any():
            raise CacheError(f"request {rid!r}: keys [{lo}, {start + q_len}) are not all held in group {group_id}")

    def sync_tables(self) -> dict[int, torch.Tensor]:
        """Brings the device copies of the block tables up to date.  The rows that have changed go through a pinned
        block in one copy that does not wait for the device, and are put into place there: a step's launches can
        then follow the last step's without the stream running empty in between."""
        dirty = [g for g in self.groups if g.dirty_slots] if self.device is not None else []
        if dirty and torch.device(self.device).type != "cuda":
            for g in dirty:
                rows = sorted(g.dirty_slots)
                self._device_tables[g.group_id].index_copy_(0, torch.as_tensor(rows, dtype=torch.long),
                                                            torch.from_numpy(g.table[rows]))
        elif dirty:
            if self._stage_host is None:
                ints = sum(self.num_slots * (g.max_blocks + 3) for g in self.groups)
                self._stage_host = torch.empty(ints, dtype=torch.int32, pin_memory=True)
                self._stage_dev = torch.empty(ints, dtype=torch.int32, device=self.device)
                self._stage_done = torch.cuda.Event()
            self._stage_done.synchronize()  # the last copy out of the pinned block has finished
            host, dev = self._stage_host.numpy(), self._stage_dev
            at, parts = 0, []
            for g in dirty:
                rows = sorted(g.dirty_slots)
                n, body = len(rows), at + 2 * len(rows)  # the rows' numbers as 64-bit integers, then the rows
                host[at:body].view(np.int64)[:] = rows
                host[body:body + n * g.max_blocks].reshape(n, g.max_blocks)[:] = g.table[rows]
                parts.append((g, at, n, body))
                at = body + n * g.max_blocks
                at += at & 1
            dev[:at].copy_(self._stage_host[:at], non_blocking=True)
            self._stage_done.record()
            for g, first, n, body in parts:
                self._device_tables[g.group_id].index_copy_(0, dev[first:body].view(torch.int64),
                                                            dev[body:body + n * g.max_blocks].view(n, g.max_blocks))
        for g in self.groups:
            g.dirty_slots.clear()
        return self._device_tables

    def bytes_per_token(self) -> int:
        """Bytes of cache that one token takes over all schedule entries that keep their own."""
        esize = torch.empty((), dtype=self.dtype).element_size()
        return sum(v.need.bytes_per_token(esize) for v in self.views if v.group_id is not None and v.write)
