"""The cache manager: paged keys and values with a block table per request, one
page pool per group of layers, and fixed-size state slots.

Layers are grouped by what they need to keep: all keys ("full") or the last W
of them ("window", one group per W).  Each group has its own pool of pages and
each request its own block table per group; all caches of a group share the
page ids, so one table serves every layer of the group (the reference keeps a
page list per layer, reference: src/backend/kvcache/block_pool.hpp:73-103).
Pages go back to the pool when the request ends, or, in a window group, as soon
as no later token can see them.  A page holds ``page_size`` tokens of one layer,
in the tensors the layer's mixer asked for (``KVCacheRequest.tensors``: names,
shapes of one page, types): the manager allocates them and hands them over by
name and knows nothing of what they hold (the reference's page is keys and values
as [slot][kv_head][head_dim], block_pool.hpp:16-25).

Admission works on promises: ``open`` promises a sequence the pages its prompt
and a reserve of generated tokens need (reference: prompt + min(max_new, 256),
src/zedinfer/scheduler.cpp:109-129) and fails when the pool cannot promise
them.  Pages are taken when tokens arrive.  A sequence that grows past its
promise takes unpromised pages while there are any and fails with OutOfPages
when there are none (reference: "KV cache exhausted during decode",
scheduler.cpp:293-319).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..config.forward_config import ScheduleStep
from ..parts.base import KVCacheRequest, LayerMemory, StateRequest
from .pages import IdPool, OutOfPages, PagePool


@dataclass
class CacheGroup:
    kind: str                      # "full" or "window"
    window: int                    # 0 for full
    page_size: int
    pool: PagePool
    caches: Dict[int, KVCacheRequest] = field(default_factory=dict)    # cache id -> what its layer asked for

    def pages_for(self, tokens: int) -> int:
        return (tokens + self.page_size - 1) // self.page_size

    def promise_for(self, tokens: int, max_step_tokens: int) -> int:
        """Most pages a sequence of ``tokens`` tokens holds at once in this group."""
        n = self.pages_for(tokens)
        if self.kind == "window":
            n = min(n, self.pages_for(self.window - 1 + max(max_step_tokens, 1)) + 1)
        return n

    def first_live_page(self, length: int) -> int:
        """First logical page a token at position >= length can still see."""
        if self.kind != "window":
            return 0
        return max(0, length - self.window + 1) // self.page_size


@dataclass
class Growth:
    """What one ``CacheManager.ensure`` took for a sequence."""

    taken: List[Tuple[int, int]]      # (group, logical page) of every page taken
    grown: List[int]                  # promises added per group, beyond what admission promised
    old_lens: List[int]               # the block tables' lengths before


NO_GROWTH = Growth(taken=[], grown=[], old_lens=[])      # what ``ensure`` returns when it took nothing


class SequenceCache:
    """What one live request holds: a state slot and, per group, its block table."""

    def __init__(self, request_id, slot: int, num_groups: int):
        self.request_id = request_id
        self.slot = slot
        self.length = 0                                     # tokens whose keys are in the cache
        self.pages: List[List[int]] = [[] for _ in range(num_groups)]   # logical page -> page id or -1
        self.held: List[int] = [0] * num_groups
        self.promised: List[int] = [0] * num_groups
        self.closed = False
        self.version = 0          # grows whenever a block table of the sequence changes


class CacheManager:
    def __init__(self, kv_requests: Dict[int, KVCacheRequest], state_requests: Dict[int, StateRequest],
                 num_pages: int, page_size: int, max_requests: int, dtype: torch.dtype,
                 device: Optional[torch.device | str], max_step_tokens: int = 1):
        """``device`` None keeps the manager host-only (no tensors), for tests of the bookkeeping."""
        if page_size <= 0 or num_pages <= 0 or max_requests <= 0:
            raise ValueError("cache: page_size, num_pages and max_requests must be positive")
        self.page_size = int(page_size)
        self.num_pages = int(num_pages)
        self.max_requests = int(max_requests)
        self.max_step_tokens = int(max_step_tokens)
        self.dtype = dtype
        self.device = torch.device(device) if device is not None else None
        self.groups: List[CacheGroup] = []
        self.group_of_cache: Dict[int, int] = {}
        keys: Dict[Tuple[str, int], int] = {}
        for cid in sorted(kv_requests):
            rq = kv_requests[cid]
            if rq.kind not in ("full", "window") or (rq.kind == "window" and rq.window <= 0):
                raise ValueError(f"cache {cid}: unknown cache kind {rq.kind!r} / window {rq.window}")
            key = (rq.kind, rq.window if rq.kind == "window" else 0)
            if key not in keys:
                keys[key] = len(self.groups)
                self.groups.append(CacheGroup(rq.kind, key[1], self.page_size, PagePool(self.num_pages)))
            g = keys[key]
            self.groups[g].caches[cid] = rq
            self.group_of_cache[cid] = g
        self.slots = IdPool(self.max_requests, "state slot")
        self.live: Dict[object, SequenceCache] = {}
        self.tensors: Dict[int, Dict[str, torch.Tensor]] = {}      # cache id -> name -> [pages, *page shape]
        self.state: Dict[int, torch.Tensor] = {}
        self.state_requests = dict(state_requests)
        if self.device is not None:
            for cid, rq in kv_requests.items():
                self.tensors[cid] = {name: torch.zeros((self.num_pages,) + pt.page_shape(self.page_size),
                                                       dtype=pt.dtype or dtype, device=self.device)
                                     for name, pt in rq.tensors}
            for cid, sr in state_requests.items():
                self.state[cid] = torch.zeros((self.max_requests,) + tuple(sr.shape), dtype=sr.dtype,
                                              device=self.device)

    # ---- sizes -------------------------------------------------------------------
    @staticmethod
    def bytes_per_page(kv_requests: Dict[int, KVCacheRequest], page_size: int, dtype: torch.dtype) -> int:
        """Device bytes one page id costs over all caches."""
        total = 0
        for r in kv_requests.values():
            for _, pt in r.tensors:
                n = 1
                for s in pt.page_shape(page_size):
                    n *= s
                total += n * torch.empty((), dtype=pt.dtype or dtype).element_size()
        return total

    def memories(self, schedule: Sequence[ScheduleStep]) -> List[LayerMemory]:
        out = []
        for st in schedule:
            g = self.group_of_cache.get(st.cache, -1)
            out.append(LayerMemory(group=g, tensors=self.tensors.get(st.cache, {}), writes=st.writes_cache,
                                   state=self.state.get(st.cache)))
        return out

    # ---- admission ---------------------------------------------------------------
    def can_open(self, expected_tokens: int) -> bool:
        if self.slots.num_free < 1:
            return False
        return all(g.pool.uncommitted >= g.promise_for(expected_tokens, self.max_step_tokens)
                   for g in self.groups)

    def open(self, request_id, expected_tokens: int = 0) -> SequenceCache:
        """Admit a sequence and promise it pages for ``expected_tokens`` tokens."""
        if request_id in self.live:
            raise ValueError(f"request {request_id!r} already holds a cache")
        want = [g.promise_for(expected_tokens, self.max_step_tokens) for g in self.groups]
        for g, n in zip(self.groups, want):
            if g.pool.uncommitted < n:
                raise OutOfPages(f"request {request_id!r} needs {n} pages of the {g.kind} group, "
                                 f"{g.pool.uncommitted} of {g.pool.total} are unpromised")
        slot = self.slots.take()
        seq = SequenceCache(request_id, slot, len(self.groups))
        for i, (g, n) in enumerate(zip(self.groups, want)):
            g.pool.commit(n)
            seq.promised[i] = n
        for cid, st in self.state.items():
            st[slot].zero_()
        self.live[request_id] = seq
        return seq

    # ---- growth ------------------------------------------------------------------
    def _release_passed(self, seq: SequenceCache) -> None:
        for gi, g in enumerate(self.groups):
            if g.kind != "window":
                continue
            first = min(g.first_live_page(seq.length), len(seq.pages[gi]))
            table = seq.pages[gi]
            for i in range(first):
                if table[i] >= 0:
                    g.pool.give_back(table[i])
                    table[i] = -1
                    seq.held[gi] -= 1
                    seq.version += 1

    def ensure(self, seq: SequenceCache, new_len: int) -> "Growth":
        """Make sure pages exist for every position below ``new_len`` that a token at or after
        ``seq.length`` can see.  All or nothing: on OutOfPages nothing has changed.  Returns what was
        taken, which ``undo`` gives back (a step that cannot grow a later request undoes the earlier ones);
        NO_GROWTH when nothing was (a decoded token inside its page: most calls, which therefore make no
        objects)."""
        if seq.closed:
            raise ValueError(f"request {seq.request_id!r} is closed")
        if new_len < seq.length:
            raise ValueError("a cache cannot shrink")
        self._release_passed(seq)
        growth = None
        try:
            for gi, g in enumerate(self.groups):
                table = seq.pages[gi]
                last = (new_len - 1) // g.page_size if new_len > 0 else -1
                if len(table) <= last:
                    if growth is None:
                        growth = Growth(taken=[], grown=[0] * len(self.groups), old_lens=[len(t) for t in seq.pages])
                    while len(table) <= last:
                        table.append(-1)
                for i in range(g.first_live_page(seq.length), last + 1):
                    if table[i] >= 0:
                        continue
                    if growth is None:
                        growth = Growth(taken=[], grown=[0] * len(self.groups), old_lens=[len(t) for t in seq.pages])
                    if seq.held[gi] + 1 > seq.promised[gi]:
                        if g.pool.uncommitted < 1:
                            raise OutOfPages(
                                f"request {seq.request_id!r} needs another page of the {g.kind} group "
                                f"and all {g.pool.total} are promised")
                        g.pool.commit(1)
                        seq.promised[gi] += 1
                        growth.grown[gi] += 1
                    table[i] = g.pool.take()
                    seq.held[gi] += 1
                    seq.version += 1
                    growth.taken.append((gi, i))
        except OutOfPages:
            self.undo(seq, growth)
            raise
        return growth if growth is not None else NO_GROWTH

    def undo(self, seq: SequenceCache, growth: "Growth") -> None:
        """Give back what one ``ensure`` took (pages, promises beyond the admission's, table rows), before
        anything was committed on top of it."""
        if growth is NO_GROWTH:
            return
        for gi, i in growth.taken:
            self.groups[gi].pool.give_back(seq.pages[gi][i])
            seq.pages[gi][i] = -1
            seq.held[gi] -= 1
        for gi, n in enumerate(growth.grown):
            self.groups[gi].pool.uncommit(n)
            seq.promised[gi] -= n
        for gi, n in enumerate(growth.old_lens):
            del seq.pages[gi][n:]
        seq.version += 1

    def commit(self, seq: SequenceCache, new_len: int) -> None:
        """The tokens below ``new_len`` are in the cache now; give back what no later token sees."""
        if new_len < seq.length:
            raise ValueError("a cache cannot shrink")
        seq.length = new_len
        self._release_passed(seq)

    def close(self, seq: SequenceCache) -> None:
        """Give back everything the sequence holds."""
        if seq.closed:
            raise ValueError(f"request {seq.request_id!r} is closed twice")
        for gi, g in enumerate(self.groups):
            for p in seq.pages[gi]:
                if p >= 0:
                    g.pool.give_back(p)
            seq.pages[gi] = []
            seq.held[gi] = 0
            seq.version += 1
            g.pool.uncommit(seq.promised[gi])
            seq.promised[gi] = 0
        self.slots.give_back(seq.slot)
        seq.closed = True
        del self.live[seq.request_id]

    # ---- views for a step --------------------------------------------------------
    def token_slots(self, seq: SequenceCache, group: int, start: int, count: int) -> np.ndarray:
        """Cache slot (page * page_size + offset) of positions start..start+count-1."""
        g = self.groups[group]
        pos = np.arange(start, start + count, dtype=np.int64)
        table = np.asarray(seq.pages[group], dtype=np.int64)
        pages = table[pos // g.page_size]
        if (pages < 0).any():
            raise RuntimeError(f"request {seq.request_id!r}: a position in [{start}, {start + count}) has no page")
        return (pages * g.page_size + pos % g.page_size).astype(np.int32)

    def check(self) -> None:
        """Every page is free or held by exactly one live sequence; counts agree."""
        for gi, g in enumerate(self.groups):
            g.pool.check()
            seen = set()
            for seq in self.live.values():
                n = 0
                for p in seq.pages[gi]:
                    if p < 0:
                        continue
                    if p in seen:
                        raise AssertionError(f"page {p} of group {gi} is held twice")
                    if not g.pool.is_held(p):
                        raise AssertionError(f"page {p} of group {gi} is in a table but free")
                    seen.add(p)
                    n += 1
                if n != seq.held[gi]:
                    raise AssertionError("a sequence's held count disagrees with its table")
                if seq.held[gi] > seq.promised[gi]:
                    raise AssertionError("a sequence holds more than it was promised")
            if len(seen) != g.pool.num_held:
                raise AssertionError(f"group {gi}: {g.pool.num_held} pages held, {len(seen)} in tables (a page is lost)")
            if sum(s.promised[gi] for s in self.live.values()) != g.pool.committed:
                raise AssertionError(f"group {gi}: promises do not add up")
        self.slots.check()
        if {s.slot for s in self.live.values()} != {i for i in range(self.slots.total) if self.slots.is_held(i)}:
            raise AssertionError("state slots and live sequences disagree")
