"""One step's batch: what the caller asks for, and its flattened device form.

A step takes, for each request in it, that request's next tokens (a portion of
its prompt, or one decoded token) and the places among them whose logits are
wanted.  All entries are flattened into one token list without padding
(reference: src/zedinfer/batch_context.cpp:21-85 builds the same flattened
ids/positions; there decode rows must come first, here any order works).

Nothing here knows a mixer.  What a mixer's kernels need beyond these arrays (how
attention divides the tokens between its kernels, for instance) comes from the
mixer's own ``StepPlanner``: its index arrays are packed into the same host buffer
and travel in the same copy.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence

import numpy as np
import torch

from ..cache.manager import CacheManager, SequenceCache
from ..ops.staging import StagingRing
from ..parts.base import HostBatch, StepPlan, StepPlanner


@dataclass
class StepEntry:
    """``tokens`` continue the sequence whose cache is ``seq`` at position ``seq.length``;
    ``want`` lists the places among ``tokens`` whose logits are returned.  ``positions`` (optional, for
    models whose position encoding has several axes): for each token its position on every axis;
    None: the token's index in its sequence on every axis."""

    seq: SequenceCache
    tokens: Sequence[int]
    want: Sequence[int] = ()
    positions: Optional[Sequence[Sequence[int]]] = None


@dataclass
class GroupView:
    slots: torch.Tensor          # [n] int32: where each token's keys and values go
    block_tables: torch.Tensor   # [entries, max_pages] int32, -1 where no page is held


@dataclass
class DeviceBatch:
    """The step as the parts see it.  Everything is int32 on the device."""

    num_tokens: int
    num_entries: int
    num_logit_rows: int
    token_ids: torch.Tensor      # [n]
    positions: torch.Tensor      # [n] index of each token in its sequence (its place in the cache)
    tok_seq: torch.Tensor        # [n] entry index of each token
    logit_rows: torch.Tensor     # [rows] flat token indices
    entry_start: torch.Tensor    # [entries] first flat token index of the entry
    entry_len: torch.Tensor      # [entries] tokens of the entry in this step
    entry_past: torch.Tensor     # [entries] tokens of the entry already in the cache
    entry_slot: torch.Tensor     # [entries] state slot of the entry
    groups: List[GroupView] = field(default_factory=list)
    # what position encodings with several axes read: [n, axes]; with one axis it is ``positions`` itself
    position_ids: Optional[torch.Tensor] = None
    # the plans of the mixers' planners, by planner key
    plans: Dict[tuple, StepPlan] = field(default_factory=dict)
    # host copies, for parts that plan their launches on the host
    host_start: Optional[np.ndarray] = None
    host_len: Optional[np.ndarray] = None
    host_past: Optional[np.ndarray] = None
    host_slot: Optional[np.ndarray] = None
    host_image: Optional[np.ndarray] = None      # all index arrays as they were copied to the device
    device_image: Optional[torch.Tensor] = None  # the device buffer that holds them (every array is a view of it)
    # every entry brings exactly one token (a pure decode step): no token's keys are written by
    # another token of the step, so a mixer may store and attend in one kernel
    single_tokens: bool = False
    # logits are wanted at every token, in order: nothing needs to be picked
    all_rows_wanted: bool = False
    # what parts compute once per step and share over the layers (for instance the rotation angles),
    # by a key of their own
    shared: dict = field(default_factory=dict)


FIXED_PIECES = 8      # token ids, positions, tok_seq, logit rows, entry start / len / past / slot


def build_device_batch(entries: Sequence[StepEntry], cache: CacheManager, vocab_size: int,
                       device: torch.device, staging: Optional[StagingRing] = None,
                       table_widths: Optional[Sequence[int]] = None,
                       static: Optional[torch.Tensor] = None, pad_to=None, pad_entries: int = 0,
                       pad_rows: int = 0, pad_more: int = 0, planners: Sequence[StepPlanner] = (), position_axes: int = 1,
                       bound_single: int = 0, bound_multi: int = 0) -> DeviceBatch:
    """Check the entries, then pack every index array into one host buffer and copy it over once.

    ``pad_to``: a function of a number of tokens; every entry that brings more than one token is run as if it
    brought ``pad_to(tokens)``.  The tokens past its own are token 0 at the positions that follow; they have no place in the cache
    (slot -1: nothing is stored for them) and no real token sees them, so they change nothing but the
    shapes, which then recur from step to step.  ``pad_more``: that many more such tokens behind the longest
    entry's.  ``pad_entries`` adds that many entries of one token that
    belong to no request (token 0 at position 0, no slot, an empty block table, state slot 0),
    ``pad_rows`` that many wanted rows after the real ones (the first token's), to the same end.  Only for
    models whose mixers all say ``padding_safe``.

    ``table_widths`` pads each group's block table to a given width; ``static`` is a device buffer
    the arrays are copied into instead of a fresh one (the layout depends only on the number of
    tokens, entries and wanted rows, on the table widths and on the sizes of the planners' arrays, so a
    captured graph that reads the arrays finds them at the same addresses every step; the buffer of a
    step built without ``static`` is ``device_image`` of the result and can serve as ``static`` for the
    next steps of the same shape).  ``planners``:
    the planners of the model's mixers, one per key; ``bound_single`` / ``bound_multi`` are handed to
    them (``HostBatch``).  ``position_axes``: the axes of the model's position encodings."""
    if not entries:
        raise ValueError("a step needs at least one entry")
    seen = set()
    lens = []
    for e in entries:
        if id(e.seq) in seen:
            raise ValueError(f"request {e.seq.request_id!r} appears twice in one step")
        seen.add(id(e.seq))
        if e.seq.closed:
            raise ValueError(f"request {e.seq.request_id!r} is closed")
        n = len(e.tokens)
        if n == 0:
            raise ValueError(f"request {e.seq.request_id!r} brings no tokens")
        for w in e.want:
            if not (0 <= w < n):
                raise ValueError(f"request {e.seq.request_id!r}: wanted place {w} is outside its {n} tokens")
        if e.positions is not None and (position_axes <= 1 or len(e.positions) != n):
            raise ValueError(f"request {e.seq.request_id!r}: positions need one row of {position_axes} axes for each "
                             f"of its {n} tokens, and a model whose position encoding has several axes")
        lens.append(n)
    E = len(entries) + int(pad_entries)
    lens = lens + [1] * int(pad_entries)
    real = list(lens)
    if pad_to:
        lens = [int(pad_to(n)) if n > 1 else n for n in lens]
        if any(a < b for a, b in zip(lens, real)):
            raise ValueError("padding cannot take tokens away")
    if pad_more:
        longest = max(range(len(lens)), key=lambda i: lens[i])
        if lens[longest] <= 1:
            raise ValueError("more padding needs an entry of several tokens to stand behind")
        lens[longest] += int(pad_more)
    N = int(sum(lens))
    starts = np.zeros(E, dtype=np.int32)
    starts[1:] = np.cumsum(lens)[:-1]
    past = np.array([e.seq.length for e in entries] + [0] * int(pad_entries), dtype=np.int32)
    slot = np.array([e.seq.slot for e in entries] + [0] * int(pad_entries), dtype=np.int32)
    lens_a = np.array(lens, dtype=np.int32)

    token_ids = np.concatenate([np.concatenate([np.asarray(e.tokens, dtype=np.int64), np.zeros(n - r, dtype=np.int64)])
                                for e, n, r in zip(entries, lens, real)] + [np.zeros(int(pad_entries), dtype=np.int64)])
    if token_ids.min() < 0 or token_ids.max() >= vocab_size:
        bad = token_ids[(token_ids < 0) | (token_ids >= vocab_size)][0]
        raise ValueError(f"token id {int(bad)} is outside the vocabulary of {vocab_size}")
    positions = np.concatenate([np.arange(p, p + n, dtype=np.int32) for p, n in zip(past, lens)])
    tok_seq = np.repeat(np.arange(E, dtype=np.int32), lens)
    rows = [starts[i] + w for i, e in enumerate(entries) for w in e.want] + [0] * int(pad_rows)
    logit_rows = np.asarray(rows, dtype=np.int32)
    R = len(rows)

    G = len(cache.groups)
    group_slots, group_tables, widths = [], [], []
    for g in range(G):
        group_slots.append(np.concatenate(
            [np.concatenate([cache.token_slots(e.seq, g, int(p), r), np.full(n - r, -1, dtype=np.int32)])
             for e, p, n, r in zip(entries, past, lens, real)] + [np.full(int(pad_entries), -1, dtype=np.int32)]))
        width = max(1, max(len(e.seq.pages[g]) for e in entries))
        if table_widths is not None:
            if table_widths[g] < width:
                raise ValueError(f"block tables of group {g} need {width} columns, {table_widths[g]} given")
            width = int(table_widths[g])
        t = np.full((E, width), -1, dtype=np.int32)
        for i, e in enumerate(entries):
            pg = e.seq.pages[g]
            t[i, :len(pg)] = pg
        group_tables.append(t)
        widths.append(width)

    single = bool((lens_a == 1).all())
    hb = HostBatch(num_tokens=N, num_entries=E, entry_start=starts, entry_len=lens_a, entry_past=past,
                   single_tokens=single, bound_single=int(bound_single), bound_multi=int(bound_multi))
    plans = {pl.key: pl.plan(hb) for pl in planners}

    pieces = [token_ids.astype(np.int32), positions, tok_seq, logit_rows, starts, lens_a, past, slot]
    for g in range(G):
        pieces += [group_slots[g], group_tables[g].reshape(-1)]
    if position_axes > 1:
        pos_ids = np.repeat(positions[:, None], position_axes, axis=1)
        for e, s, r in zip(entries, starts, real):
            if e.positions is not None:
                pos_ids[s:s + r] = np.asarray(e.positions, dtype=np.int32).reshape(r, position_axes)
        pieces.append(pos_ids.reshape(-1))
    plan_names = []
    for key, plan in plans.items():
        for name, a in plan.arrays.items():
            if a.dtype != np.int32:
                raise TypeError(f"planner {key}: array '{name}' must be int32")
            pieces.append(a.reshape(-1))
            plan_names.append((key, name, a.shape))
    sizes = [p.size for p in pieces]
    total = max(1, sum(sizes))
    host = staging.acquire(total) if staging is not None else torch.empty(
        (total,), dtype=torch.int32, pin_memory=device.type == "cuda")
    hv = host.numpy()
    off = 0
    for p in pieces:
        hv[off:off + p.size] = p
        off += p.size
    image = hv[:sum(sizes)].copy()
    if static is not None:
        if static.numel() < total or static.dtype != torch.int32:
            raise ValueError("the static batch buffer is too small")
        dev = static[:total]
        dev.copy_(host, non_blocking=True)
    else:
        dev = host.to(device, non_blocking=True)
    if staging is not None:
        staging.copied()
    views = []
    off = 0
    for s in sizes:
        views.append(dev[off:off + s])
        off += s
    groups = [GroupView(views[FIXED_PIECES + 2 * g], views[FIXED_PIECES + 1 + 2 * g].view(E, widths[g]))
              for g in range(G)]
    nxt = FIXED_PIECES + 2 * G
    position_ids = views[1]
    if position_axes > 1:
        position_ids = views[nxt].view(N, position_axes)
        nxt += 1
    for i, (key, name, shape) in enumerate(plan_names):
        plans[key].dev[name] = views[nxt + i].view(shape)
    return DeviceBatch(num_tokens=N, num_entries=E, num_logit_rows=R, token_ids=views[0], positions=views[1],
                       tok_seq=views[2], logit_rows=views[3], entry_start=views[4], entry_len=views[5],
                       entry_past=views[6], entry_slot=views[7], groups=groups, position_ids=position_ids,
                       plans=plans, host_start=starts, host_len=lens_a, host_past=past, host_slot=slot,
                       host_image=image, device_image=dev, single_tokens=single,
                       all_rows_wanted=bool(R == N and (logit_rows == np.arange(N, dtype=np.int32)).all()))


class DecodeImage:
    """The host image of a decode step's index arrays (every entry one token), kept from step to step.

    While the same sequences go on decoding, only the token ids, the positions and the cache slots
    change, and a block table row when its sequence took or gave back a page: ``refresh`` rewrites
    just those in place instead of packing everything anew (and the arrays of planners that do not say
    ``fixed_for_single_tokens``).  The layout is the one ``build_device_batch`` makes for the same
    entries and table widths.  ``pad_entries`` / ``pad_rows``: entries that belong to no request and wanted
    rows behind the real ones, as in ``build_device_batch``; they stay as they were made."""

    def __init__(self, entries: Sequence[StepEntry], cache: CacheManager, vocab_size: int, device: torch.device,
                 staging: StagingRing, widths: Sequence[int], static: Optional[torch.Tensor],
                 planners: Sequence[StepPlanner] = (), position_axes: int = 1, bound_single: int = 0,
                 pad_entries: int = 0, pad_rows: int = 0):
        self.cache, self.vocab_size, self.staging, self.static = cache, vocab_size, staging, static
        self.widths = tuple(int(w) for w in widths)
        self.planners, self.axes, self.bound_single = tuple(planners), int(position_axes), int(bound_single)
        self.batch = build_device_batch(entries, cache, vocab_size, device, staging, widths, static,
                                        planners=planners, position_axes=position_axes, bound_single=bound_single,
                                        pad_entries=pad_entries, pad_rows=pad_rows)
        self.static = self.batch.device_image       # the buffer given, or the one this step made
        self.real = len(entries)                    # the entries of requests come first
        E, R = len(entries) + int(pad_entries), self.batch.num_logit_rows
        self.seqs = [e.seq for e in entries]
        self.wants = tuple(len(e.want) for e in entries)
        self.versions = [e.seq.version for e in entries]
        sizes = [E, E, E, R, E, E, E, E]
        for w in self.widths:
            sizes += [E, E * w]
        if self.axes > 1:
            sizes.append(E * self.axes)
        self.plan_pieces = {}          # (planner key, array name) -> index of its piece
        for key, plan in self.batch.plans.items():
            for name, a in plan.arrays.items():
                self.plan_pieces[(key, name)] = len(sizes)
                sizes.append(int(a.size))
        self.total = sum(sizes)
        self.offsets = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int64)
        self.image = np.empty(max(self.total, 1), dtype=np.int32)
        self.image[:self.total] = self.batch.host_image
        self.page_sizes = [g.page_size for g in cache.groups]
        self.entries_made = E
        self.rows = np.arange(self.real)

    def piece(self, i: int) -> np.ndarray:
        return self.image[self.offsets[i]:self.offsets[i + 1]]

    def matches(self, entries: Sequence[StepEntry]) -> bool:
        if len(entries) != len(self.seqs):
            return False
        for e, s, w in zip(entries, self.seqs, self.wants):
            if (e.seq is not s or len(e.tokens) != 1 or len(e.want) != w or (w and e.want[0] != 0)
                    or e.positions is not None):
                return False
        return True

    def refresh(self, entries: Sequence[StepEntry]) -> DeviceBatch:
        """The image for this step (``matches(entries)`` holds), copied to the device buffer."""
        E, made = len(entries), self.entries_made
        toks = np.fromiter((e.tokens[0] for e in entries), dtype=np.int64, count=E)
        if toks.min() < 0 or toks.max() >= self.vocab_size:
            bad = toks[(toks < 0) | (toks >= self.vocab_size)][0]
            raise ValueError(f"token id {int(bad)} is outside the vocabulary of {self.vocab_size}")
        pos = np.fromiter((s.length for s in self.seqs), dtype=np.int32, count=E)
        self.piece(0)[:E] = toks
        self.piece(1)[:E] = pos
        self.piece(6)[:E] = pos
        G = len(self.widths)
        for g, w in enumerate(self.widths):
            table = self.piece(FIXED_PIECES + 1 + 2 * g).reshape(made, w)
            for i, s in enumerate(self.seqs):
                if s.version != self.versions[i]:
                    pg = s.pages[g]
                    if len(pg) > w:
                        raise ValueError(f"block tables of group {g} need {len(pg)} columns, {w} given")
                    table[i, :len(pg)] = pg
                    table[i, len(pg):] = -1
            ps = self.page_sizes[g]
            pages = table[self.rows, pos // ps]
            if (pages < 0).any():
                raise RuntimeError("a decoded token's position has no page")
            self.piece(FIXED_PIECES + 2 * g)[:E] = pages * ps + pos % ps
        if self.axes > 1:
            self.piece(FIXED_PIECES + 2 * G)[:E * self.axes] = np.repeat(pos, self.axes)
        for i, s in enumerate(self.seqs):
            self.versions[i] = s.version
        moving = [pl for pl in self.planners if not pl.fixed_for_single_tokens]
        if moving:
            past = pos if made == E else np.concatenate([pos, np.zeros(made - E, dtype=np.int32)])
            hb = HostBatch(num_tokens=made, num_entries=made, entry_start=self.batch.host_start,
                           entry_len=self.batch.host_len, entry_past=past, single_tokens=True,
                           bound_single=self.bound_single)
            for pl in moving:
                plan = pl.plan(hb)
                old = self.batch.plans[pl.key]
                if plan.sizes != old.sizes:
                    raise RuntimeError(f"planner {pl.key}: launch sizes moved under a recorded step")
                for name, a in plan.arrays.items():
                    piece = self.piece(self.plan_pieces[(pl.key, name)])
                    if a.size != piece.size:
                        raise RuntimeError(f"planner {pl.key}: array '{name}' changed its size under a recorded step")
                    piece[:] = a.reshape(-1)
        host = self.staging.acquire(self.total)
        host.numpy()[:] = self.image[:self.total]
        self.static[:self.total].copy_(host, non_blocking=True)
        self.staging.copied()
        self.batch.host_past = pos if made == E else np.concatenate([pos, np.zeros(made - E, dtype=np.int32)])
        return self.batch
