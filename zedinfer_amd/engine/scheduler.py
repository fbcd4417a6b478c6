"""The scheduler: admits requests, cuts prompts into portions under a token budget, decodes,
finishes and frees.

The policy is the reference's (reference: src/zedinfer/scheduler.cpp:267-394 schedule(),
:553-879 process_results()):
  * every step first gives each running request its one decode token;
  * what is left of ``max_batch_tokens``, capped by ``max_prefill_tokens``, goes to prompts,
    taken strictly from the head of the queue; a prompt that does not fit is cut and its rest
    waits at the head for the next step, so at most one request is partly prefilled;
  * the portion that completes a prompt yields the request's first token;
  * a request ends on a stop token ("stop") or at ``max_new_tokens`` ("length").
When pages run out:
  * at admission the head of the queue waits, unless nothing at all is running, in which case
    it can never be admitted and fails (reference: scheduler.cpp:343-359);
  * at decode the request that cannot grow fails with "KV cache exhausted during decode" and
    the others go on; nothing is preempted or swapped (reference: scheduler.cpp:293-319).
It needs the cache manager's bookkeeping only, no device.
"""
from __future__ import annotations

import threading
import time
from collections import deque
from dataclasses import dataclass, field
from typing import Deque, Iterable, List, Optional, Sequence

from ..cache.manager import CacheManager
from ..cache.pages import OutOfPages, OutOfSlots
from ..config.scheduler_config import SchedulerConfig
from ..sampling.sampler import RequestSampler
from .batch import StepEntry
from .request import (GenerationResult, InferenceRequest, RequestPhase, resolve_max_new_tokens)


class QueueFull(RuntimeError):
    pass


@dataclass
class ScheduledBatch:
    """(reference: include/zedinfer/batch_context.hpp:52-63)"""

    decode_requests: List[InferenceRequest] = field(default_factory=list)
    prefill_requests: List[InferenceRequest] = field(default_factory=list)
    prefill_chunk_starts: List[int] = field(default_factory=list)
    prefill_chunk_sizes: List[int] = field(default_factory=list)

    def empty(self) -> bool:
        return not self.decode_requests and not self.prefill_requests

    def num_tokens(self) -> int:
        return len(self.decode_requests) + sum(self.prefill_chunk_sizes)

    def completes_prompt(self, i: int) -> bool:
        r = self.prefill_requests[i]
        return self.prefill_chunk_starts[i] + self.prefill_chunk_sizes[i] >= len(r.input_ids)

    # a batch that was scheduled before the tokens of the step before it were known: its decode
    # tokens are read on the device from what that step sampled, in the order of decode_requests
    tokens_on_device: bool = False

    def entries(self) -> List[StepEntry]:
        """Decode rows first, then the prompt portions; logits are wanted for each decode token and
        for the last token of a portion that completes its prompt
        (reference: src/zedinfer/batch_context.cpp:21-85)."""
        out = [StepEntry(r.seq, [0 if self.tokens_on_device else r.last_token], [0]) for r in self.decode_requests]
        for i, r in enumerate(self.prefill_requests):
            s, n = self.prefill_chunk_starts[i], self.prefill_chunk_sizes[i]
            out.append(StepEntry(r.seq, r.input_ids[s:s + n], [n - 1] if self.completes_prompt(i) else []))
        return out

    def sampled_requests(self) -> List[InferenceRequest]:
        """The requests that get a token from this step, in the order of the logits rows."""
        return list(self.decode_requests) + [r for i, r in enumerate(self.prefill_requests)
                                              if self.completes_prompt(i)]


class Scheduler:
    def __init__(self, config: SchedulerConfig, cache: CacheManager, stop_token_ids: Iterable[int] = (),
                 default_sampling=None):
        config.validate()
        self.config = config
        self.cache = cache
        self.default_sampling = default_sampling      # for requests that set no sampling option (None: greedy)
        self.stop_token_ids = set(int(t) for t in stop_token_ids)
        self.waiting: Deque[InferenceRequest] = deque()
        self.active: List[InferenceRequest] = []
        self.finished: List[InferenceRequest] = []
        self._next_id = 1
        self._lock = threading.Lock()
        self._work = threading.Condition(self._lock)

    # ---- submitting ------------------------------------------------------------------
    def submit(self, req: InferenceRequest) -> int:
        """Queue a request (reference: scheduler.cpp:41-53).  Resolves max_new_tokens against the
        context length (reference: src/zedinfer/serving_loop.cpp:119-136)."""
        req.config.validate()
        if not req.input_ids:
            raise ValueError("a request needs at least one prompt token")
        req.config.max_new_tokens = resolve_max_new_tokens(req.config.max_new_tokens, len(req.input_ids),
                                                           self.config.max_seq_len)
        with self._work:
            if len(self.waiting) >= self.config.max_queue_size:
                raise QueueFull(f"Queue full ({self.config.max_queue_size})")
            req.request_id = self._next_id
            self._next_id += 1
            req.phase = RequestPhase.QUEUED
            req.sampler = RequestSampler(req.config.sampling(self.default_sampling))
            req.stats.prompt_tokens = len(req.input_ids)
            self.waiting.append(req)
            self._work.notify_all()
        return req.request_id

    def pending_count(self) -> int:
        return len(self.waiting)

    def active_count(self) -> int:
        return len(self.active)

    def has_work(self) -> bool:
        return bool(self.waiting or self.active)

    def wait_for_work(self, timeout: Optional[float] = None) -> bool:
        with self._work:
            if not self.has_work():
                self._work.wait(timeout)
            return self.has_work()

    # ---- one step's batch ----------------------------------------------------------------
    def _reserve(self, req: InferenceRequest) -> int:
        """Tokens a request is promised pages for at admission: its prompt and
        min(max_new_tokens, generation_reserve) generated ones."""
        return len(req.input_ids) + min(req.config.max_new_tokens, self.config.generation_reserve)

    def schedule(self) -> ScheduledBatch:
        batch = ScheduledBatch()
        budget = self.config.max_batch_tokens
        with self._lock:
            # 1. decode first
            for req in list(self.active):
                if budget <= 0:
                    break
                if req.done:
                    continue
                if req.cancelled:
                    self._complete(req, "stop")
                    continue
                try:
                    self.cache.ensure(req.seq, req.seq.length + 1)
                except OutOfPages as e:
                    self._fail(req, f"KV cache exhausted during decode for request {req.request_id}: {e}")
                    continue
                batch.decode_requests.append(req)
                budget -= 1
            self.active = [r for r in self.active if not r.done]
            self._schedule_prompts(batch, budget)
        return batch

    def _schedule_prompts(self, batch: ScheduledBatch, budget: int) -> None:
        """The second half of a step's batch: portions of prompts, from the head of the queue, under what the
        decoding requests left of the token budget.  The caller holds the lock."""
        prefill_budget = min(budget, self.config.max_prefill_tokens)
        while self.waiting and prefill_budget > 0:
            req = self.waiting[0]
            if len(self.active) + len([r for r in batch.prefill_requests if r not in self.active]) \
                    >= self.config.max_batch_requests:
                break
            if req.seq is None:
                reserve = self._reserve(req)
                if not self.cache.can_open(reserve):
                    msg = (f"Cannot admit request {req.request_id}: prompt={len(req.input_ids)} tokens, "
                           f"reserve={reserve} tokens, free pages="
                           f"{[g.pool.uncommitted for g in self.cache.groups]}, "
                           f"free slots={self.cache.slots.num_free}")
                    req.admission_warned = True
                    if batch.empty() and not self.active:
                        self.waiting.popleft()
                        self._fail(req, msg)
                        continue
                    break
                try:
                    req.seq = self.cache.open(req.request_id, reserve)
                except (OutOfPages, OutOfSlots) as e:
                    self.waiting.popleft()
                    self._fail(req, f"Cannot allocate KV cache for request {req.request_id}: {e}")
                    continue
            remaining = len(req.input_ids) - req.prefill_progress
            chunk = min(remaining, prefill_budget)
            try:
                self.cache.ensure(req.seq, req.seq.length + chunk)
            except OutOfPages as e:
                self.waiting.popleft()
                self._fail(req, f"Cannot allocate KV cache for request {req.request_id}: {e}")
                continue
            batch.prefill_requests.append(req)
            batch.prefill_chunk_starts.append(req.prefill_progress)
            batch.prefill_chunk_sizes.append(chunk)
            prefill_budget -= chunk
            req.prefill_progress += chunk
            req.phase = RequestPhase.PREFILL
            if req.prefill_progress >= len(req.input_ids):
                self.active.append(self.waiting.popleft())
            else:
                break

    def schedule_ahead(self, batch: ScheduledBatch) -> Optional[ScheduledBatch]:
        """The batch after ``batch``, made while ``batch`` still runs, or None when it cannot be known
        yet.  It can when the results of ``batch`` will change nothing but the tokens: the requests it
        samples for are all that run, and none of them reaches its length with this token, is cancelled or
        needs its history for sampling.  Every such request then decodes in the next step, whatever its token
        (read on the device), and the prompts' portions beside them are what ``schedule()`` would take: lengths
        and pages are booked when a step is queued, not when it ends.  A request that ends on a stop token in
        ``batch`` has one token too many computed; ``process_results`` drops it.  A waiting prompt that only a
        request's end makes room for enters one step later than it would without looking ahead."""
        with self._lock:
            sampled = batch.sampled_requests()
            if len(sampled) != len(self.active) or any(a is not b for a, b in zip(self.active, sampled)):
                return None
            if not sampled and not self.waiting:
                return None
            if len(sampled) > self.config.max_batch_tokens:
                return None
            for r in sampled:
                made = (r.generated_count if r.phase == RequestPhase.DECODE else 0) + 1
                if r.done or r.cancelled or made >= r.config.max_new_tokens:
                    return None
                if r.sampler.params.repetition_penalty != 1.0:
                    return None
            try:
                for r in sampled:
                    self.cache.ensure(r.seq, r.seq.length + 1)
            except OutOfPages:
                return None             # the ordinary step decides who fails
            ahead = ScheduledBatch(decode_requests=list(sampled), tokens_on_device=True)
            self._schedule_prompts(ahead, self.config.max_batch_tokens - len(sampled))
            return None if ahead.empty() else ahead

    # ---- after the step ------------------------------------------------------------------
    def process_results(self, batch: ScheduledBatch, tokens: Sequence[int]) -> None:
        """``tokens``: one sampled token per request of ``batch.sampled_requests()``, in that order.
        The engine has already committed the new cache lengths."""
        sampled = batch.sampled_requests()
        if len(tokens) != len(sampled):
            raise ValueError(f"{len(tokens)} tokens for {len(sampled)} sampled requests")
        with self._lock:
            for req, tok in zip(sampled, tokens):
                if req.done or (batch.tokens_on_device and req.cancelled):
                    continue            # it ended, or was cancelled, while this step, scheduled ahead, was running
                tok = int(tok)
                first = req.phase != RequestPhase.DECODE
                req.phase = RequestPhase.DECODE
                req.output_ids.append(tok)
                req.last_token = tok
                req.generated_count = 1 if first else req.generated_count + 1
                if not req.config.ignore_eos and tok in self.stop_token_ids:
                    self._complete(req, "stop")
                elif req.generated_count >= req.config.max_new_tokens:
                    self._complete(req, "length")
                elif req.config.stream and req.config.stream_callback:
                    req.config.stream_callback(tok)
            self.active = [r for r in self.active if not r.done]

    def fail_batch(self, batch: ScheduledBatch, message: str) -> None:
        """A step that raised fails every request in it and frees what they hold; the loop goes on
        (reference: src/zedinfer/serving_loop.cpp:412-419,467-495)."""
        with self._lock:
            for req in list(batch.decode_requests) + list(batch.prefill_requests):
                if not req.done:
                    if self.waiting and self.waiting[0] is req:
                        self.waiting.popleft()
                    self._fail(req, message)
            self.active = [r for r in self.active if not r.done]

    # ---- finishing -----------------------------------------------------------------------
    def _release(self, req: InferenceRequest) -> None:
        if req.seq is not None and not req.seq.closed:
            self.cache.close(req.seq)

    def _complete(self, req: InferenceRequest, reason: str) -> None:
        """(reference: complete_request, scheduler.cpp:881-907)"""
        req.finish_reason = reason
        req.phase = RequestPhase.COMPLETE
        self._release(req)
        req.stats.generated_tokens = len(req.output_ids)
        req.stats.total_time_ms = (time.perf_counter() - req.arrival_time) * 1000.0
        req.result = GenerationResult(list(req.output_ids), req.stats, reason, req.error)
        self.finished.append(req)

    def _fail(self, req: InferenceRequest, message: str) -> None:
        req.error = message
        self._complete(req, "error")
