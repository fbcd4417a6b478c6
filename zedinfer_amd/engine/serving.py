"""The serving loop and the engine object users hold.

``InferenceEngine.create(model_path, ...)`` builds model, cache, scheduler and sampler;
``serving_loop().submit_async`` queues requests, ``step()`` runs one scheduled batch,
``run_loop()`` runs until nothing is left, ``generate_tokens`` does all of it for one prompt
(reference: include/zedinfer/serving_loop.hpp:36-56, src/zedinfer/serving_loop.cpp:182-422;
include/zedinfer/engine.hpp:96-166, src/zedinfer/engine.cpp:338-522).
"""
from __future__ import annotations

import os
import time
from typing import Iterable, List, Optional, Sequence

import torch

from ..config import SchedulerConfig
from ..ops.staging import StagingRing
from ..sampling.sampler import Sampler
from ..parts.rows import sizes_between
from .engine import Engine
from .request import GenerationConfig, GenerationResult, InferenceRequest
from .scheduler import ScheduledBatch, Scheduler


class _Flight:
    """A step that has been queued on the device: its batch, where its tokens will arrive on the host,
    and the event after which they are there."""

    def __init__(self, batch: ScheduledBatch, tokens_dev: Optional[torch.Tensor], tokens_host: Optional[torch.Tensor],
                 done: torch.cuda.Event, t0: float):
        self.batch, self.tokens_dev, self.tokens_host, self.done, self.t0 = batch, tokens_dev, tokens_host, done, t0

    def wait(self) -> List[int]:
        self.done.synchronize()
        return self.tokens_host.tolist() if self.tokens_host is not None else []


class ServingLoop:
    """``look_ahead``: while a step runs, the next one is queued behind it with its decoding requests' tokens
    read on the device from what the running step samples, so the device does not wait for the host between
    steps.  The tokens a request gets are the same either way (``Scheduler.schedule_ahead`` says when the
    next batch is known early).  The reference's loop waits for every step's tokens before it schedules
    the next (src/zedinfer/serving_loop.cpp:330-408)."""

    def __init__(self, engine: Engine, stop_token_ids: Iterable[int] = (), look_ahead: Optional[bool] = None):
        self.engine = engine
        self.scheduler = Scheduler(engine.sched, engine.cache, stop_token_ids,
                                   getattr(engine, "default_sampling", None))
        self.sampler = Sampler(engine.device, engine.vocab_size)
        self.look_ahead = os.environ.get("ZEDINFER_DISABLE_LOOKAHEAD", "0") in ("", "0") if look_ahead is None \
            else bool(look_ahead)
        self.steps_ahead = 0            # steps that were queued before the one before them had finished
        self.prompt_steps_ahead = 0     # those of them that carried portions of prompts
        self._flight: Optional[_Flight] = None
        self._token_ring = StagingRing(engine.device)
        self._last_results = 0.0
        self._running = False

    def submit_async(self, request: InferenceRequest) -> InferenceRequest:
        """Queue a request; its ``result`` is set when it completes."""
        self.scheduler.submit(request)
        return request

    def pending_count(self) -> int:
        return self.scheduler.pending_count()

    def active_count(self) -> int:
        return self.scheduler.active_count()

    def _launch(self, batch: ScheduledBatch, token_source: Optional[torch.Tensor]) -> Optional[_Flight]:
        """Queue the batch's step, its sampling and the copy of the tokens to the host; nothing is waited
        for.  A step that raises fails its batch, not the loop."""
        t0 = time.perf_counter()
        try:
            logits = self.engine.step(batch.entries(), copy=False, token_source=token_source)
            sampled = batch.sampled_requests()
            tokens_dev = tokens_host = None
            if sampled:
                tokens_dev = self.sampler.launch(logits, [r.sampler for r in sampled], [r.output_ids for r in sampled])
                tokens_host = self._token_ring.acquire(len(sampled))
                tokens_host.copy_(tokens_dev, non_blocking=True)
                self._token_ring.copied()
            done = torch.cuda.Event()
            done.record()
        except Exception as e:  # noqa: BLE001
            self.scheduler.fail_batch(batch, f"step failed: {type(e).__name__}: {e}")
            return None
        return _Flight(batch, tokens_dev, tokens_host, done, t0)

    def step(self) -> bool:
        """One scheduled batch through the model, to the point where its tokens have reached their
        requests.  Returns False when there was nothing to run."""
        flight, self._flight = self._flight, None
        if flight is None:
            batch = self.scheduler.schedule()
            if batch.empty():
                return False
            flight = self._launch(batch, None)
            if flight is None:
                return True
        batch = flight.batch
        if self.look_ahead:
            ahead = self.scheduler.schedule_ahead(batch)
            if ahead is not None:
                self._flight = self._launch(ahead, flight.tokens_dev)
                self.steps_ahead += self._flight is not None
                self.prompt_steps_ahead += self._flight is not None and bool(ahead.prefill_requests)
        try:
            tokens = flight.wait()
        except Exception as e:  # noqa: BLE001
            self.scheduler.fail_batch(batch, f"step failed: {type(e).__name__}: {e}")
            if self._flight is not None:
                # the step queued behind it may carry portions of other requests' prompts: what it computed for
                # them is not to be trusted either, and its tokens will not be read
                self.scheduler.fail_batch(self._flight.batch, f"step failed: {type(e).__name__}: {e}")
            self._flight = None
            return True
        now = time.perf_counter()
        ms = (now - max(flight.t0, self._last_results)) * 1000.0
        self._last_results = now
        # time is split like the reference's: a step's time goes to prefill for prompt portions and is
        # shared evenly among the decoding requests (reference: serving_loop.cpp:287-305)
        n_dec, n_pre = len(batch.decode_requests), len(batch.prefill_requests)
        for r in batch.prefill_requests:
            r.stats.prefill_time_ms += ms / n_pre if not n_dec else ms * 0.5 / n_pre
        for r in batch.decode_requests:
            r.stats.decode_time_ms += ms / n_dec if not n_pre else ms * 0.5 / n_dec
        self.scheduler.process_results(batch, tokens)
        if (self._flight is not None and not self._flight.batch.prefill_requests
                and all(r.done for r in self._flight.batch.decode_requests)):
            self._flight = None         # everything the step ahead computes for has ended
        return True

    def run_loop(self) -> None:
        """Run until every queued and running request is done (reference: run_loop, offline mode)."""
        while self.scheduler.has_work():
            if not self.step() and not self.scheduler.has_work():
                break

    def run_serving(self) -> None:
        """Run until ``stop()``; sleeps while idle."""
        self._running = True
        while self._running:
            if not self.step():
                self.scheduler.wait_for_work(timeout=0.05)

    def stop(self) -> None:
        self._running = False

    def generate_tokens(self, input_ids: Sequence[int], config: Optional[GenerationConfig] = None) -> GenerationResult:
        req = InferenceRequest(input_ids, config)
        self.submit_async(req)
        while not req.done:
            self.step()
        if req.error:
            raise RuntimeError(req.error)
        return req.result


class InferenceEngine:
    """Everything for generation from one model folder."""

    WARM_UP_EVERY_SIZE_UP_TO = 8192     # rows; measuring every size of longer steps would take minutes

    @classmethod
    def default_warm_up_sizes(cls, sched: SchedulerConfig, step_rows, most_entries: int = 256) -> List[int]:
        """The numbers of rows that the padded steps of an engine with these limits come in, largest first.
        ``step_rows(rows, kind)`` is the model's (``DecoderModel.step_rows``: the parts say which numbers of rows
        steps are run with).  Every size a step with portions of prompts can bring up to WARM_UP_EVERY_SIZE_UP_TO
        rows, of longer steps the two that recur (a full portion alone and beside decoding requests), and the
        sizes of pure decode steps.  What, if anything, is measured at a size is each part's business
        (``Part.tune``)."""
        beside = step_rows(1, "beside")         # decoding entries beside a portion are rounded up: one more size
        most = min(sched.max_batch_tokens, sched.max_prefill_tokens + sched.max_batch_requests)
        sizes = sizes_between(step_rows, "mixed", step_rows(2, "portion"), min(most, cls.WARM_UP_EVERY_SIZE_UP_TO) + beside)
        if most > cls.WARM_UP_EVERY_SIZE_UP_TO:
            sizes += [step_rows(sched.max_prefill_tokens, "mixed"),
                      step_rows(min(most, sched.max_prefill_tokens + beside) + beside, "mixed")]
        sizes += sizes_between(step_rows, "decode", 1, min(sched.max_batch_requests, most_entries))
        return sorted(set(sizes), reverse=True)

    def __init__(self, engine: Engine, warm_up_sizes: Optional[Sequence[int]] = None, freeze_gc: Optional[bool] = None):
        """``warm_up_sizes``: numbers of rows to measure the parts' choices for now (None: none now; every size
        is measured when a step of that size first comes.  "all": every size a step can bring under the
        scheduler's limits, now: minutes for a large model, and no step ever waits for a measurement).
        ``freeze_gc``: take what the process holds by now out of the garbage collector's passes (None: what
        ZEDINFER_GC_FREEZE says, off without it: a library should not change its host's collector; the command
        line programs switch it on)."""
        self.engine = engine
        self._loop = ServingLoop(engine, engine.fc.eos_token_ids)
        # The products' algorithms (and other choices of the parts) for steps of many rows are measured, once for
        # every number of rows that steps come in: the library's first proposal for a shape can be a third slower
        # than what timing finds, and what timing finds for one number of rows does not carry over to its
        # neighbours (measured).  By default a size is measured when its first step is about to run
        # (``Engine.tune_when_scheduled``), between steps: making the engine takes no longer than loading the model.
        # ZEDINFER_WARM_UP=all measures every size now, ZEDINFER_WARM_UP=0 (or the reference's own switch,
        # ZEDINFER_DISABLE_WARMUP set, src/zedinfer/engine.cpp:506) measures nothing, ever: the defaults.
        mode = os.environ.get("ZEDINFER_WARM_UP", "1")
        if mode not in ("", "0") and "ZEDINFER_DISABLE_WARMUP" not in os.environ and engine.device.type == "cuda":
            if mode == "all" or (isinstance(warm_up_sizes, str) and warm_up_sizes == "all"):
                warm_up_sizes = self.default_warm_up_sizes(engine.sched, engine.model.step_rows, engine.graph_max_entries)
            engine.tune_when_scheduled = True
            if warm_up_sizes:
                engine.warm_up(list(warm_up_sizes))
        # What the process holds by now (modules, the model's parts and tensors) lives as long as the engine:
        # taken out of the garbage collector's passes, a full collection in the middle of serving costs
        # little (measured: one of 50 ms among decode steps of 6.5 ms without this).
        if freeze_gc is None:
            freeze_gc = os.environ.get("ZEDINFER_GC_FREEZE", "0") not in ("", "0")
        if freeze_gc:
            import gc
            gc.collect()
            gc.freeze()

    @classmethod
    def create(cls, model_path: str, dtype="bfloat16", scheduler_config: Optional[SchedulerConfig] = None,
               warm_up_sizes: Optional[Sequence[int]] = None, freeze_gc: Optional[bool] = None) -> "InferenceEngine":
        return cls(Engine.from_folder(model_path, dtype, scheduler_config), warm_up_sizes, freeze_gc)

    @property
    def default_sampling(self):
        """What requests without sampling options of their own sample with."""
        return self.engine.default_sampling

    def serving_loop(self) -> ServingLoop:
        return self._loop

    def stop_token_ids(self) -> List[int]:
        return sorted(self._loop.scheduler.stop_token_ids)

    def block_pool(self):
        return self.engine.cache

    def generate_tokens(self, input_ids: Sequence[int], config: Optional[GenerationConfig] = None) -> GenerationResult:
        return self._loop.generate_tokens(input_ids, config)

    def generate(self, prompts: Sequence[Sequence[int]], config: Optional[GenerationConfig] = None
                 ) -> List[GenerationResult]:
        """Token ids in, token ids out, for several prompts batched continuously."""
        import copy
        reqs = [self._loop.submit_async(InferenceRequest(p, copy.copy(config) if config else None)) for p in prompts]
        self._loop.run_loop()
        for r in reqs:
            if r.error:
                raise RuntimeError(r.error)
        return [r.result for r in reqs]
