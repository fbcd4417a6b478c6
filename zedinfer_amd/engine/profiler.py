"""Timing one synthetic request: a whole-prompt step, then single-token steps
(reference: src/zedinfer/profiler.cpp:119-162 run_profile_sequence, :194-213 profile; random ids in
[100, vocab-100], :79-84).  It drives ``Engine.step`` directly, without the scheduler."""
from __future__ import annotations

import random
import time
from typing import Tuple

import torch

from .. import ops
from .batch import StepEntry
from .engine import Engine


class Profiler:
    def __init__(self, engine: Engine, seed: int = 0):
        self.engine = engine
        self.rng = random.Random(seed)

    def random_ids(self, n: int):
        V = self.engine.vocab_size
        lo, hi = (100, V - 100) if V > 300 else (0, V)
        return [self.rng.randrange(lo, hi) for _ in range(n)]

    def warmup(self, prefill_len: int = 128, decode_steps: int = 128) -> None:
        # twice: a step of a shape is recorded as a graph the second time it comes, and replayed from then on
        self.profile(prefill_len, min(decode_steps, 8))
        self.profile(prefill_len, min(decode_steps, 8))

    def profile(self, prefill_len: int, decode_steps: int) -> Tuple[float, float]:
        """(prefill ms, decode ms): the prompt step includes taking its first token; decode covers the
        remaining decode_steps - 1 single-token steps."""
        eng = self.engine
        seq = eng.open(("profile", time.perf_counter_ns()), prefill_len + decode_steps)
        try:
            ids = self.random_ids(prefill_len)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            logits = eng.step([StepEntry(seq, ids, [prefill_len - 1])], copy=False)
            tok = ops.argmax(logits).tolist()[0]
            t1 = time.perf_counter()
            for _ in range(decode_steps - 1):
                logits = eng.step([StepEntry(seq, [tok], [0])], copy=False)
                tok = ops.argmax(logits).tolist()[0]
            torch.cuda.synchronize()
            t2 = time.perf_counter()
        finally:
            eng.close(seq)
        return (t1 - t0) * 1000.0, (t2 - t1) * 1000.0
