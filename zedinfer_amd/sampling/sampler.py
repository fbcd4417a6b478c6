"""Choosing the next token: argmax, and temperature / top-k / top-p / repetition-penalty
sampling, one kernel launch for all rows of a step.

Options and their meanings are the reference's (reference: include/frontend/sampler/sampler.hpp:27-40
SamplerParams; validation src/frontend/sampler/sampler.cpp:24-38; the order of the steps
:195-265).  The uniform draw comes from the host, as in the reference's GPU path
(sampler.cpp:400-407), but from a generator kept per request, so that what a request samples
does not depend on what else is in the batch (the reference shares one generator,
src/zedinfer/scheduler.cpp:584-600).
"""
from __future__ import annotations

import json
import os
import random
from dataclasses import dataclass
from typing import List, Optional, Sequence

import numpy as np
import torch

from .. import ops
from ..ops.staging import StagingRing


@dataclass
class SamplingParams:
    """temperature <= 0 or ``use_argmax`` means greedy (reference: scheduler.cpp:581-583)."""

    temperature: float = 0.0
    top_k: int = 0                   # 0: off
    top_p: float = 1.0               # 1: off
    repetition_penalty: float = 1.0  # 1: off; applied to generated tokens only
    seed: int = 0                    # 0: seeded from the system
    use_argmax: bool = False

    @property
    def greedy(self) -> bool:
        return self.use_argmax or self.temperature <= 0.0

    def validate(self) -> None:
        if self.top_k < 0:
            raise ValueError("top_k must be non-negative")
        if not (0.0 < self.top_p <= 1.0):
            raise ValueError("top_p must be in (0, 1]")
        if not (self.repetition_penalty > 0.0):
            raise ValueError("repetition_penalty must be positive")
        if not self.use_argmax and self.temperature < 0.0:
            raise ValueError("temperature must be non-negative (0 means greedy)")


def default_sampling(model_path: Optional[str]) -> SamplingParams:
    """What a request samples with when it sets no sampling option of its own: the model folder's
    generation_config.json when it says ``do_sample`` (temperature default 1, top_k 0, top_p 1,
    repetition_penalty 1, seed 0), else greedy; also greedy when the file is missing, unreadable or its
    values do not validate.  ``ZEDINFER_FORCE_ARGMAX`` (set, not "0") forces greedy,
    ``ZEDINFER_REPETITION_PENALTY`` overrides the file's penalty
    (reference: src/zedinfer/engine.cpp:49-126)."""
    greedy = SamplingParams(use_argmax=True)
    force = os.environ.get("ZEDINFER_FORCE_ARGMAX", "")
    if force not in ("", "0"):
        return greedy
    if not model_path:
        return greedy
    path = os.path.join(model_path, "generation_config.json")
    if not os.path.isfile(path):
        return greedy
    try:
        with open(path) as f:
            j = json.load(f)
        if not bool(j.get("do_sample", False)):
            return greedy
        p = SamplingParams(temperature=float(j.get("temperature", 1.0)), top_k=int(j.get("top_k", 0)),
                           top_p=float(j.get("top_p", 1.0)), repetition_penalty=float(j.get("repetition_penalty", 1.0)),
                           seed=int(j.get("seed", 0)))
        env = os.environ.get("ZEDINFER_REPETITION_PENALTY", "")
        if env:
            try:
                p.repetition_penalty = float(env)
            except ValueError:
                pass
        # the reference's check: a temperature of 0 is not a valid sampler here, it falls back to greedy
        if not (p.temperature > 0.0):
            return greedy
        p.validate()
        return p
    except (OSError, ValueError, TypeError):
        return greedy


class RequestSampler:
    """The sampling state of one request: its parameters and its own generator."""

    def __init__(self, params: SamplingParams):
        params.validate()
        self.params = params
        self.rng = random.Random(params.seed) if params.seed != 0 else random.Random()

    def draw(self) -> float:
        u = np.float32(self.rng.random())
        return float(min(u, np.float32(0.99999994)))     # stays below 1 after rounding to float32


class Sampler:
    """Samples one token for each row of float32 logits [rows, vocab] on the device."""

    def __init__(self, device: torch.device, vocab_size: int):
        self.device = device
        self.vocab_size = vocab_size
        self.staging = StagingRing(device)

    def sample(self, logits: torch.Tensor, samplers: Sequence[RequestSampler],
               histories: Optional[Sequence[Sequence[int]]] = None) -> List[int]:
        """``samplers[i]`` and ``histories[i]`` (the tokens generated so far) belong to row i."""
        return self.launch(logits, samplers, histories).tolist()

    def launch(self, logits: torch.Tensor, samplers: Sequence[RequestSampler],
               histories: Optional[Sequence[Sequence[int]]] = None) -> torch.Tensor:
        """As ``sample``, but the tokens stay on the device (int32 [rows]) and nothing is waited for."""
        R = logits.shape[0]
        if R != len(samplers):
            raise ValueError(f"{R} rows of logits for {len(samplers)} requests")
        if all(s.params.greedy and s.params.repetition_penalty == 1.0 for s in samplers):
            return ops.argmax(logits)
        # the per-row parameters travel in one pinned buffer, so that nothing here waits for the device
        par = self.staging.acquire(5 * R)
        pv = par.numpy().reshape(5, R)
        pv[0].view(np.float32)[:] = [0.0 if s.params.greedy else s.params.temperature for s in samplers]
        pv[1][:] = [s.params.top_k for s in samplers]
        pv[2].view(np.float32)[:] = [s.params.top_p for s in samplers]
        pen = pv[3].view(np.float32)
        pen[:] = [s.params.repetition_penalty for s in samplers]
        pv[4].view(np.float32)[:] = [0.0 if s.params.greedy else s.draw() for s in samplers]
        recent = recent_len = None
        if histories is not None and any(p != 1.0 for p in pen):
            width = max(1, max(len(h) if pen[i] != 1.0 else 0 for i, h in enumerate(histories)))
            rc = np.zeros((R, width), dtype=np.int32)
            rl = np.zeros((R,), dtype=np.int32)
            for i, h in enumerate(histories):
                if pen[i] != 1.0 and len(h):
                    rc[i, :len(h)] = h
                    rl[i] = len(h)
            recent = torch.from_numpy(rc).to(self.device)
            recent_len = torch.from_numpy(rl).to(self.device)
        d = par.to(self.device, non_blocking=True).view(5, R)
        self.staging.copied()
        return ops.sample(logits, d[0].view(torch.float32), d[1], d[2].view(torch.float32), d[3].view(torch.float32),
                          d[4].view(torch.float32), recent, recent_len)
