"""Requests, their options and their results (reference: include/zedinfer/request.hpp:23-243,
include/zedinfer/generation_types.hpp:20-126)."""
from __future__ import annotations

import time
from dataclasses import dataclass, field
from enum import Enum
from typing import Callable, List, Optional

from ..sampling.sampler import RequestSampler, SamplingParams


class RequestPhase(Enum):
    QUEUED = "queued"        # waiting for admission
    PREFILL = "prefill"      # prompt partly in the cache
    DECODE = "decode"        # generating one token a step
    COMPLETE = "complete"    # finished, failed or cancelled


@dataclass
class GenerationConfig:
    """``max_new_tokens`` 0 means "until the context is full" (reference: generation_types.hpp:20-25).
    Sampling fields as in the reference's per-request overrides (:70-78)."""

    max_new_tokens: int = 0
    temperature: float = 0.0
    top_k: int = 0
    top_p: float = 1.0
    repetition_penalty: float = 1.0
    seed: int = 0
    use_argmax: bool = False
    ignore_eos: bool = False          # benchmarks generate a fixed number of tokens
    stream: bool = False
    stream_callback: Optional[Callable[[int], None]] = None   # called with each new token id

    def validate(self) -> None:
        if self.max_new_tokens < 0:
            raise ValueError("max_new_tokens must be non-negative (0 means unlimited)")
        if self.stream and self.stream_callback is None:
            raise ValueError("stream_callback required when stream=True")
        self.sampling().validate()

    def overrides_sampling(self) -> bool:
        """Whether the request sets a sampling option of its own (the reference's has_sampling_override,
        generation_types.hpp:56-67); a seed alone is none."""
        return (self.use_argmax or self.temperature != 0.0 or self.top_k != 0 or self.top_p != 1.0
                or self.repetition_penalty != 1.0)

    def sampling(self, default: Optional[SamplingParams] = None) -> SamplingParams:
        """The request's own options, or ``default`` (the engine's: from the model's
        generation_config.json) when it sets none; its seed, when it has one, holds either way
        (reference: pick_sampler, src/zedinfer/scheduler.cpp:576-600)."""
        if default is not None and not self.overrides_sampling():
            return SamplingParams(default.temperature, default.top_k, default.top_p, default.repetition_penalty,
                                  self.seed or default.seed, default.use_argmax)
        return SamplingParams(self.temperature, self.top_k, self.top_p, self.repetition_penalty, self.seed,
                              self.use_argmax)


def resolve_max_new_tokens(requested: int, used_context_tokens: int, max_seq_len: int) -> int:
    """0 or too large becomes the room left in the context; no room is an error
    (reference: src/zedinfer/generation_types.cpp:39-61)."""
    if requested < 0:
        raise ValueError("max_new_tokens must be non-negative (0 means unlimited)")
    if used_context_tokens < 0:
        raise ValueError("used_context_tokens must be non-negative")
    if max_seq_len <= 0:
        raise ValueError("max_seq_len must be positive")
    remaining = max_seq_len - used_context_tokens
    if remaining <= 0:
        raise ValueError(f"prompt leaves no room for generation: context={used_context_tokens} tokens "
                         f"(max {max_seq_len})")
    if requested == 0 or requested > remaining:
        return remaining
    return requested


@dataclass
class GenerationStats:
    """(reference: generation_types.hpp:95-126, summary at generation_types.cpp:67-83)"""

    prompt_tokens: int = 0
    generated_tokens: int = 0
    prefill_time_ms: float = 0.0
    decode_time_ms: float = 0.0
    total_time_ms: float = 0.0

    @property
    def total_tokens(self) -> int:
        return self.prompt_tokens + self.generated_tokens

    def prefill_tokens_per_second(self) -> float:
        return self.prompt_tokens * 1000.0 / self.prefill_time_ms if self.prefill_time_ms > 0 else 0.0

    def decode_tokens_per_second(self) -> float:
        return self.generated_tokens * 1000.0 / self.decode_time_ms if self.decode_time_ms > 0 else 0.0

    def summary(self) -> str:
        return ("\n=== Generation Statistics ===\n"
                "Tokens:\n"
                f"  Prompt:     {self.prompt_tokens}\n"
                f"  Generated:  {self.generated_tokens}\n"
                f"  Total:      {self.total_tokens}\n"
                "Performance:\n"
                f"  Prefill:  {self.prefill_time_ms:.2f} ms ({self.prefill_tokens_per_second():.2f} token/s)\n"
                f"  Decode:   {self.decode_time_ms:.2f} ms ({self.decode_tokens_per_second():.2f} token/s)\n"
                f"  Total:    {self.total_time_ms:.2f} ms\n"
                "=============================")


@dataclass
class GenerationResult:
    output_ids: List[int] = field(default_factory=list)
    stats: GenerationStats = field(default_factory=GenerationStats)
    finish_reason: str = "stop"       # "stop", "length" or "error"
    error: Optional[str] = None


class InferenceRequest:
    def __init__(self, input_ids, config: Optional[GenerationConfig] = None):
        self.request_id: int = 0
        self.input_ids: List[int] = [int(t) for t in input_ids]
        self.config = config or GenerationConfig()
        self.phase = RequestPhase.QUEUED
        self.prefill_progress = 0
        self.generated_count = 0
        self.last_token = -1
        self.output_ids: List[int] = []
        self.finish_reason = "stop"
        self.error: Optional[str] = None
        self.stats = GenerationStats()
        self.seq = None                       # cache.SequenceCache once admitted
        self.sampler: Optional[RequestSampler] = None
        self.admission_warned = False
        self.cancelled = False
        self.arrival_time = time.perf_counter()
        self.result: Optional[GenerationResult] = None

    @property
    def done(self) -> bool:
        return self.phase == RequestPhase.COMPLETE
