"""Options of the scheduler and the cache, with the reference's names and defaults
(reference: include/zedinfer/scheduler.hpp:42-60)."""
from __future__ import annotations

from dataclasses import dataclass


@dataclass
class SchedulerConfig:
    max_batch_tokens: int = 2048
    max_batch_requests: int = 64
    max_prefill_tokens: int = 512
    max_queue_size: int = 256
    gpu_memory_utilization: float = 0.9
    kv_block_size: int = 16
    # Tokens reserved for generation when a request is admitted: the reference
    # reserves min(max_new_tokens, 256) (reference: src/zedinfer/scheduler.cpp:109-129).
    generation_reserve: int = 256
    # Pages in each cache group's pool; 0 sizes the pool from free device memory.
    num_kv_blocks: int = 0
    # Longest sequence a request may reach (reference: ExecutorConfig.max_seq_len,
    # include/zedinfer/activation.hpp:12-21; 16384 by default there).
    max_seq_len: int = 16384

    def validate(self) -> None:
        for k in ("max_batch_tokens", "max_batch_requests", "max_prefill_tokens", "max_queue_size",
                  "kv_block_size", "max_seq_len"):
            if getattr(self, k) <= 0:
                raise ValueError(f"SchedulerConfig.{k} must be positive, got {getattr(self, k)}")
        if not (0.0 < self.gpu_memory_utilization <= 1.0):
            raise ValueError("SchedulerConfig.gpu_memory_utilization must be in (0, 1]")
        if self.num_kv_blocks < 0 or self.generation_reserve < 0:
            raise ValueError("SchedulerConfig.num_kv_blocks and generation_reserve must be non-negative")
