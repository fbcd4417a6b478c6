from .batch import DeviceBatch, GroupView, StepEntry, build_device_batch
from .engine import Engine, parse_dtype, require_gpu
from .request import (GenerationConfig, GenerationResult, GenerationStats, InferenceRequest, RequestPhase,
                      resolve_max_new_tokens)
from .scheduler import QueueFull, ScheduledBatch, Scheduler
from .serving import InferenceEngine, ServingLoop

__all__ = ["DeviceBatch", "GroupView", "StepEntry", "build_device_batch", "Engine", "parse_dtype", "require_gpu",
           "GenerationConfig", "GenerationResult", "GenerationStats", "InferenceRequest", "RequestPhase",
           "resolve_max_new_tokens", "QueueFull", "ScheduledBatch", "Scheduler", "InferenceEngine", "ServingLoop"]
