"""zedinfer_amd: a single-GPU inference engine for MI355X (gfx950).

    from zedinfer_amd import InferenceEngine, GenerationConfig
    engine = InferenceEngine.create("/path/to/model", dtype="bfloat16")
    result = engine.generate_tokens([1, 2, 3], GenerationConfig(max_new_tokens=16))

The op-level surface (``zedinfer_amd.ops``: add, argmax, embedding, linear, rms_norm, rope, swiglu)
follows the reference's Python module.
"""
__version__ = "0.1.0"

from . import models  # noqa: F401  (registers the architectures)
from .config import SchedulerConfig
from .engine import (Engine, GenerationConfig, GenerationResult, InferenceEngine, InferenceRequest, StepEntry)
from .sampling import SamplingParams


def load_model(model_path: str, dtype="bfloat16", scheduler_config=None) -> InferenceEngine:
    """Model, cache, scheduler and sampler from a model folder (``InferenceEngine.create``)."""
    return InferenceEngine.create(model_path, dtype, scheduler_config)


__all__ = ["Engine", "GenerationConfig", "GenerationResult", "InferenceEngine", "InferenceRequest",
           "SamplingParams", "SchedulerConfig", "StepEntry", "load_model", "models"]
