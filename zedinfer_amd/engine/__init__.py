from .batch import DeviceBatch, GroupView, StepEntry, build_device_batch
from .engine import Engine, parse_dtype, require_gpu

__all__ = ["DeviceBatch", "GroupView", "StepEntry", "build_device_batch", "Engine", "parse_dtype", "require_gpu"]
