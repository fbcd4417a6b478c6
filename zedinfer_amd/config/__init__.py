from .model_config import ConfigError, ModelConfig, Qwen2Config, read_config_json
from .forward_config import (LayerSpec, ModelForwardConfig, PartSpec, ScheduleStep,
                             default_schedule)
from .registry import (Architecture, find_architecture, load_config, register_architecture,
                       registered_architectures)
from .scheduler_config import SchedulerConfig

__all__ = [
    "ConfigError", "ModelConfig", "Qwen2Config", "read_config_json", "LayerSpec",
    "ModelForwardConfig", "PartSpec", "ScheduleStep", "default_schedule", "Architecture",
    "find_architecture", "load_config", "register_architecture", "registered_architectures",
    "SchedulerConfig",
]
