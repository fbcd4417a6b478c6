from . import qwen2  # noqa: F401  (registers the architecture)
from .model import DecoderModel, expected_weights

__all__ = ["DecoderModel", "expected_weights", "qwen2"]
