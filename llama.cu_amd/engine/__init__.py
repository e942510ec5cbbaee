"""The step function, the scheduler above it, and the engine that ties them to sampling."""
from .batch import BatchBuilder, StepContext
from ..parts.base import LayerCache
from .config import EngineConfig
from .runner import ModelRunner

__all__ = ["BatchBuilder", "StepContext", "LayerCache", "ModelRunner", "EngineConfig"]
