"""llama.cu_amd: a small, whole inference engine for one MI355X (gfx950).

One architecture (the Llama dense decoder), everything between a request's tokens and
its next token: configuration and registry, weights, parts, paged cache, one step
function, scheduler, sampling, and hand-written HIP kernels.
"""
from . import config, parts, models, weights  # noqa: F401
from .config import LlamaConfig, register_architecture
from .parts import register_part

__all__ = ["config", "parts", "models", "weights", "LlamaConfig", "register_architecture", "register_part"]
