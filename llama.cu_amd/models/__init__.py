"""Architectures: each module turns its typed configuration into a ModelSpec and
registers itself under the name that config.json's ``architectures`` holds."""
from . import llama  # noqa: F401
