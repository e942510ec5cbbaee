"""Typed configurations, read from a model folder's config.json, and the registry
that maps an architecture's name to its configuration class and its model."""
from .base import ConfigError, read_config_json
from .llama import LlamaConfig
from .registry import (Architecture, architecture_of, register_architecture, registered_architectures, load_config,
                       load_plugins, load_plugins_from_env, PLUGINS_ENV)

__all__ = ["ConfigError", "read_config_json", "LlamaConfig", "Architecture", "architecture_of",
           "register_architecture", "registered_architectures", "load_config", "load_plugins", "load_plugins_from_env",
           "PLUGINS_ENV"]
