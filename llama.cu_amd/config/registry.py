"""One registry from an architecture's name (config.json's ``architectures[0]``) to
its configuration class and to the function that lays its model out of parts.

The reference switches on the architecture name in code
(llama.cu/src/model/mod.rs:62-67: ``"llama"``, ``"qwen2"``, else panic); here the
switch is a table that anyone may add to.
"""
from __future__ import annotations

import importlib
import os
from dataclasses import dataclass
from typing import Any, Callable, Dict, Iterable, List, Tuple

from .base import ConfigError, read_config_json


@dataclass(frozen=True)
class Architecture:
    name: str
    config_from_dict: Callable[[Dict[str, Any]], Any]   # dict of config.json -> typed configuration
    build_spec: Callable[[Any], Any]                    # typed configuration -> parts.ModelSpec
    ignored_tensors: Tuple[str, ...] = ()               # regular expressions: tensors that this architecture's files may
                                                        # carry beside the weights, which the loader passes over


_REGISTRY: Dict[str, Architecture] = {}


def register_architecture(name: str, config_from_dict, build_spec, replace: bool = False,
                          ignored_tensors: Iterable[str] = ()) -> None:
    """``ignored_tensors``: regular expressions (matched from a tensor name's start) for tensors that files of this
    architecture may hold and that are no weights; every other tensor that the model does not expect is an error."""
    if name in _REGISTRY and not replace:
        raise ValueError(f"architecture {name!r} is already registered")
    _REGISTRY[name] = Architecture(name, config_from_dict, build_spec, tuple(ignored_tensors))


def registered_architectures() -> List[str]:
    return sorted(_REGISTRY)


def architecture_of(data: Dict[str, Any], where: str = "config.json") -> Architecture:
    names = data.get("architectures")
    if not isinstance(names, list) or not names or not isinstance(names[0], str):
        raise ConfigError(f"{where}: required key 'architectures' is missing or holds no name")
    arch = _REGISTRY.get(names[0])
    if arch is None:
        raise ConfigError(f"{where}: architecture {names[0]!r} is not registered; "
                          f"registered: {registered_architectures()} (a module that registers another one is "
                          f"named with --plugin or in {PLUGINS_ENV})")
    return arch


PLUGINS_ENV = "LLAMA_CU_AMD_PLUGINS"
_loaded_plugins: List[str] = []


def load_plugins(names: Iterable[str]) -> List[str]:
    """Import the modules ``names`` (found as any module is, on ``sys.path``): modules of the user's that call
    ``register_architecture`` and ``register_part`` when they are imported, so that the command line, the replay
    program and the Python entry point know an architecture or a part that is no file of this package.  A module
    is imported once; one that cannot be imported raises a ConfigError that names it."""
    done = []
    for name in names:
        name = name.strip()
        if not name or name in _loaded_plugins:
            continue
        try:
            importlib.import_module(name)
        except Exception as e:
            raise ConfigError(f"plugin module {name!r} could not be imported: {type(e).__name__}: {e}") from e
        _loaded_plugins.append(name)
        done.append(name)
    return done


def load_plugins_from_env() -> List[str]:
    """The modules named in the environment variable LLAMA_CU_AMD_PLUGINS (separated by commas)."""
    return load_plugins(os.environ.get(PLUGINS_ENV, "").split(","))


def load_config(folder: str):
    """(architecture, typed configuration) of a model folder."""
    data = read_config_json(folder)
    arch = architecture_of(data, where=f"{folder}/config.json")
    return arch, arch.config_from_dict(data)
