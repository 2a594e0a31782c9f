"""The one registry: architecture name -> (configuration class, model builder).

``config.json["architectures"][0]`` selects the entry everywhere in the engine
(loader, random-weights writer, command line, trace replay).  A folder without
``architectures`` is matched by its ``model_type``.  The reference has a single
hard-wired check instead (qil/config.py:37, qil/__main__.py:25,33).

An entry's ``build(config, dtype=, device=)`` returns an unloaded model
(``parts.model.CausalLM``): its parts are assembled, its tensors are not filled.
"""
from dataclasses import dataclass
from typing import Callable

from .config.base import ConfigError, read_config_json


@dataclass(frozen=True)
class Architecture:
    name: str
    model_type: str
    config_class: type
    build: Callable


_ARCHITECTURES = {}


def register_architecture(name, *, model_type, config_class, build, replace=False):
    if name in _ARCHITECTURES and not replace:
        raise ValueError(f'architecture {name!r} is already registered')
    _ARCHITECTURES[name] = Architecture(name, model_type, config_class, build)
    return _ARCHITECTURES[name]


def known_architectures():
    _load_builtin()
    return sorted(_ARCHITECTURES)


def architecture_for(data):
    """Entry for a parsed config.json dict."""
    _load_builtin()
    names = data.get('architectures')
    if names:
        if not isinstance(names, list) or not isinstance(names[0], str):
            raise ConfigError("'architectures' must be a list of names")
        if names[0] not in _ARCHITECTURES:
            raise ConfigError(f'unknown architecture {names[0]!r}; known: {sorted(_ARCHITECTURES)}')
        return _ARCHITECTURES[names[0]]
    matches = [a for a in _ARCHITECTURES.values() if a.model_type == data.get('model_type')]
    if len(matches) != 1:
        raise ConfigError(f"config.json names no architecture and model_type {data.get('model_type')!r} "
                          f'selects none; known: {sorted(_ARCHITECTURES)}')
    return matches[0]


def read_model_config(directory):
    """(architecture entry, typed configuration) of a model folder."""
    data = read_config_json(directory)
    entry = architecture_for(data)
    return entry, entry.config_class.from_dict(data)


def _load_builtin():
    from . import models  # noqa: F401  (registers the built-in architecture on import)
