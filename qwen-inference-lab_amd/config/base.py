"""Helpers shared by every architecture's typed configuration.

A configuration class is a frozen dataclass whose fields are the config.json keys
the architecture reads.  It offers ``from_dict(data)``, ``read(directory)`` and
``to_dict()``; nothing else in the engine reads config.json.
"""
import json
import math
from pathlib import Path


class ConfigError(ValueError):
    """config.json is missing, malformed, or asks for something unsupported."""


def read_config_json(directory):
    path = Path(directory) / 'config.json'
    if not path.is_file():
        raise ConfigError(f'no config.json in {directory}')
    try:
        data = json.loads(path.read_text())
    except json.JSONDecodeError as error:
        raise ConfigError(f'{path}: not valid JSON ({error})') from None
    if not isinstance(data, dict):
        raise ConfigError(f'{path}: top level must be an object')
    return data


def check_positive_int(name, value):
    if type(value) is not int or value < 1:
        raise ConfigError(f'{name} must be a positive integer, got {value!r}')


def check_positive_finite(name, value):
    if isinstance(value, bool) or not isinstance(value, (int, float)) or not math.isfinite(value) or value <= 0:
        raise ConfigError(f'{name} must be positive and finite, got {value!r}')


def check_bool(name, value):
    if type(value) is not bool:
        raise ConfigError(f'{name} must be true or false, got {value!r}')
