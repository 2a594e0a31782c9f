"""Typed configurations.  One class per architecture; ``registry`` maps names to them."""
from .base import ConfigError, read_config_json
from .qwen3 import Qwen3Config

__all__ = ['ConfigError', 'read_config_json', 'Qwen3Config']
