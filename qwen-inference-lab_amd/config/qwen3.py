"""Typed configuration of dense Qwen3, read from its own config.json keys.

Same keys, defaults and rejections as the reference's ``ModelConfig``
(qil/config.py:8-45): eight required positive integers, ``rms_norm_eps`` 1e-6,
``rope_theta`` 1e6, ``attention_bias`` false, ``tie_word_embeddings`` true when
absent, ``eos_token_id`` int | list | null; ``model_type`` must be ``qwen3``;
scaled RoPE, sliding windows, non-full layer types and activations other than
SiLU are refused.  ``torch_dtype`` is kept as information only: weights are
converted to the dtype the caller asks for.
"""
from dataclasses import dataclass, fields, asdict

from .base import (ConfigError, read_config_json, check_positive_int,
                   check_positive_finite, check_bool)

_REQUIRED = ('vocab_size', 'hidden_size', 'intermediate_size', 'num_hidden_layers',
             'num_attention_heads', 'num_key_value_heads', 'head_dim', 'max_position_embeddings')


@dataclass(frozen=True)
class Qwen3Config:
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    max_position_embeddings: int
    rms_norm_eps: float = 1e-6            # qil/config.py:18
    rope_theta: float = 1000000.          # qil/config.py:19
    attention_bias: bool = False          # qil/config.py:20
    tie_word_embeddings: bool = True      # qil/config.py:21 (default when the key is absent)
    eos_token_id: int | list | None = None
    torch_dtype: str | None = None        # what the checkpoint says it was saved in; the caller's dtype decides

    architecture = 'Qwen3ForCausalLM'
    model_type = 'qwen3'

    def __post_init__(self):
        for name in _REQUIRED:                                       # qil/config.py:25-28
            check_positive_int(name, getattr(self, name))
        if self.num_attention_heads % self.num_key_value_heads:      # qil/config.py:29-30
            raise ConfigError('num_attention_heads must be a multiple of num_key_value_heads')
        if self.head_dim % 2:
            raise ConfigError('head_dim must be even (rotary pairs)')
        check_positive_finite('rms_norm_eps', self.rms_norm_eps)     # qil/config.py:31-32
        check_positive_finite('rope_theta', self.rope_theta)
        check_bool('attention_bias', self.attention_bias)
        check_bool('tie_word_embeddings', self.tie_word_embeddings)
        eos = self.eos_token_id
        ids = eos if isinstance(eos, list) else [] if eos is None else [eos]
        if any(type(t) is not int or not 0 <= t for t in ids):
            raise ConfigError('eos_token_id must be an integer, a list of integers or null')
        if isinstance(eos, list):
            object.__setattr__(self, 'eos_token_id', list(eos))
        if self.torch_dtype is not None and not isinstance(self.torch_dtype, str):
            raise ConfigError('torch_dtype must be a string or null')

    @property
    def eos_ids(self):
        eos = self.eos_token_id
        return frozenset(eos if isinstance(eos, list) else [] if eos is None else [eos])

    @classmethod
    def from_dict(cls, data):
        if data.get('model_type') != cls.model_type:                 # qil/config.py:37-38
            raise ConfigError(f"model_type must be 'qwen3' (dense text model), got {data.get('model_type')!r}")
        if data.get('rope_scaling') is not None:                     # qil/config.py:39-40
            raise ConfigError('rope_scaling is not supported')
        if data.get('use_sliding_window', False):
            raise ConfigError('use_sliding_window is not supported')
        if any(t != 'full_attention' for t in data.get('layer_types') or []):   # qil/config.py:41-42
            raise ConfigError('every layer must be full_attention')
        if data.get('hidden_act', 'silu') != 'silu':                 # qil/config.py:43-44
            raise ConfigError("hidden_act must be 'silu'")
        missing = [name for name in _REQUIRED if name not in data]
        if missing:
            raise ConfigError(f'config.json lacks required keys: {missing}')
        return cls(**{f.name: data[f.name] for f in fields(cls) if f.name in data})

    @classmethod
    def read(cls, directory):
        return cls.from_dict(read_config_json(directory))

    def to_dict(self):
        data = asdict(self)
        data.update(architectures=[self.architecture], model_type=self.model_type, hidden_act='silu')
        return data
