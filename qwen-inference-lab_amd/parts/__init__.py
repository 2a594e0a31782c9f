"""Parts that models are assembled from."""
from .base import (ParamSpec, KVNeed, PagedNeed, StateNeed, Part, Norm, PositionEncoding, Rotation,
                   Mixer, FeedForward, Block)
from .norm import RMSNorm
from .rotary import Rotary
from .attention import Attention
from .mlp import GatedMLP
from .block import PreNormBlock
from .embedding import Embedding, LMHead
from .model import CausalLM, ScheduleEntry

__all__ = ['ParamSpec', 'KVNeed', 'PagedNeed', 'StateNeed', 'Part', 'Norm', 'PositionEncoding', 'Rotation', 'Mixer',
           'FeedForward', 'Block', 'RMSNorm', 'Rotary', 'Attention', 'GatedMLP', 'PreNormBlock',
           'Embedding', 'LMHead', 'CausalLM', 'ScheduleEntry']
