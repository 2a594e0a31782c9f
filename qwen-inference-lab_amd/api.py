"""Python entry points in the reference's manner (qil/model.py:178-179)."""
import torch

from .config.qwen3 import Qwen3Config
from .registry import architecture_for
from .weights import load_model, init_random


class Qwen3:
    """Named constructors of a dense Qwen3 model; the model itself is a ``parts.CausalLM``."""

    @staticmethod
    def from_directory(path, *, device='cuda', dtype=torch.float32):
        """Load a checkpoint folder.  The GPU is the only device (the reference defaults to 'cpu')."""
        if torch.device(device).type != 'cuda':
            raise ValueError("this engine runs on the GPU only: device must be 'cuda'")
        return load_model(path, dtype=dtype, device=device)

    @staticmethod
    def from_config(config, *, seed=0, device='cuda', dtype=torch.bfloat16, on_device=False):
        """Random weights for a configuration (typed or a config.json dict)."""
        data = config if isinstance(config, dict) else config.to_dict()
        entry = architecture_for(data)
        typed = config if not isinstance(config, dict) else entry.config_class.from_dict(data)
        return init_random(entry.build(typed, dtype=dtype, device=device), seed, on_device=on_device)


__all__ = ['Qwen3', 'Qwen3Config']
