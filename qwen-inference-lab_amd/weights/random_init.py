"""Random weights from a configuration and a seed (the reference has no such mode).

Matrices and biases N(0, 0.02); norm scales 1 + N(0, 0.01).  Every tensor has a
generator of its own, seeded by (seed, tensor name), so a tensor's values do not
depend on which other tensors exist or in which order they are made.
"""
import json
import zlib
from pathlib import Path

import torch

from ..registry import architecture_for
from .loader import placement_dtype

MATRIX_STD = 0.02
NORM_STD = 0.01


def _generator(seed, name, device):
    g = torch.Generator(device=device)
    g.manual_seed((int(seed) * 1000003 + zlib.crc32(name.encode())) % (2 ** 63))
    return g


def random_tensor(spec, seed, name, device='cpu'):
    """float32 tensor of the spec's shape on ``device``."""
    if spec.kind == 'table':
        raise ValueError('integer tables have no random initialiser')
    if spec.init == 'zeros':
        return torch.zeros(spec.shape, dtype=torch.float32, device=device)
    noise = torch.randn(spec.shape, generator=_generator(seed, name, device), dtype=torch.float32, device=device)
    return 1.0 + NORM_STD * noise if spec.init == 'one_plus_normal' else MATRIX_STD * noise


def init_random(model, seed, *, on_device=False):
    """Fill a built model in place.  ``on_device`` draws with the device's generator
    (fast for billions of values; values then differ from the CPU's)."""
    where = model.device if on_device else 'cpu'
    for name, (part, local) in model.names.items():
        spec = part.param_specs()[local]
        tensor = random_tensor(spec, seed, name, where).to(placement_dtype(spec, model.dtype))
        part.set_param(local, tensor.to(model.device).contiguous())
    model.finalize()
    return model


def write_random_model(directory, config, seed, *, dtype=torch.bfloat16):
    """Write ``config.json`` and ``model.safetensors`` for a configuration.

    ``config`` is a typed configuration or a config.json dict.  Tensors are stored
    in ``dtype``; stored as bfloat16, a float32 and a bfloat16 engine read exactly
    the same values.
    """
    from safetensors.torch import save_file
    data = config if isinstance(config, dict) else config.to_dict()
    entry = architecture_for(data)
    typed = entry.config_class.from_dict(data)
    model = entry.build(typed, dtype=dtype, device='cpu')
    tensors = {}
    for name, (part, local) in model.names.items():
        spec = part.param_specs()[local]
        tensors[name] = random_tensor(spec, seed, name).to(dtype).contiguous()
    directory = Path(directory)
    directory.mkdir(parents=True, exist_ok=True)
    (directory / 'config.json').write_text(json.dumps(data, indent=2) + '\n')
    save_file(tensors, str(directory / 'model.safetensors'))
    return directory
