"""Strict loading of safetensors by tensor name.

Every file ``*.safetensors`` of the folder is read in sorted order, as the
reference does (qil/model.py:184-191; no index file is consulted).  All faults
are collected and raised as ONE ``WeightsError`` that lists missing tensors,
unexpected or duplicate names, wrong shapes and inconsistent tied tensors
(reference: separate ValueErrors, qil/model.py:185-205).

Placement: matrices take the model's dtype (qil/model.py:197); norm scales and
biases are held in float32, which keeps a bfloat16 or a float32 file value
exactly; integer tables become int32.
"""
from pathlib import Path

import torch

from ..registry import read_model_config


class WeightsError(ValueError):
    pass


_FLOATS = {'F64', 'F32', 'F16', 'BF16'}
_INTS = {'I64', 'I32', 'I16', 'I8', 'U8'}


def placement_dtype(spec, model_dtype):
    return {'matrix': model_dtype, 'vector': torch.float32, 'table': torch.int32}[spec.kind]


def load_weights(model, directory):
    """Fill ``model`` (built, not loaded) from the folder's safetensors files."""
    from safetensors import safe_open
    files = sorted(Path(directory).glob('*.safetensors'))
    if not files:
        raise WeightsError(f'no *.safetensors file in {directory}')

    names, tied = model.names, model.tied
    where, unexpected, duplicate, wrong_shape, wrong_type = {}, [], [], [], []
    for file in files:
        with safe_open(str(file), framework='pt', device='cpu') as shard:
            for name in shard.keys():
                canonical = tied.get(name, name)
                if canonical not in names:
                    unexpected.append(name)
                    continue
                if name in where:
                    duplicate.append(name)
                    continue
                part, local = names[canonical]
                spec = part.param_specs()[local]
                view = shard.get_slice(name)
                shape, stored = tuple(view.get_shape()), view.get_dtype()
                if shape != tuple(spec.shape):
                    wrong_shape.append(f'{name}: file {list(shape)}, model {list(spec.shape)}')
                if stored not in (_INTS if spec.kind == 'table' else _FLOATS):
                    wrong_type.append(f'{name}: stored as {stored}')
                where[name] = file
    present = {tied.get(name, name) for name in where}
    missing = sorted(name for name in names if name not in present)
    problems = []
    if missing:
        problems.append(f'missing tensors ({len(missing)}): {missing}')
    if unexpected:
        problems.append(f'unexpected tensors ({len(unexpected)}): {sorted(unexpected)}')
    if duplicate:
        problems.append(f'tensors present in more than one file: {sorted(duplicate)}')
    if wrong_shape:
        problems.append(f'wrong shapes ({len(wrong_shape)}): {wrong_shape}')
    if wrong_type:
        problems.append(f'wrong element types: {wrong_type}')
    if problems:
        raise WeightsError(f'cannot load {directory}: ' + '; '.join(problems))

    by_file = {}
    for name, file in where.items():
        by_file.setdefault(file, []).append(name)
    held = {}          # canonical name -> CPU tensor in placement dtype, kept only while an alias may follow
    inconsistent = []
    aliased = set(tied.values())
    for file in files:
        with safe_open(str(file), framework='pt', device='cpu') as shard:
            for name in by_file.get(file, ()):
                canonical = tied.get(name, name)
                part, local = names[canonical]
                target = placement_dtype(part.param_specs()[local], model.dtype)
                tensor = shard.get_tensor(name).to(target)
                if canonical in held:                       # second name of a tied tensor
                    if not torch.equal(held[canonical], tensor):   # qil/model.py:198-199
                        inconsistent.append(f'{name} differs from {canonical}')
                    continue
                if canonical in aliased:
                    held[canonical] = tensor
                part.set_param(local, tensor.to(model.device).contiguous())
    if inconsistent:
        raise WeightsError(f'cannot load {directory}: inconsistent tied tensors: {inconsistent}')
    model.finalize()
    return model


def load_model(directory, *, dtype=torch.bfloat16, device='cuda'):
    """Model folder -> loaded model; the class is chosen by config.json through the registry."""
    entry, config = read_model_config(directory)
    model = entry.build(config, dtype=dtype, device=device)
    return load_weights(model, directory)
