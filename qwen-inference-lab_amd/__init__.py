"""MI355X-native inference engine for dense Qwen3 (single GPU).

    from qil_amd import Engine, Qwen3, load_model
    model = Qwen3.from_directory('model_dir', dtype=torch.bfloat16)
    engine = Engine(model, num_pages=256, page_size=16)
    engine.generate([[1, 2, 3]], max_new_tokens=8)

Heavy modules are imported on first use, as in the reference (qil/__init__.py:5-12).
"""
__version__ = '0.1.0'


def __getattr__(name):
    if name == 'Engine':
        from .engine import Engine
        return Engine
    if name == 'Qwen3':
        from .api import Qwen3
        return Qwen3
    if name in ('load_model', 'write_random_model', 'init_random', 'WeightsError'):
        from . import weights
        return getattr(weights, name)
    if name == 'ModelRunner':
        from .engine import ModelRunner
        return ModelRunner
    if name in ('register_architecture', 'known_architectures', 'read_model_config'):
        from . import registry
        return getattr(registry, name)
    raise AttributeError(name)


__all__ = ['Engine', 'Qwen3', 'load_model', 'write_random_model', 'init_random', 'ModelRunner',
           'register_architecture', 'known_architectures', 'read_model_config', 'WeightsError']
