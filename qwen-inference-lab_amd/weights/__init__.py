"""Weights: strict safetensors loading and seeded random models."""
from .loader import WeightsError, load_weights, load_model
from .random_init import init_random, write_random_model, random_tensor

__all__ = ['WeightsError', 'load_weights', 'load_model', 'init_random', 'write_random_model', 'random_tensor']
