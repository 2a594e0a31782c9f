"""Next-token choice: greedy or seeded temperature sampling, on the GPU.

Greedy is the reference's sampler: an all-finite check, then argmax with the
lowest index on ties (qil/engine.py:96-100).  Temperature sampling is not in the
reference: a request has a temperature and a seed, and its k-th output token is
drawn from softmax(logits / T) with uniforms keyed by (seed, k), so the draw
depends neither on the batch nor on how the work was cut.
"""
from dataclasses import dataclass

import torch

from .. import ops


@dataclass(frozen=True)
class SamplingParams:
    temperature: float = 0.0
    seed: int = 0

    def __post_init__(self):
        if isinstance(self.temperature, bool) or not isinstance(self.temperature, (int, float)) \
                or self.temperature != self.temperature or self.temperature < 0 or self.temperature == float('inf'):
            raise ValueError('temperature must be a finite number >= 0')
        if type(self.seed) is not int:
            raise ValueError('seed must be an integer')


def _int32(value):
    value &= 0xFFFFFFFF
    return value - (1 << 32) if value >= (1 << 31) else value


class Sampler:
    def sample(self, logits, params, counters):
        """logits float32 [M, V] on the GPU; params: SamplingParams per row; counters: output index per row."""
        rows = logits.shape[0]
        if rows != len(params) or rows != len(counters):
            raise ValueError('one SamplingParams and one counter per row of logits')
        host = torch.tensor([[_int32(p.seed) for p in params], [_int32(c) for c in counters]], dtype=torch.int32)
        meta = host.to(logits.device)
        temperatures = torch.tensor([float(p.temperature) for p in params], dtype=torch.float32).to(logits.device)
        tokens, finite = ops.sample(logits, temperatures, meta[0].contiguous(), meta[1].contiguous())
        result = torch.stack((tokens, finite)).tolist()
        if not all(result[1]):
            raise RuntimeError('model returned non-finite logits')
        return result[0]
