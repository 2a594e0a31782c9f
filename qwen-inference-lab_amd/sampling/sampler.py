"""Next-token choice: greedy or seeded temperature sampling, on the GPU.

Greedy is the reference's sampler: an all-finite check, then argmax with the
lowest index on ties (qil/engine.py:96-100).  Temperature sampling is not in the
reference: a request has a temperature and a seed, and its k-th output token is
drawn from softmax(logits / T) with uniforms keyed by (seed, k), so the draw
depends neither on the batch nor on how the work was cut.
"""
from dataclasses import dataclass

import numpy as np
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
    """``sample`` is the whole thing for logits in hand.  A step function that wants the draw inside its
    own launch sequence (a captured graph, say) uses the three pieces: ``pack`` on the host, ``draw`` on
    the device, ``unpack`` on the host."""

    def pack(self, params, counters):
        """int32 [3, M] host array: seeds, output indices, temperatures (their float32 bits)."""
        if len(params) != len(counters):
            raise ValueError('one SamplingParams and one counter per row of logits')
        packed = np.empty((3, len(params)), dtype=np.int32)
        packed[0] = [_int32(p.seed) for p in params]
        packed[1] = [_int32(c) for c in counters]
        packed[2] = np.asarray([p.temperature for p in params], dtype=np.float32).view(np.int32)
        return packed

    def draw(self, logits, packed, out):
        """Device only: ``packed`` int32 [3, M] as ``pack`` makes it, ``out`` int32 [2, M] (tokens, finite flags)."""
        ops.sample(logits, packed[2].view(torch.float32), packed[0], packed[1], out=out)

    def unpack(self, out):
        """Tokens from the host copy of ``out`` ([2, M] nested lists); refuses rows with non-finite logits."""
        tokens, finite = out
        if not all(finite):
            raise RuntimeError('model returned non-finite logits')
        return tokens

    def sample(self, logits, params, counters):
        """logits float32 [M, V] on the GPU; params: SamplingParams per row; counters: output index per row."""
        if logits.shape[0] != len(params):
            raise ValueError('one SamplingParams and one counter per row of logits')
        packed = torch.from_numpy(self.pack(params, counters)).to(logits.device)
        out = torch.empty((2, logits.shape[0]), dtype=torch.int32, device=logits.device)
        self.draw(logits, packed, out)
        return self.unpack(out.tolist())
