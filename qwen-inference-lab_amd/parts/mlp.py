"""Gated feed-forward: down(act(gate(x)) * up(x)).  Formula: qil/model.py:71."""
import torch

from .base import FeedForward, ParamSpec
from .. import ops


class GatedMLP(FeedForward):
    """``activation`` names the gate's function; 'silu' (z * sigmoid(z)) is the one
    the kernels have.  Gate and up matrices become one [2 * intermediate, width] matrix at
    ``finalize`` (rows in turns of 16, or gate rows first where the sizes do not allow that): a pure re-layout."""

    def __init__(self, *, width, intermediate, activation='silu', dtype=torch.bfloat16):
        super().__init__()
        self.dtype = dtype
        if activation != 'silu':
            raise ValueError(f'no kernel for activation {activation!r}')
        self.width, self.intermediate, self.activation = width, intermediate, activation

    def param_specs(self):
        return {'gate_proj.weight': ParamSpec((self.intermediate, self.width)),
                'up_proj.weight': ParamSpec((self.intermediate, self.width)),
                'down_proj.weight': ParamSpec((self.width, self.intermediate))}

    def finalize(self):
        p = self.p
        gate, up = p.pop('gate_proj.weight'), p.pop('up_proj.weight')
        # on the GPU, rows in turns of 16 where the sizes allow (the kernels read a gate tile and its up tile side by side)
        self.interleaved = self.intermediate % 16 == 0 and gate.is_cuda
        p['gate_up_proj.weight'] = ops.interleave_gate_up(gate, up) if self.interleaved else torch.cat([gate, up]).contiguous()

    adds_to_stream = True

    def forward(self, h, add_to=None):
        hidden = ops.gated_linear(h, self.p['gate_up_proj.weight'], self.dtype, interleaved=self.interleaved, lazy=True)
        if add_to is not None and hidden.is_cuda:              # few rows: the down product adds into the stream itself
            return ops.linear(hidden, self.p['down_proj.weight'], None, partials=True, add_to=add_to)
        return ops.linear(hidden, self.p['down_proj.weight'], None, partials=True)
