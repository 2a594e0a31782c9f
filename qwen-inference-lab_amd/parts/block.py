"""Pre-norm residual arrangement: norm -> sub-layer -> add to the un-normalised stream.

Two sub-layers per block, mixer then feed-forward (qil/model.py:48-71).  The
stream is float32 and every residual sum is made in float32; the add of a
sub-layer's output is fused into the norm that follows it.
"""
from .base import Block
from .. import ops


class PreNormBlock(Block):
    def __init__(self, *, mixer_norm, mixer, ffn_norm, ffn, dtype, names=None):
        super().__init__()
        self.mixer_norm, self.mixer, self.ffn_norm, self.ffn, self.dtype = mixer_norm, mixer, ffn_norm, ffn, dtype
        self._names = names or dict(mixer_norm='mixer_norm', mixer='mixer', ffn_norm='ffn_norm', ffn='ffn')

    def parts(self):
        n = self._names
        return {n['mixer_norm']: self.mixer_norm, n['mixer']: self.mixer,
                n['ffn_norm']: self.ffn_norm, n['ffn']: self.ffn}

    def forward(self, stream, pending, ctx, cache):
        h = None
        if isinstance(pending, ops.Added):                     # the stream is complete
            if self.mixer.takes_lazy_norm:                     # the mixer's first product may make the norm itself
                h = self.mixer_norm.forward_lazy(stream, self.dtype, pending)
            pending = None
        if h is None:
            h = self.mixer_norm.forward(stream, pending, self.dtype)
        mixed = self.mixer.forward(h, ctx, cache)
        h = self.ffn_norm.forward(stream, None if isinstance(mixed, ops.Added) else mixed, self.dtype)
        return self.ffn.forward(h, add_to=stream) if self.ffn.adds_to_stream else self.ffn.forward(h)
