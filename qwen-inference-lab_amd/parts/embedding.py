"""Token embedding into the float32 stream, and the output head."""
from .base import Part, ParamSpec
from .. import ops


class Embedding(Part):
    """stream[n] = float32(table[token[n]]), no scaling (qil/model.py:126)."""

    def __init__(self, vocab, width):
        super().__init__()
        self.vocab, self.width = vocab, width

    def param_specs(self):
        return {'weight': ParamSpec((self.vocab, self.width))}

    def forward(self, token_ids):
        return ops.embed(token_ids, self.p['weight'])

    def forward_step(self, ctx):
        """The float32 stream [N, width] of a step's rows.  What the model calls; an embedding that also needs
        the rows' positions (learned absolute positions, say) finds them in ``ctx`` (engine/batch.py)."""
        return self.forward(ctx.token_ids)


class LMHead(Part):
    """float32 logits = rows @ weight^T, no bias (qil/model.py:134).

    ``tied_to`` names an Embedding whose table is the head's matrix too
    (qil/model.py:96-98); the head then declares no tensor of its own.
    """

    def __init__(self, vocab, width, tied_to=None):
        super().__init__()
        self.vocab, self.width, self.tied_to = vocab, width, tied_to

    def param_specs(self):
        return {} if self.tied_to is not None else {'weight': ParamSpec((self.vocab, self.width))}

    @property
    def weight(self):
        return self.tied_to.p['weight'] if self.tied_to is not None else self.p['weight']

    def forward(self, rows):
        import torch
        return ops.linear(rows, self.weight, None, out_dtype=torch.float32)
