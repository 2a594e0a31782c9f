"""RMSNorm with float32 statistics.  Formula: qil/model.py:15-23."""
import torch

from .base import Norm, ParamSpec
from .. import ops


class RMSNorm(Norm):
    """y = cast(x * rsqrt(mean(x^2) + eps)) * weight; weight multiplies as stored."""

    def __init__(self, width, eps):
        super().__init__()
        self.width, self.eps = int(width), float(eps)

    def param_specs(self):
        return {'weight': ParamSpec((self.width,), 'vector', 'one_plus_normal')}

    def forward(self, stream, delta, out_dtype):
        return ops.add_rmsnorm(stream, delta, self.p['weight'], self.eps, out_dtype)

    def forward_lazy(self, stream, out_dtype, added):
        if stream.is_cuda and out_dtype == torch.bfloat16 and stream.shape[0] <= ops.NORMED_GEMM_MOST_ROWS:
            return ops.Normed(stream, self.p['weight'], self.eps, out_dtype, added)
        return None

    def forward_rows(self, stream, delta, rows, out_dtype):
        return ops.rows_rmsnorm(stream, delta, rows, self.p['weight'], self.eps, out_dtype)
