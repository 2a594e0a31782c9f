"""Rotary position encoding: float32 tables built on the CPU.

inv_freq[i] = 1 / theta**(2i/rot_dim) is computed on the CPU in float32 with the
positive exponent and a reciprocal, and the angle is float32(position) * inv_freq
(qil/model.py:99-108).  Computing theta**(-e), or computing on the GPU, crosses
bfloat16 rounding edges of cos/sin (docs/OPTIMIZATION_DEBUG_LOG.md:23-33).  The
tables stay float32 whatever the model's dtype.  Pairing is (i, i + rot_dim/2)
(qil/model.py:42-46).
"""
import torch

from .base import PositionEncoding, Rotation


class Rotary(PositionEncoding):
    def __init__(self, head_dim, theta, max_positions, *, rot_dim=None, device='cpu'):
        super().__init__()
        self.head_dim, self.theta, self.max_positions = int(head_dim), float(theta), int(max_positions)
        self.rot_dim = self.head_dim if rot_dim is None else int(rot_dim)
        if self.rot_dim % 2 or not 0 < self.rot_dim <= self.head_dim:
            raise ValueError('rot_dim must be even and at most head_dim')
        self.device = device
        self._rotation = None

    def angles(self, positions):
        exponent = torch.arange(0, self.rot_dim, 2, device='cpu', dtype=torch.float32) / self.rot_dim
        inv_freq = 1.0 / (self.theta ** exponent)
        return positions.to('cpu', torch.float32)[:, None] * inv_freq[None, :]

    def rotation(self):
        if self._rotation is None:
            angles = self.angles(torch.arange(self.max_positions))
            self._rotation = Rotation(angles.cos().to(self.device).contiguous(),
                                      angles.sin().to(self.device).contiguous(), self.rot_dim)
        return self._rotation
