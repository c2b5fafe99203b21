"""Rotary position encoding, NeoX pairing (j, j + rotary_dim/2)."""
import torch

from .base import Part
from .registry import register_position


@register_position("rope_neox")
class RotaryNeoX(Part):
    """Tables sin/cos[p, j] of angle (float)p * inv_freq[j], inv_freq[j] = 1 / theta^(j / half), all in
    32-bit as the reference builds them (ginfer/core/op/kernels/cuda/rope_kernel.cu:13-16 and :61-72),
    computed once on the host and uploaded.  The rotation itself is part of the mixer's kernel
    (ginfer/core/op/kernels/cuda/rope_kernel.cu:83-102)."""

    capturable = True

    style = "neox"

    def __init__(self, theta, rotary_dim, max_positions, dtype=None, device=None):
        if rotary_dim % 2 or rotary_dim <= 0:
            raise ValueError("rotary_dim must be positive and even, got %r" % (rotary_dim,))
        self.theta, self.rotary_dim, self.max_positions = float(theta), int(rotary_dim), int(max_positions)
        self.device = device
        self._tables = None
        self._limit = None

    def limit_positions(self, n):
        """Tables need not be longer than the longest sequence the engine will hold."""
        self._limit = min(self.max_positions, int(n))
        self._tables = None

    @property
    def num_positions(self):
        return self._limit or self.max_positions

    def tables(self):
        """(cos, sin), float32 [num_positions, rotary_dim / 2] on the device."""
        if self._tables is None:
            half = self.rotary_dim // 2
            j = torch.arange(half, dtype=torch.float32)
            inv_freq = 1.0 / torch.pow(torch.tensor(self.theta, dtype=torch.float32), j / float(half))
            p = torch.arange(self.num_positions, dtype=torch.float32)
            ang = p[:, None] * inv_freq[None, :]
            self._tables = (torch.cos(ang).to(self.device).contiguous(), torch.sin(ang).to(self.device).contiguous())
        return self._tables
