"""RMSNorm fused with the residual add that precedes it."""
import torch

from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import Part
from .registry import register_norm


@register_norm("rmsnorm")
class RMSNorm(Part):
    """y = (h * g) / sqrt(mean(h^2) + eps) with h = residual + delta; plain gain, no bias, no mean
    subtraction (ginfer/core/op/kernels/cuda/rmsnorm_kernel.cu:27-66, ginfer/core/layer/rmsnorm.cc:6-22)."""

    capturable = True
    accepts_partial_sums = True
    foldable = True          # a plain gain over the root mean square: the products around it can fold it

    def __init__(self, size, eps, dtype, device):
        self.size, self.eps, self.dtype, self.device = int(size), float(eps), dtype, device
        self.weight = None

    def weight_specs(self):
        return {"weight": WeightSpec((self.size,), init="one_plus_normal", keep_32bit=True)}

    def bind_weights(self, tensors):
        self.weight = tensors["weight"]

    def kernel_modules(self):
        return ["norm"]

    def forward(self, residual, delta=None, rows=None):
        return ops.add_rmsnorm(residual, delta, self.weight, self.eps, self.dtype, rows=rows)
