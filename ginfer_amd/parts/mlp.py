"""Dense feed-forward with a gated SiLU."""
import torch

from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import Part
from .linear import linear, gated_linear, linear_into_norm
from .registry import register_feed_forward


@register_feed_forward("swiglu")
class SwiGLU(Part):
    """down(silu(gate(x)) * up(x)), no biases (ginfer/core/layer/transformer/feedforward.cc:22-25); gate and
    up are one product over the stacked weights, which equals the two separate ones."""

    capturable = True
    takes_scaled_rows = True
    folds_norm = True

    def __init__(self, hidden_size, intermediate_size, dtype, device):
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.dtype, self.device = dtype, device
        self.w_gate_up = self.w_down = None

    def weight_specs(self):
        H, I = self.hidden_size, self.intermediate_size
        return {"gate_proj.weight": WeightSpec((I, H)), "up_proj.weight": WeightSpec((I, H)),
                "down_proj.weight": WeightSpec((H, I))}

    def bind_weights(self, t):
        self.w_gate_up = torch.cat([t["gate_proj.weight"], t["up_proj.weight"]], dim=0).contiguous()
        self.w_down = t["down_proj.weight"]

    def kernel_modules(self):
        return ["activation", "gemm"] + (["gemm_skinny"] if self.dtype == torch.bfloat16 else [])

    def forward(self, x, into_norm=None):
        """into_norm = (residual, norm): where the down projection's kernel can, the result is added to the
        residual here and the rows of `norm` come back as ops.ScaledRows."""
        act = gated_linear(x, self.w_gate_up)
        if into_norm is not None:
            folded = linear_into_norm(act, self.w_down, None, *into_norm)
            if folded is not None:
                return folded
        # the result may be partial sums of a K-split product: the norm that follows adds them up
        return linear(act, self.w_down, parts_ok=True)
