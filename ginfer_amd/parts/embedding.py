"""Token embedding and output head."""
import torch

from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import Part
from .linear import linear
from .registry import register_embedding, register_head


@register_embedding("embedding")
class Embedding(Part):
    """x[t, :] = E[ids[t], :], no scaling (ginfer/core/layer/embedding.cc:5-21); widened to the 32-bit
    residual stream as it is gathered."""

    capturable = True

    def __init__(self, vocab_size, hidden_size, dtype, device):
        self.vocab_size, self.hidden_size, self.dtype, self.device = int(vocab_size), int(hidden_size), dtype, device
        self.weight = None

    def weight_specs(self):
        return {"weight": WeightSpec((self.vocab_size, self.hidden_size))}

    def bind_weights(self, t):
        self.weight = t["weight"]

    def kernel_modules(self):
        return ["embedding"]

    def forward(self, token_ids, step=None):
        return ops.embedding_gather(self.weight, token_ids)


@register_head("lm_head")
class LMHead(Part):
    """logits = x . W^T, no bias, returned in 32-bit; W is the embedding table when tied
    (ginfer/core/layer/transformer/lmhead.cc:15-27, ginfer/model/qwen2.cc:42-46).  One device copy serves
    both uses when tied (the reference uploads it twice)."""

    capturable = True

    def __init__(self, vocab_size, hidden_size, tied, dtype, device):
        self.vocab_size, self.hidden_size, self.tied = int(vocab_size), int(hidden_size), bool(tied)
        self.dtype, self.device = dtype, device
        self.weight = None

    def weight_specs(self):
        return {} if self.tied else {"weight": WeightSpec((self.vocab_size, self.hidden_size))}

    def unread_weights(self):
        # a checkpoint of a tied model may still hold the head's copy of the table; like the reference
        # (ginfer/model/qwen2.cc:42-46) the model does not read it
        return ["weight"] if self.tied else []

    def bind_weights(self, t):
        if not self.tied:
            self.weight = t["weight"]

    def tie(self, embedding_weight):
        self.weight = embedding_weight

    def kernel_modules(self):
        return ["gemm"] + (["gemm_skinny"] if self.dtype == torch.bfloat16 else [])

    def forward(self, x):
        return linear(x, self.weight, None, out_dtype=torch.float32)
