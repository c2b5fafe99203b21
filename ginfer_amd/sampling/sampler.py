"""Next tokens from logits, on the device."""
import numpy as np
import torch

from ..kernels import ops
from .rng import uniform, request_seed


class Sampler:
    def __init__(self, device):
        self.device = device

    def sample(self, logits, params, output_positions, request_ids=None):
        """logits float32 [R, V]; params: R SamplingParams; output_positions: which output token of its
        request each row decides (indexes the request's random stream); request_ids: the key of the stream of a
        request whose parameters name no seed.  Returns a list of R ints."""
        out = self.sample_on_device(logits, params, output_positions, request_ids)
        return [] if out is None else out.cpu().tolist()

    def sample_on_device(self, logits, params, output_positions, request_ids=None):
        """As sample(), but the tokens stay on the device: int32 [R] (None for no rows).  Nothing waits."""
        R = logits.shape[0]
        if R == 0:
            return None
        if all(p.temperature <= 0 for p in params):
            return ops.sample_rows(logits)
        temp = torch.tensor([float(p.temperature) for p in params], dtype=torch.float32, device=self.device)
        ids = request_ids if request_ids is not None else [0] * R
        uni = torch.tensor(np.asarray([uniform(p.seed if p.seed is not None else request_seed(rid), n)
                                       for p, n, rid in zip(params, output_positions, ids)], dtype=np.float32),
                           device=self.device)
        return ops.sample_rows(logits, temp, uni)
