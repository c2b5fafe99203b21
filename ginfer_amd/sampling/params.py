"""Sampling options.  `max_tokens` and `ignore_eos` are the reference's, with its defaults
(ginfer/engine/sampling_params.h:5-8); temperature and seed are added (the reference is greedy)."""
from dataclasses import dataclass, field
from typing import List, Optional


@dataclass
class SamplingParams:
    max_tokens: int = 64
    ignore_eos: bool = False
    temperature: float = 0.0          # 0: greedy (argmax, lowest index among equals)
    # with temperature: the n-th output token uses uniform(seed, n); None: a seed of the request's own (its id is the
    # key), so that two requests with the same settings do not draw the same numbers
    seed: Optional[int] = None
    stop_token_ids: Optional[List[int]] = None   # None: the configuration's end-of-sequence ids

    def validate(self):
        if self.max_tokens < 1:
            raise ValueError("max_tokens must be at least 1")
        if self.temperature < 0:
            raise ValueError("temperature must not be negative")
