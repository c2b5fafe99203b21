"""One request as the scheduler sees it (ginfer/engine/sequence.h:12-80, plus what cutting prompts into
portions needs: how many of its tokens are already in the cache)."""
import enum
import time
from dataclasses import dataclass, field
from typing import List, Optional

from ..sampling import SamplingParams


class State(enum.Enum):
    WAITING = 0
    RUNNING = 1
    FINISHED = 2


@dataclass
class Sequence:
    request_id: int
    token_ids: List[int]                 # prompt followed by what was generated
    num_prompt_tokens: int
    params: SamplingParams
    state: State = State.WAITING
    num_computed: int = 0                # tokens whose keys and values are in the cache
    decoding: bool = False               # every known token has been handed to the device; it gets one a step now
    finish_reason: Optional[str] = None
    evictions: int = 0
    request_ts: float = field(default_factory=time.perf_counter)
    first_token_ts: Optional[float] = None
    finish_ts: Optional[float] = None

    @property
    def num_tokens(self):
        return len(self.token_ids)

    @property
    def num_output_tokens(self):
        return len(self.token_ids) - self.num_prompt_tokens

    @property
    def output_ids(self):
        return self.token_ids[self.num_prompt_tokens:]

    @property
    def remaining(self):
        """Known tokens not yet computed; 1 while decoding, more while a prompt (or, after an eviction,
        prompt and output) is still being fed."""
        return len(self.token_ids) - self.num_computed
