"""The engine: requests in, token ids out.  Field names of the configuration are the reference's
(ginfer/engine/config.h:8-21); `generate` and `step` follow ginfer/engine/engine.cc:93-151, without the
tokenizer: prompts are lists of token ids and so are the results."""
import collections
import time
from dataclasses import dataclass

import torch
from typing import List, Optional

from ..kernels.tuning import TUNING
from ..sampling import SamplingParams, Sampler
from .runner import ModelRunner, StepEntry
from .scheduler import Scheduler
from .sequence import Sequence


@dataclass
class EngineConfig:
    model_path: Optional[str]             # folder with config.json and the weights; None: model_config and random_seed
    dtype: str = "bfloat16"               # "bfloat16" or "float32" (everything in true 32-bit)
    max_num_batched_tokens: int = 2048    # token budget of one step
    max_num_seqs: int = 64                # requests running at a time
    max_seq_len: int = 4096               # longest sequence (prompt + output) a request may reach
    gpu_memory_utilization: float = 0.9   # share of the free device memory that becomes cache pages
    kvcache_block_size: int = 16          # tokens per cache page
    # pages per cache group; None: from the memory that is free with the weights loaded, times gpu_memory_utilization;
    # groups of layers with a window then get only what a window can hold, the others share the rest
    num_kvcache_blocks: Optional[int] = None
    pipeline_decode: bool = True          # launch a decode step before the tokens of the step before it are read
    # requests share the cache pages of a common prefix (ginfer/engine/block_manager.cc:63-110, where it cannot be
    # switched off).  None: wherever the model allows it (no window, no per-request state); True: or refuse
    enable_prefix_caching: Optional[bool] = None
    # without a model folder: a typed configuration (the reference's `model_config` field, ginfer/engine/config.h:8-21)
    # and the seed that its weights are drawn from on the device
    model_config: Optional[object] = None
    random_seed: Optional[int] = None
    # one portion of a prompt and one decoded token run through the model when the engine starts, so that the first
    # request does not pay for what is set up at a kernel's or a library's first call
    # (ginfer/engine/model_runner.cc:34-50 warms up with one token)
    warmup: bool = True
    # steps with prompt portions of up to 512 token rows are laid into recorded steps of padded sizes: their launches
    # would cost the host more than the device works on them
    graph_mixed_steps: bool = True
    # a tensor in the model folder that the model does not read: an error instead of a warning
    strict_weights: bool = False
    # before a step of some number of rows is recorded, the products that can be done in several ways are timed in
    # each, on this model's own weights, and the fastest kept (a second or so per number of rows, once)
    autotune: bool = False


@dataclass
class RequestOutput:
    request_id: int
    prompt_token_ids: List[int]
    token_ids: List[int]
    finish_reason: str
    ttft: Optional[float]
    tpot: Optional[float]
    evictions: int


class Engine:
    def __init__(self, config: EngineConfig):
        self.config = config
        self.runner = ModelRunner(config.model_path, dtype=config.dtype, page_size=config.kvcache_block_size,
                                  num_pages=config.num_kvcache_blocks, max_requests=config.max_num_seqs,
                                  max_model_len=config.max_seq_len,
                                  max_num_batched_tokens=config.max_num_batched_tokens,
                                  gpu_memory_utilization=config.gpu_memory_utilization,
                                  prefix_caching=config.enable_prefix_caching,
                                  graph_mixed_steps=config.graph_mixed_steps,
                                  strict_weights=config.strict_weights, autotune=config.autotune,
                                  config=config.model_config if config.model_path is None else None,
                                  random_seed=config.random_seed if config.model_path is None else None)
        self.scheduler = Scheduler(self.runner.cache, config.max_num_seqs, config.max_num_batched_tokens,
                                   self.runner.spec.eos_token_ids, self.runner.max_model_len)
        self.sampler = Sampler(self.runner.device)
        self._next_id = 0
        self._launched = None            # a step that is on the device and whose tokens have not been read yet
        # sampled tokens come to the host through pinned buffers, each with an event: a step's tokens can then be
        # waited for while the step launched after it is still running
        self._token_ring = [(torch.empty(max(config.max_num_seqs, 1), dtype=torch.int32, pin_memory=True),
                             torch.cuda.Event()) for _ in range(4)]
        self._ring_at = 0
        self.stats = dict(prefill_tokens=0, prefill_time=0.0, decode_tokens=0, decode_time=0.0, steps=0,
                          steps_launched_ahead=0, device_time=0.0)
        # one record a step: wall time of Engine.step, the device's own time for the step's kernels (model and sampling,
        # between two events on the stream) and the step's tokens; the reference accounts wall time only
        # (ginfer/engine/engine.cc:93-121)
        self.step_log = collections.deque(maxlen=1 << 16)      # the last 65,536 steps
        self.last_logits = None          # the logits of the step launched last (a buffer that the next step overwrites)
        if config.warmup:
            self._warm_up()

    def _warm_up(self):
        """Prompt portions of several lengths (the library picks other kernels for other numbers of rows, and loads each
        at its first use), then decoded tokens, with sampling, through the model's own step; the request is given
        back afterwards and leaves nothing behind (it is admitted without its tokens, so no page of it is remembered)."""
        runner, cfg = self.runner, self.config
        room = min(runner.max_model_len - 3, cfg.max_num_batched_tokens,
                   min(g.pool.num_free for g in runner.cache.groups) * runner.page_size - 3 if runner.cache.groups else 1 << 30)
        rid = ("warm-up",)
        greedy = [SamplingParams()]
        try:
            done = set()
            for n in TUNING.warmup_portion_lengths:
                n = min(n, room)
                if n < 1 or n in done:
                    continue
                done.add(n)
                # short portions three times: the second run records the padded step that a lone prompt of about this
                # length will be laid into, the third replays it
                runs = 3 if n < TUNING.warmup_record_below else 1
                for k in range(runs):
                    logits = runner.step([StepEntry(rid, [0] * n, [n - 1])], borrow=True)
                    self.sampler.sample_on_device(logits, greedy, [0])
                    if len(done) == 1 and k == runs - 1:
                        for _ in range(2):
                            logits = runner.step([StepEntry(rid, [0], [0])], borrow=True)
                            self.sampler.sample_on_device(logits, greedy, [0])
                    runner.release(rid)
            torch.cuda.synchronize()
        finally:
            runner.release(rid)

    def add_request(self, prompt_token_ids, params: Optional[SamplingParams] = None):
        params = params or SamplingParams()
        params.validate()
        ids = [int(t) for t in prompt_token_ids]
        V = self.runner.vocab_size
        if any(not 0 <= t < V for t in ids):
            raise ValueError("prompt holds a token id outside [0, %d)" % V)
        rid = self._next_id
        self._next_id += 1
        self.scheduler.add(Sequence(rid, ids, len(ids), params))
        return rid

    def abort(self, request_id) -> Optional[RequestOutput]:
        """Ends a request now, wherever it stands; returns what it has produced, or None if it is not alive."""
        seq = self.scheduler.abort(request_id, time.perf_counter())
        return None if seq is None else self._output(seq)

    def has_unfinished(self):
        return self._launched is not None or not self.scheduler.is_finished()

    def _launch(self, scheduled, device_tokens=None):
        """Hands a scheduled step to the device: model step and sampling are queued, nothing is waited for.
        device_tokens: the ids of single-token items that are still on the device (a step launched ahead)."""
        entries = []
        for sc in scheduled:
            s = sc.seq
            toks = [0] if device_tokens is not None else s.token_ids[s.num_computed:s.num_computed + sc.num_tokens]
            entries.append(StepEntry(s.request_id, toks, [sc.num_tokens - 1] if sc.samples else []))
        began, ended = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        began.record()
        logits = self.runner.step(entries, borrow=True, device_tokens=device_tokens)
        self.last_logits = logits
        sampling = [sc.seq for sc in scheduled if sc.samples]
        ahead = 1 if device_tokens is not None else 0      # the token before is not in the request's list yet
        tokens = self.sampler.sample_on_device(logits, [s.params for s in sampling],
                                               [s.num_output_tokens + ahead for s in sampling],
                                               [s.request_id for s in sampling])
        ended.record()
        arrival = None
        if tokens is not None:               # the copy to the host is queued now, behind this step only
            host, event = self._token_ring[self._ring_at]
            self._ring_at = (self._ring_at + 1) % len(self._token_ring)
            host[:tokens.shape[0]].copy_(tokens, non_blocking=True)
            event.record()
            arrival = (host, event, tokens.shape[0])
        n_prefill = sum(sc.num_tokens for sc in scheduled if not sc.seq.decoding)   # prompts, and evicted requests fed again
        self.scheduler.advance(scheduled)
        return dict(scheduled=scheduled, tokens=tokens, arrival=arrival, n_prefill=n_prefill,
                    n_decode=sum(sc.num_tokens for sc in scheduled) - n_prefill, events=(began, ended))

    def step(self, on_token=None) -> List[RequestOutput]:
        """One scheduled batch through the model; returns the requests that finished in it.  While every
        running request just decodes, the next step is launched before this step's tokens are read
        (`pipeline_decode`): the host's work on a step then overlaps the device's work on the next.
        on_token(request_id, token): called for every token that a request gets in this step, as soon as it is read."""
        t0 = time.perf_counter()
        cur = self._launched
        self._launched = None
        if cur is None:
            cur = self._launch(self.scheduler.schedule())
        nxt = None
        if self.config.pipeline_decode and cur["tokens"] is not None:
            ahead = self.scheduler.schedule_ahead(cur["scheduled"])
            if ahead is not None:
                items, index = ahead
                toks = cur["tokens"]
                if len(index) != toks.shape[0]:
                    toks = toks[torch.as_tensor(index, device=toks.device)]
                nxt = self._launch(items, device_tokens=toks)
                self.stats["steps_launched_ahead"] += 1
        tokens = []
        if cur["arrival"] is not None:
            host, event, n = cur["arrival"]
            event.synchronize()
            tokens = host[:n].tolist()
        now = time.perf_counter()
        before = [(sc.seq, sc.seq.num_tokens) for sc in cur["scheduled"] if sc.samples] if on_token else ()
        finished = self.scheduler.absorb(cur["scheduled"], tokens, now)
        for seq, n in before:
            if seq.num_tokens > n:
                on_token(seq.request_id, seq.token_ids[-1])
        self._launched = nxt
        dt = now - t0
        n_prefill, n_decode = cur["n_prefill"], cur["n_decode"]
        st = self.stats
        st["steps"] += 1
        # a mixed step's time is shared out by tokens
        total = max(n_prefill + n_decode, 1)
        st["prefill_tokens"] += n_prefill
        st["decode_tokens"] += n_decode
        st["prefill_time"] += dt * n_prefill / total
        st["decode_time"] += dt * n_decode / total
        began, ended = cur["events"]
        if cur["arrival"] is None:
            ended.synchronize()              # a step that samples nothing: its end has not been waited for yet
        device_s = began.elapsed_time(ended) * 1e-3
        st["device_time"] += device_s
        self.step_log.append((dt, device_s, n_prefill, n_decode))
        return [self._output(s) for s in finished]

    @staticmethod
    def _output(s):
        ttft = None if s.first_token_ts is None else s.first_token_ts - s.request_ts
        tpot = None
        if s.finish_ts is not None and s.first_token_ts is not None and s.num_output_tokens > 1:
            tpot = (s.finish_ts - s.first_token_ts) / (s.num_output_tokens - 1)
        return RequestOutput(s.request_id, s.token_ids[:s.num_prompt_tokens], s.output_ids, s.finish_reason,
                             ttft, tpot, s.evictions)

    def generate(self, prompts, params=None, on_token=None) -> List[RequestOutput]:
        """prompts: lists of token ids; params: one SamplingParams for all, or one per prompt.  Returns the
        outputs in the order of the prompts.  on_token(request_id, token): called as the tokens arrive; the
        request ids are those of add_request, counted up from the engine's first request."""
        if params is None or isinstance(params, SamplingParams):
            params = [params] * len(prompts)
        if len(params) != len(prompts):
            raise ValueError("%d prompts but %d sampling parameter sets" % (len(prompts), len(params)))
        import copy
        ids = [self.add_request(p, copy.copy(sp)) for p, sp in zip(prompts, params)]
        done = {}
        while self.has_unfinished():
            for out in self.step(on_token):
                done[out.request_id] = out
        return [done[i] for i in ids]
