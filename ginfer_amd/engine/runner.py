"""The model runner: one step function for a batch of (request, its next tokens).

`step(entries)` runs only the tokens it is given, as one batch, against the cache that earlier steps
left, and returns 32-bit logits at the wanted places.  Prompt portions and single decoded tokens sit
side by side; a request may be cut anywhere.  The reference's runner takes a batch that is all
prompts or all single tokens and returns token ids (ginfer/engine/model_runner.cc:177-317,
ginfer/model/model.cc:180-228); the side inputs built here are the same in kind (ids, positions,
block tables, slot mapping: model_runner.cc:145-298), flattened per token.
"""
from dataclasses import dataclass, field
from typing import List, Sequence

import numpy as np
import torch

from ..cache import CacheManager
from ..config import config_from_folder
from ..kernels import build
from ..parts.base import KVCacheSpec, StateSpec
from ..parts.model import build_model, StepContext, KVView, StateView
from ..weights import load_weights

DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32}


@dataclass
class StepEntry:
    request_id: object
    tokens: Sequence[int]
    want: Sequence[int] = field(default_factory=list)   # places among `tokens` whose logits are wanted


def require_gpu():
    if not torch.cuda.is_available():
        raise RuntimeError("ginfer_amd needs a GPU (gfx950); none is visible and there is no CPU path")
    return torch.device("cuda", torch.cuda.current_device())


class ModelRunner:
    def __init__(self, model_path, dtype="bfloat16", page_size=16, num_pages=None, max_requests=64,
                 max_model_len=None, gpu_memory_utilization=0.9, device=None, config=None):
        self.device = device or require_gpu()
        if dtype not in DTYPES:
            raise ValueError("dtype must be one of %s, got %r" % (sorted(DTYPES), dtype))
        self.dtype = DTYPES[dtype]
        self.config = config or config_from_folder(model_path)
        self.spec = self.config.model_spec()
        self.model = build_model(self.spec, self.dtype, self.device)
        self.max_model_len = int(min(max_model_len or self.spec.max_positions, self.spec.max_positions))
        for p in self.model.position_parts():
            p.limit_positions(self.max_model_len)
        # compile what this model needs, all at once, before anything runs
        build.build_all(modules=self.model.kernel_modules())
        load_weights(self.model, model_path, self.device)
        self.page_size = int(page_size)
        specs = self.model.cache_specs()
        if num_pages is None:
            num_pages = self._pages_from_free_memory(specs, gpu_memory_utilization)
        self.cache = CacheManager(specs, self.page_size, int(num_pages), int(max_requests))
        self.cache.allocate_device(self.dtype, self.device)
        self._owner_of = [i if e.cache_of is None else e.cache_of for i, e in enumerate(self.model.schedule)]

    def _pages_from_free_memory(self, specs, utilization):
        """Pages = free device memory (after the weights are resident) * utilization / bytes per page, the
        reference's sizing (ginfer/engine/model_runner.cc:52-70)."""
        probe = CacheManager(specs, self.page_size, 0, 1)
        per_page = probe.bytes_per_page(torch.empty(0, dtype=self.dtype).element_size())
        if per_page == 0:
            return 0
        free, _ = torch.cuda.mem_get_info(self.device)
        pages = int(free * utilization) // per_page
        if pages < 1:
            raise RuntimeError("no memory left for the cache: %d bytes free, a page takes %d" % (free, per_page))
        return pages

    @property
    def vocab_size(self):
        return self.spec.vocab_size

    # ---- the step
    def step(self, entries: List[StepEntry]):
        """Returns float32 logits [R, V] on the device: the wanted places in the order of the entries
        and of each entry's `want`."""
        if not entries:
            return torch.empty((0, self.vocab_size), dtype=torch.float32, device=self.device)
        cache = self.cache
        seen = set()
        for e in entries:
            if e.request_id in seen:
                raise ValueError("request %r appears twice in one step" % (e.request_id,))
            seen.add(e.request_id)
            n = len(e.tokens)
            if n < 1:
                raise ValueError("request %r brings no tokens" % (e.request_id,))
            for w in e.want:
                if not 0 <= w < n:
                    raise ValueError("request %r wants place %r of %d tokens" % (e.request_id, w, n))
        reserved_here = []
        try:
            for e in entries:
                if not cache.has(e.request_id):
                    cache.admit(e.request_id)
                if cache.pending(e.request_id) == 0:
                    if cache.length(e.request_id) + len(e.tokens) > self.max_model_len:
                        raise ValueError("request %r would grow to %d tokens, beyond max_model_len %d"
                                         % (e.request_id, cache.length(e.request_id) + len(e.tokens),
                                            self.max_model_len))
                    cache.append(e.request_id, len(e.tokens))
                    reserved_here.append(e.request_id)
                elif cache.pending(e.request_id) != len(e.tokens):
                    raise ValueError("request %r has %d tokens reserved but brings %d"
                                     % (e.request_id, cache.pending(e.request_id), len(e.tokens)))
            ctx = self._build_context(entries)
        except Exception:
            for rid in reserved_here:       # leave the cache as it was
                cache.requests[rid].pending = 0
            raise
        logits = self.model.forward(ctx)
        for e in entries:
            cache.commit(e.request_id)
        return logits

    def release(self, request_id):
        if self.cache.has(request_id):
            self.cache.release(request_id)

    def _build_context(self, entries):
        cache, ps = self.cache, self.page_size
        E = len(entries)
        q_len = [len(e.tokens) for e in entries]
        q_start = [cache.length(e.request_id) for e in entries]
        T = sum(q_len)
        ids = np.empty(T, dtype=np.int32)
        pos = np.empty(T, dtype=np.int32)
        ent = np.empty(T, dtype=np.int32)
        cu = np.zeros(E + 1, dtype=np.int32)
        rows = []
        o = 0
        for i, e in enumerate(entries):
            n = q_len[i]
            ids[o:o + n] = np.asarray(e.tokens, dtype=np.int64)
            pos[o:o + n] = np.arange(q_start[i], q_start[i] + n, dtype=np.int32)
            ent[o:o + n] = i
            rows.extend(o + w for w in e.want)
            o += n
            cu[i + 1] = o
        if ids.min() < 0 or ids.max() >= self.vocab_size:
            raise ValueError("token id outside [0, %d)" % self.vocab_size)
        dev = self.device

        def up(a):
            return torch.from_numpy(a).to(dev, non_blocking=False)

        # per group: block tables [E, W] and slot mapping [T]
        group_views = []
        for gi, g in enumerate(cache.groups):
            width = max(1, max(len(cache.table(e.request_id, gi)) for e in entries))
            bt = np.full((E, width), -1, dtype=np.int32)
            slots = np.empty(T, dtype=np.int64)
            o = 0
            for i, e in enumerate(entries):
                table = cache.table(e.request_id, gi)
                bt[i, :len(table)] = table
                p = np.arange(q_start[i], q_start[i] + q_len[i])
                pages = np.asarray(table, dtype=np.int64)[p // ps]
                if (pages < 0).any():
                    raise AssertionError("request %r: a new token has no page in group %d" % (e.request_id, gi))
                slots[o:o + q_len[i]] = pages * ps + p % ps
                o += q_len[i]
            group_views.append((up(bt), up(slots)))
        state_slots = up(np.asarray([cache.slot(e.request_id) for e in entries], dtype=np.int64))
        caches = []
        for i, sched in enumerate(self.model.schedule):
            owner = self._owner_of[i]
            spec = cache.cache_specs[owner]
            if isinstance(spec, KVCacheSpec):
                gi, j = cache.group_of[owner]
                bt, slots = group_views[gi]
                kp, vp = cache.kv_views(owner)
                caches.append(KVView(kp, vp, bt, slots, ps, owner == i))
            elif isinstance(spec, StateSpec):
                caches.append(StateView(cache.state_tensors[owner], state_slots, owner == i))
            else:
                caches.append(None)
        return StepContext(
            token_ids=up(ids), positions=up(pos), token_entry=up(ent), cu_tokens=up(cu),
            q_start=up(np.asarray(q_start, dtype=np.int32)),
            logit_rows=up(np.asarray(rows, dtype=np.int32)),
            num_tokens=T, num_entries=E, host_q_start=q_start, host_q_len=q_len, caches=caches, extra={})
