"""The model runner: one step function for a batch of (request, its next tokens).

`step(entries)` runs only the tokens it is given, as one batch, against the cache that earlier steps
left, and returns 32-bit logits at the wanted places.  Prompt portions and single decoded tokens sit
side by side; a request may be cut anywhere.  The reference's runner takes a batch that is all
prompts or all single tokens and returns token ids (ginfer/engine/model_runner.cc:177-317,
ginfer/model/model.cc:180-228); the side inputs built here are the same in kind (ids, positions,
block tables, slot mapping: model_runner.cc:145-298), flattened per token.

Steps whose shapes come again are recorded into HIP graphs and replayed: steps of single tokens by their exact
number of requests, short steps with prompt portions laid into padded sizes (`_run_padded`); all side inputs of
a recorded step live in one static buffer that every replay refills.
"""
import os
import time
from dataclasses import dataclass, field
from typing import List, Sequence

import numpy as np
import torch

from ..cache import CacheManager
from ..cache.manager import caches_of
from ..config import config_from_folder
from ..kernels import autotune as tuner, build
from ..kernels.tuning import TUNING
from ..parts.base import KVCacheSpec, StateSpec
from ..parts.model import build_model, StepContext, KVView, StateView
from ..weights import load_weights, bind_random_weights

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
                 max_model_len=None, gpu_memory_utilization=0.9, device=None, config=None, use_graphs=True,
                 prefix_caching=False, random_seed=None, graph_mixed_steps=True, max_num_batched_tokens=None,
                 strict_weights=False, autotune=False):
        """model_path: a folder with config.json and the weights.  With model_path None, `config` (a typed
        configuration) and `random_seed` make a model whose weights are drawn on the device, for shapes too
        large to pass through a file.  num_pages: pages of every cache group (or a list, one count per group);
        None: from the memory that is free once the weights are loaded and the largest step (max_num_batched_tokens
        tokens, max_requests requests) has run, times gpu_memory_utilization.  strict_weights: a tensor in the folder
        that the model does not read is an error, not a warning.  autotune: before a step of some number of rows is
        recorded, the products that can be done in several ways are timed in each and the fastest kept
        (kernels/autotune.py); takes a second or so per number of rows, once.  True: the runner keeps its own table of
        plans (`plans`); a table of another runner (its `plans`) may be given instead, to share what it measured."""
        self.device = device or require_gpu()
        if dtype not in DTYPES:
            raise ValueError("dtype must be one of %s, got %r" % (sorted(DTYPES), dtype))
        self.dtype = DTYPES[dtype]
        if model_path is None and (config is None or random_seed is None):
            raise ValueError("without a model folder, a configuration and a random_seed are needed")
        self.config = config or config_from_folder(model_path)
        self.spec = self.config.model_spec()
        self.model = build_model(self.spec, self.dtype, self.device)
        self.max_model_len = int(min(max_model_len or self.spec.max_positions, self.spec.max_positions))
        for p in self.model.position_parts():
            p.limit_positions(self.max_model_len)
        # compile what this model needs, all at once, before anything runs
        build.build_all(modules=self.model.kernel_modules())
        if model_path is None:
            bind_random_weights(self.model, int(random_seed), self.device)
        else:
            load_weights(self.model, model_path, self.device, strict=strict_weights)
        self.page_size = int(page_size)
        self.max_requests = int(max_requests)
        self.max_step_tokens = int(min(max_num_batched_tokens or 2048, self.max_model_len))
        specs = self.model.cache_specs()
        if prefix_caching is None:       # where the model allows it
            prefix_caching = CacheManager.supports_prefix_caching(specs)
        self.graph_mixed_steps = bool(graph_mixed_steps)
        # the plans this runner's products run by: its own table, one handed over, or none (by the rules)
        self.plans = autotune if isinstance(autotune, tuner.Table) else (tuner.Table() if autotune else None)
        self.autotune = self.plans is not None
        self._reserved_by_tuning = 0
        self._graphs, self._graph_seen, self._padded_buffers = {}, {}, {}
        self._graph_budget, self._graph_bytes, self._graph_bytes_seen = None, 0, {}
        # Padding pays while the host's launches (~5 ms a step) outlast the device's work on the padded rows, which may
        # be twice the step's own: with some 1e15 operations a second that is rows * weights < ~1.5e12 (512 rows for a
        # 1.5B model, 128 for a 7B one, none for a 72B one)
        weights = sum(int(np.prod(ws.shape)) for ws in self.model.weight_specs().values())
        self._padded_max_rows = min(TUNING.mixed_graph_max_tokens, int(TUNING.padded_rows_times_weights // max(weights, 1)))
        # how steps ran: launched kernel by kernel, replayed as a recorded decode step, replayed as a recorded step
        # with prompt portions; and how many steps were recorded
        self.counts = dict(launched=0, replayed_decode=0, replayed_padded=0, recorded=0, recording_seconds=0.0)
        self.use_graphs = False          # nothing is recorded while the pool is being planned
        self.memory_plan = None
        if num_pages is None:
            num_pages = self._plan_pool(specs, float(gpu_memory_utilization))
            self.counts["launched"] = 0
        self._install_cache(specs, num_pages, prefix_caching)
        self.use_graphs = bool(use_graphs) and self.model.capturable()

    def _install_cache(self, specs, num_pages, prefix_caching):
        self.cache = CacheManager(specs, self.page_size, num_pages, self.max_requests, prefix_caching=prefix_caching)
        self.cache.allocate_device(self.dtype, self.device)
        self._owner_of = [i if e.cache_of is None else e.cache_of for i, e in enumerate(self.model.schedule)]
        self._buffers = _BufferCache(len(self.cache.groups), self.device)

    def _plan_pool(self, specs, utilization):
        """Page counts per cache group from the device's memory, in the reference's order (ginfer/model/model.cc:48-120
        makes the scratch memory first, ginfer/engine/model_runner.cc:52-70 then sizes the pool from what is free).
        The largest step runs once over a small pool of its own: a prompt portion beside a single token of every other
        request, every request sampled, which tells what activations, logits and the library's workspace take at
        their peak.  From the memory that is free with the weights loaded, the per-request state (fixed: a slot for
        every request and one more) is taken first; the pool is what is left x utilization; beside the pool there has
        to be room for that peak (and for the tuner's buffers, with autotune), else the utilization is refused; what
        is left beyond that, up to a bound, is what recorded steps may hold (`_record` never takes from the step's
        own room).  Groups with a window get what they can ever hold, the groups that keep all keys share the rest
        (`CacheManager.plan_pages`)."""
        if not 0.0 < utilization <= 1.0:
            raise ValueError("gpu_memory_utilization must lie in (0, 1], got %r" % (utilization,))
        esize = torch.empty(0, dtype=self.dtype).element_size()
        if not CacheManager.group_specs(specs):
            return 0
        T, R, ps = self.max_step_tokens, self.max_requests, self.page_size
        # the largest step over a pool that just holds it: a portion beside one token of each of the other requests
        singles = max(0, min(R - 1, T - 1))
        portion = T - singles
        probe_pages = -(-portion // ps) + singles + 1
        self._install_cache(specs, probe_pages, False)
        torch.cuda.synchronize(self.device)
        resident = torch.cuda.memory_allocated(self.device)
        torch.cuda.reset_peak_memory_stats(self.device)
        try:
            entries = [StepEntry(("probe", 0), [0] * portion, [portion - 1])]
            entries += [StepEntry(("probe", r), [0], [0]) for r in range(1, singles + 1)]
            self.step(entries)
            for e in entries:
                self.release(e.request_id)
            torch.cuda.synchronize(self.device)
        finally:
            peak = torch.cuda.max_memory_allocated(self.device) - resident
            del self.cache, self._buffers
            torch.cuda.empty_cache()
        free, total = torch.cuda.mem_get_info(self.device)
        state = CacheManager.state_bytes(specs, R)
        need = int(peak * 1.1) + (64 << 20)          # the step's own peak, a tenth more, and the allocator's rounding
        if self.autotune:
            # the tuner's buffer that is overwritten between timings, and the outputs of the candidates it runs (a step's
            # own peak bounds them)
            need += tuner.FLUSH_BYTES + int(peak)
        avail = free - state
        pool = int(avail * utilization) if avail > 0 else 0
        if avail - pool < need or pool <= 0:
            raise ValueError("gpu_memory_utilization %.3f leaves %d MB beside the cache, but a step of %d tokens and %d "
                             "requests takes up to %d MB: at most %.3f fits (%d MB are free with the weights loaded, "
                             "%d MB of them go to the per-request state)"
                             % (utilization, max(avail - pool, 0) >> 20, T, R, need >> 20,
                                max(0.0, (avail - need) / avail) if avail > 0 else 0.0, free >> 20, state >> 20))
        counts = CacheManager.plan_pages(specs, ps, esize, pool, R, T, self.max_model_len)
        # what recorded steps may hold: what is left beside pool, state and the step's own room, at most an eighth of the card
        self._graph_budget = max(0, min(avail - pool - need, total // 8))
        self.memory_plan = dict(free_bytes=int(free), state_bytes=int(state), pool_bytes=pool, step_peak_bytes=int(peak),
                                step_room_bytes=int(need), graph_budget_bytes=int(self._graph_budget), pages=list(counts))
        return counts

    @property
    def vocab_size(self):
        return self.spec.vocab_size

    # ---- the step
    def step(self, entries: List[StepEntry], borrow=False, device_tokens=None):
        """Returns float32 logits [R, V] on the device: the wanted places in the order of the entries
        and of each entry's `want`.  With borrow=True the result may be a buffer that the next step
        overwrites (the engine samples from it at once).
        device_tokens (int32 [len(entries)] on the device): every entry brings ONE token whose id the host does
        not know yet (the entry's own token is a placeholder): the ids are taken from this tensor on the device,
        in the order of the entries.  This lets a caller launch a decode step before it has read the tokens of
        the step before.
        Cache pages: a request that the step meets for the first time is admitted; tokens that the caller has not
        reserved (`cache.append`) are reserved and committed here; tokens that the caller reserved stay for the caller to
        commit once the step is launched."""
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
        if device_tokens is not None:
            if any(len(e.tokens) != 1 for e in entries):
                raise ValueError("tokens that are still on the device stand for single-token entries only")
            if device_tokens.dtype != torch.int32 or tuple(device_tokens.shape) != (len(entries),) or not device_tokens.is_cuda:
                raise ValueError("device_tokens must be int32 [%d] on the device" % len(entries))
        reserved_here = []
        try:
            reserve_for_step(cache, entries, self.max_model_len, reserved_here)
            host = self._host_arrays(entries)
            logits = self._run(host, borrow, device_tokens)
        except Exception:
            for rid in reserved_here:       # nothing is committed: the requests stay as long as they were
                cache.cancel(rid)
            raise
        # What this step reserved it also commits.  A caller that reserved the tokens itself (the scheduler) commits them
        # too, with the request's tokens: the cache manager then remembers the pages that are full now, for requests
        # that share the prefix (ginfer/engine/block_manager.cc:98-108 registers a block as soon as it is full).
        for rid in reserved_here:
            cache.commit(rid)
        return logits

    def release(self, request_id):
        if self.cache.has(request_id):
            self.cache.release(request_id)

    # ---- the step's side inputs
    def _host_arrays(self, entries):
        """Everything the kernels need to know about the batch, as numpy arrays (no device work)."""
        cache, ps = self.cache, self.page_size
        E = len(entries)
        slots = np.fromiter((cache.slot(e.request_id) for e in entries), dtype=np.int64, count=E)
        q_len = np.fromiter((len(e.tokens) for e in entries), dtype=np.int64, count=E)
        q_start = cache.lengths_array(slots)
        T = int(q_len.sum())
        cu = np.zeros(E + 1, dtype=np.int32)
        np.cumsum(q_len, out=cu[1:])
        if T == E:                          # every request brings one token: no loop over tokens
            ids = np.fromiter((e.tokens[0] for e in entries), dtype=np.int64, count=E)
            ent = np.arange(E, dtype=np.int32)
            pos = q_start.astype(np.int32)
        else:
            ids = np.concatenate([np.asarray(e.tokens, dtype=np.int64) for e in entries])
            ent = np.repeat(np.arange(E, dtype=np.int32), q_len)
            pos = (np.arange(T, dtype=np.int64) - np.repeat(cu[:-1].astype(np.int64), q_len)
                   + np.repeat(q_start, q_len)).astype(np.int32)
        if ids.min() < 0 or ids.max() >= self.vocab_size:
            raise ValueError("token id outside [0, %d)" % self.vocab_size)
        if int(pos.max()) >= self.max_model_len:
            raise ValueError("a token at position %d lies beyond max_model_len %d" % (int(pos.max()), self.max_model_len))
        rows = [int(cu[i]) + w for i, e in enumerate(entries) for w in e.want]
        max_kv = int((q_start + q_len).max())
        width = -(-max_kv // ps)
        tables, slot_maps = [], []
        for gi in range(len(cache.groups)):
            bt = cache.tables_array(gi, slots, width)
            pages = bt[ent, pos // ps].astype(np.int64)
            if (pages < 0).any():
                raise AssertionError("a new token has no page in cache group %d" % gi)
            tables.append(bt)
            slot_maps.append(pages * ps + pos % ps)
        return dict(E=E, T=T, ids=ids.astype(np.int32), pos=pos, ent=ent, cu=cu, q_start=q_start.astype(np.int32),
                    q_len=q_len, rows=np.asarray(rows, dtype=np.int32), width=width, tables=tables,
                    slot_maps=slot_maps, state_slots=slots, max_kv=max_kv,
                    decode_info=self._decode_info(cu, q_len, q_start, ent, T == E))

    @staticmethod
    def _decode_info(cu, q_len, q_start, ent, all_single):
        """int32 [n, 4]: (row in the step, position, entry, 0) of every entry that brings a single token."""
        if all_single:
            rows, pos, entries = ent, q_start, ent
        else:
            mask = q_len == 1
            rows, pos, entries = cu[:-1][mask], q_start[mask], np.flatnonzero(mask)
        info = np.zeros((len(rows), 4), dtype=np.int32)
        info[:, 0], info[:, 1], info[:, 2] = rows, pos, entries
        return info

    def _context(self, host, buf):
        """Uploads the host arrays through one packed buffer and wraps the device views."""
        buf.fill(host)
        cache, ps = self.cache, self.page_size
        def view(owner, place, spec, owns):
            if isinstance(spec, StateSpec):
                return StateView(cache.state_tensors[(owner, place)], buf.dev["state_slots"], owns)
            gi, _ = cache.group_of[(owner, place)]
            if isinstance(spec, KVCacheSpec):
                kp, vp = cache.kv_views(owner, place)
                return KVView(kp, vp, buf.dev["table%d" % gi], buf.dev["slots%d" % gi], ps, owns)
            return KVView(None, None, buf.dev["table%d" % gi], buf.dev["slots%d" % gi], ps, owns,
                          pages=cache.page_views(owner, place))
        caches = []
        for i, sched in enumerate(self.model.schedule):
            owner = self._owner_of[i]
            spec = cache.cache_specs[owner]
            views = [view(owner, k, c, owner == i) for k, c in enumerate(caches_of(spec))]
            # a block that names a list of caches gets a list of views, any other its one view (or None)
            caches.append(views if isinstance(spec, (list, tuple)) else (views[0] if views else None))
        # decode rows come first in cu order only when every entry is a single token; the list is general
        return StepContext(
            token_ids=buf.dev["ids"], positions=buf.dev["pos"], token_entry=buf.dev["ent"], cu_tokens=buf.dev["cu"],
            q_start=buf.dev["q_start"], logit_rows=buf.dev["rows"], num_tokens=host["T"], num_entries=host["E"],
            host_q_start=host["q_start"].tolist(), host_q_len=host["q_len"].tolist(), caches=caches,
            extra={"decode_info": buf.dev["decode_info"], "decode_span": _context_bucket(host["max_kv"])})

    def _run(self, host, borrow, device_tokens=None):
        E, T = host["E"], host["T"]
        graphable = self.use_graphs and T == E and E <= TUNING.graph_max_rows and len(host["rows"]) == E and \
            bool((host["rows"] == np.arange(E)).all())
        if graphable:
            bucket = _context_bucket(host["max_kv"])
            key = (E, bucket)
            g = self._graphs.pop(key, None)
            if g is not None:
                self._graphs[key] = g        # most recently used last
            else:
                self._graph_seen[key] = self._graph_seen.get(key, 0) + 1
                if self._graph_seen[key] >= TUNING.graph_after:
                    g = self._record(self._capture, key, host)
            if g is not None:
                g["buf"].fill(host)
                if device_tokens is not None:
                    g["buf"].buf.dev["ids"].copy_(device_tokens)
                g["graph"].replay()
                self.counts["replayed_decode"] += 1
                return g["logits"] if borrow else g["logits"].clone()
        if not graphable and device_tokens is None and self.use_graphs and self.graph_mixed_steps:
            logits = self._run_padded(host, borrow)
            if logits is not None:
                return logits
        buf = self._buffers.get(T, E, len(host["rows"]), host["width"], len(host["decode_info"]))
        ctx = self._context(host, buf)
        if device_tokens is not None:
            buf.dev["ids"].copy_(device_tokens)
        self.counts["launched"] += 1
        return self._forward(ctx)

    def _forward(self, ctx):
        """The model's forward, its products running by this runner's plans (none: by the rules)."""
        with tuner.using(self.plans):
            return self.model.forward(ctx)

    def _record(self, capture, key, host):
        """Records a step unless the device memory that recorded steps may hold is used up (each holds its buffers and
        its activations): the least recently used ones are forgotten first, by count and by bytes.  None: not
        recorded, the step runs launch by launch."""
        if self._graph_budget is None:
            # the pool was given, not planned: half of what is free now, at most 1/8 of the card
            free, total = torch.cuda.mem_get_info(self.device)
            self._graph_budget = min((free + torch.cuda.memory_reserved(self.device)
                                      - torch.cuda.memory_allocated(self.device)) // 2, total // 8)
        need = self._graph_bytes_seen.get(key[0] == "padded", 0)
        while self._graphs and (len(self._graphs) >= TUNING.graph_keep or self._graph_bytes + need > self._graph_budget):
            old = self._graphs.pop(next(iter(self._graphs)))
            self._graph_bytes -= old["bytes"]
            del old
        if need > self._graph_budget:
            return None
        before = torch.cuda.memory_reserved(self.device)     # a recorded step keeps a pool of its own reserved
        self._reserved_by_tuning = 0
        t0 = time.perf_counter()
        try:
            g = capture(key, host)
        except torch.cuda.OutOfMemoryError as e:
            # the plan left recorded steps a budget that the device does not have: better said than run on slowly
            self._graphs.pop(key, None)
            raise RuntimeError("the device ran out of memory while a step of %s was being recorded (%d MB held by "
                               "recorded steps, budget %d MB): lower gpu_memory_utilization or max_num_seqs, or run "
                               "without recorded steps" % (key, self._graph_bytes >> 20, self._graph_budget >> 20)) from e
        except Exception as e:           # recording is a matter of speed only: the steps go on launch by launch
            import sys
            sys.stderr.write("[ginfer_amd] recording a step failed (%s: %s); steps are launched kernel by kernel from "
                             "now on\n" % (type(e).__name__, e))
            self._graphs.pop(key, None)
            self.use_graphs = False
            torch.cuda.synchronize()
            return None
        self.counts["recording_seconds"] = round(self.counts["recording_seconds"] + time.perf_counter() - t0, 4)
        g["bytes"] = max(0, torch.cuda.memory_reserved(self.device) - before - self._reserved_by_tuning)
        self._graph_bytes += g["bytes"]
        kind = key[0] == "padded"
        self._graph_bytes_seen[kind] = max(self._graph_bytes_seen.get(kind, 0), g["bytes"])
        return g

    # ---- recorded steps that hold prompt portions
    def _run_padded(self, host, borrow):
        """A step with prompt portions, short enough that the host's launches would take longer than the device's
        work: it is laid into a recorded step of fixed sizes (token rows and entries powers of two, the context
        bucket), recorded the second time such sizes are seen.  Rows and entries beyond the step's own
        are padding: tokens of an extra entry whose one page is page 0, which write nothing to the cache; the tiles
        and single-token records that fill the plan point at the first padding row.  Rows do not mix in any kernel,
        so what the padding computes stays in the padding.  None: the step runs launch by launch."""
        T, E, R = host["T"], host["E"], len(host["rows"])
        if T + 1 > self._padded_max_rows or E > TUNING.graph_max_rows:
            return None
        t_pad = 64                       # coarse sizes, so that few recorded steps serve many: rows 64, 128, 256, 512
        while t_pad < T + 1:
            t_pad *= 2
        if t_pad > self._padded_max_rows:
            return None
        e_pad = 8                        # entries 8, 16, ... 256
        while e_pad < E:
            e_pad *= 2
        if R > e_pad:
            return None
        bucket = _context_bucket(host["max_kv"])
        key = ("padded", t_pad, e_pad, bucket)
        g = self._graphs.pop(key, None)
        if g is not None:
            self._graphs[key] = g
        else:
            self._graph_seen[key] = self._graph_seen.get(key, 0) + 1
            if self._graph_seen[key] >= TUNING.graph_after:
                g = self._record(self._capture_padded, key, host)
        if g is None:
            # not recorded yet: launched kernel by kernel, but with the same padded sizes, so that a step's bits do not
            # depend on whether its sizes have been seen before
            width = max(1, -(-bucket // self.page_size))
            buf = self._padded_buffers.pop(key, None)
            if buf is None:
                buf = _StepBuffers(t_pad, e_pad + 1, e_pad, width, e_pad, len(self.cache.groups), self.device,
                                   n_tiles=self._padded_tiles(t_pad, e_pad))
                while len(self._padded_buffers) >= 8:
                    self._padded_buffers.pop(next(iter(self._padded_buffers)))
            self._padded_buffers[key] = buf
            ctx = self._padded_context(host, buf, t_pad, e_pad, width, bucket)
            self.counts["launched"] += 1
            return self._forward(ctx)[:R]
        g["buf"].fill(self._pad(host, t_pad, e_pad, g["width"]))
        g["graph"].replay()
        self.counts["replayed_padded"] += 1
        out = g["logits"][:R]
        return out if borrow else out.clone()

    @staticmethod
    def _padded_tiles(t_pad, e_pad):
        from ..kernels import ops
        return t_pad // ops.PLAN_TILE_ROWS + e_pad

    def _padded_context(self, host, buf, t_pad, e_pad, width, bucket):
        from ..kernels import ops
        ctx = self._context(self._pad(host, t_pad, e_pad, width), buf)
        ctx.extra = {"decode_info": buf.dev["decode_info"], "decode_span": bucket,
                     "static_plan": dict(tiles=buf.dev["tiles"], n_tiles=self._padded_tiles(t_pad, e_pad), n_decode=e_pad,
                                         tile_rows=ops.PLAN_TILE_ROWS)}
        return ctx

    def _pad(self, host, t_pad, e_pad, width):
        return pad_step(host, t_pad, e_pad, width, self.cache.pad_slot)

    def _capture_padded(self, key, host):
        _, t_pad, e_pad, bucket = key
        width = max(1, -(-bucket // self.page_size))
        buf = _StepBuffers(t_pad, e_pad + 1, e_pad, width, e_pad, len(self.cache.groups), self.device,
                           n_tiles=self._padded_tiles(t_pad, e_pad))
        ctx = self._padded_context(host, buf, t_pad, e_pad, width, bucket)
        self._settle(ctx, dict(ctx.extra))
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            logits = self._forward(ctx)
        g = dict(graph=graph, buf=buf, logits=logits, ctx=ctx, width=width)
        self._graphs[key] = g
        return g

    def _capture(self, key, host):
        """Records the decode step of E single tokens (contexts up to `bucket`) into a HIP graph.  All
        side inputs live in one static buffer that later steps refill; the attention kernels split the
        keys for the bucket's longest context, so the grid does not depend on the step."""
        E, bucket = key
        width = max(1, -(-bucket // self.page_size))
        buf = _StepBuffers(E, E, E, width, E, len(self.cache.groups), self.device)
        padded = dict(host, width=width, tables=[self._widen(t, width) for t in host["tables"]])
        ctx = self._context(padded, buf)
        self._settle(ctx, {"decode_info": buf.dev["decode_info"], "decode_span": bucket})
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            logits = self._forward(ctx)
        g = dict(graph=graph, buf=_GraphBuffers(buf, width, self._widen), logits=logits, ctx=ctx)
        self._graphs[key] = g
        return g

    def _settle(self, ctx, extra):
        """What precedes the recording of a step: with autotune, a run in which the products report themselves and the
        timing of their plans; then the run that warms up what the recording will call.  Every run starts from the
        same `extra` (a run leaves its plans of rows and tiles there)."""
        if self.autotune:
            ctx.extra = dict(extra)
            with tuner.collecting() as seen:
                self._run_once_unrecorded(ctx, count=False)
            t0 = time.perf_counter()
            reserved = torch.cuda.memory_reserved(self.device)
            self.counts["autotuned_keys"] = self.counts.get("autotuned_keys", 0) + tuner.tune(
                seen, self.device, self.plans, verbose=bool(os.environ.get("GINFER_AMD_AUTOTUNE_VERBOSE")))
            self.counts["autotune_seconds"] = round(self.counts.get("autotune_seconds", 0.0) + time.perf_counter() - t0, 3)
            # what the timing left in the allocator's hands is not the recorded step's
            self._reserved_by_tuning += max(0, torch.cuda.memory_reserved(self.device) - reserved)
        ctx.extra = dict(extra)
        self._run_once_unrecorded(ctx)
        ctx.extra = dict(extra)

    def _run_once_unrecorded(self, ctx, count=True):
        """Before a step is recorded it runs once outside the graph, on a stream of its own: libraries load what they
        need, the allocator settles.  The step itself is the replay that follows, so this run must leave nothing
        behind: keys and values it writes are written again by the replay, the same ones into the same places, and
        per-request state, which a second run would advance twice, is put back as it was."""
        saved = {e: t.clone() for e, t in self.cache.state_tensors.items()}
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            self._forward(ctx)
        torch.cuda.current_stream().wait_stream(side)
        for e, t in saved.items():
            self.cache.state_tensors[e].copy_(t)
        torch.cuda.synchronize()
        if count:
            self.counts["recorded"] += 1

    @staticmethod
    def _widen(table, width):
        if table.shape[1] == width:
            return table
        out = np.full((table.shape[0], width), -1, dtype=np.int32)
        out[:, :table.shape[1]] = table
        return out


def reserve_for_step(cache, entries, max_model_len, reserved):
    """Cache pages for a step's entries, as far as the caller has not reserved them: a request that the cache does not
    know is admitted, and tokens that are not reserved yet are (all of an entry's or none).  The requests whose tokens
    were reserved here are appended to `reserved` as they are, so that the caller can undo them if the step fails, and
    commit them (only them) when it is launched."""
    for e in entries:
        if not cache.has(e.request_id):
            cache.admit(e.request_id)
        if cache.pending(e.request_id) == 0:
            if cache.length(e.request_id) + len(e.tokens) > max_model_len:
                raise ValueError("request %r would grow to %d tokens, beyond max_model_len %d"
                                 % (e.request_id, cache.length(e.request_id) + len(e.tokens), max_model_len))
            cache.append(e.request_id, len(e.tokens))
            reserved.append(e.request_id)
        elif cache.pending(e.request_id) != len(e.tokens):
            raise ValueError("request %r has %d tokens reserved but brings %d"
                             % (e.request_id, cache.pending(e.request_id), len(e.tokens)))


def pad_step(host, t_pad, e_pad, width, pad_slot):
    """The host arrays of a step laid into t_pad token rows and e_pad + 1 entries: the step's own come first, the
    rest is padding (see ModelRunner._run_padded).  Tables are `width` wide.  pad_slot: the state slot of the entries
    that are padding, one that no request holds (a mixer with state of its own reads and writes it for them)."""
    from ..kernels import ops
    T, E = host["T"], host["E"]
    dummy, entries = e_pad, e_pad + 1

    def grown(a, n, fill):
        out = np.full((n,) + a.shape[1:], fill, dtype=a.dtype)
        out[:a.shape[0]] = a
        return out
    cu = np.full(entries + 1, T, dtype=np.int32)
    cu[:E + 1] = host["cu"]
    cu[entries] = t_pad
    q_len = grown(host["q_len"], entries, 0)
    q_len[dummy] = t_pad - T
    tables = []
    for t in host["tables"]:
        bt = np.full((entries, width), -1, dtype=np.int32)
        bt[:E, :t.shape[1]] = t
        bt[dummy, 0] = 0
        tables.append(bt)
    _, _, _, tiles = ops.plan_rows(host["q_len"].tolist(), host["q_start"].tolist(), ops.PLAN_TILE_ROWS)
    tile_arr = np.empty(((t_pad // ops.PLAN_TILE_ROWS + e_pad), 4), dtype=np.int32)
    tile_arr[:] = (dummy, T, 1, 0)
    if tiles:
        tile_arr[:len(tiles)] = np.asarray(tiles, dtype=np.int32)
    info = np.empty((e_pad, 4), dtype=np.int32)
    info[:] = (T, 0, dummy, 0)
    info[:len(host["decode_info"])] = host["decode_info"]
    return dict(host, T=t_pad, E=entries, ids=grown(host["ids"], t_pad, 0), pos=grown(host["pos"], t_pad, 0),
                ent=grown(host["ent"], t_pad, dummy), cu=cu, q_start=grown(host["q_start"], entries, 0), q_len=q_len,
                rows=grown(host["rows"], e_pad, 0), width=width, tables=tables,
                slot_maps=[grown(sm, t_pad, -1) for sm in host["slot_maps"]],
                state_slots=grown(host["state_slots"], entries, pad_slot), decode_info=info, tiles=tile_arr)


def _context_bucket(max_kv):
    """Contexts are rounded up to a power of two (at least 256): the attention kernels split the keys for
    the bucket's longest context, in recorded and in eager steps alike, so that both do the same sums."""
    bucket = 256
    while bucket < max_kv:
        bucket *= 2
    return bucket


class _StepBuffers:
    """One pinned host buffer and one device buffer that hold all side inputs of a step; `fill` copies the
    host arrays in and uploads them in one transfer."""

    def __init__(self, T, E, R, width, n_decode, ngroups, device, n_tiles=0):
        self.shape = (T, E, R, width, n_decode)
        fields = [("slots%d" % g, np.int64, (T,)) for g in range(ngroups)]
        fields += [("state_slots", np.int64, (E,))]
        fields += [("ids", np.int32, (T,)), ("pos", np.int32, (T,)), ("ent", np.int32, (T,)), ("cu", np.int32, (E + 1,)),
                   ("q_start", np.int32, (E,)), ("rows", np.int32, (R,)), ("decode_info", np.int32, (n_decode, 4)),
                   ("tiles", np.int32, (n_tiles, 4))]
        fields += [("table%d" % g, np.int32, (E, max(width, 1))) for g in range(ngroups)]
        offset, self.layout = 0, {}
        for name, dt, shape in fields:
            n = int(np.prod(shape)) * np.dtype(dt).itemsize
            self.layout[name] = (offset, dt, shape)
            offset += -(-max(n, 1) // 16) * 16
        self.nbytes = offset
        self.host_t = torch.empty(self.nbytes, dtype=torch.uint8, pin_memory=True)
        self.dev_t = torch.empty(self.nbytes, dtype=torch.uint8, device=device)
        host_np = self.host_t.numpy()
        self.host, self.dev = {}, {}
        tdt = {np.int64: torch.int64, np.int32: torch.int32}
        for name, (off, dt, shape) in self.layout.items():
            n = int(np.prod(shape))
            nb = n * np.dtype(dt).itemsize
            self.host[name] = host_np[off:off + nb].view(dt).reshape(shape)
            self.dev[name] = self.dev_t[off:off + nb].view(tdt[dt]).view(shape)
        self.event = torch.cuda.Event()
        self.used = False

    def fill(self, host):
        if self.used:
            self.event.synchronize()     # the last upload from this pinned buffer is through
        h = self.host
        h["ids"][:] = host["ids"]
        h["pos"][:] = host["pos"]
        h["ent"][:] = host["ent"]
        h["cu"][:] = host["cu"]
        h["q_start"][:] = host["q_start"]
        h["rows"][:] = host["rows"]
        h["decode_info"][:] = host["decode_info"]
        h["state_slots"][:] = host["state_slots"]
        if "tiles" in host:
            h["tiles"][:] = host["tiles"]
        for g, (bt, sm) in enumerate(zip(host["tables"], host["slot_maps"])):
            h["table%d" % g][:, :bt.shape[1]] = bt
            h["slots%d" % g][:] = sm
        self.dev_t.copy_(self.host_t, non_blocking=True)
        self.event.record()
        self.used = True


class _GraphBuffers:
    """The static buffers of a recorded step: tables are padded to the bucket's width on the way in."""

    def __init__(self, buf, width, widen):
        self.buf, self.width, self.widen = buf, width, widen

    def fill(self, host):
        self.buf.fill(dict(host, tables=[self.widen(t, self.width) for t in host["tables"]]))


class _BufferCache:
    """Step buffers by (rounded) sizes, so that pinned memory is not allocated step after step."""

    def __init__(self, ngroups, device, keep=24):
        self.ngroups, self.device, self.keep = ngroups, device, keep
        self.items = {}

    def get(self, T, E, R, width, n_decode):
        key = (T, E, R, width, n_decode)
        buf = self.items.pop(key, None)
        if buf is None:
            buf = _StepBuffers(T, E, R, width, n_decode, self.ngroups, self.device)
            while len(self.items) >= self.keep:
                self.items.pop(next(iter(self.items)))
        self.items[key] = buf            # most recently used last
        return buf
