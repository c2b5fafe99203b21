"""The scheduler: admits requests, cuts prompts into portions under a token budget, decodes,
finishes and frees.

Every step is one mixed batch.  First every running request that is decoding gets its one token;
then what is left of the budget goes to prompt portions, first of running requests whose prompt is
not through yet, then of waiting requests in arrival order, while fewer than max_num_seqs requests
run and a state slot is free.  A portion is cut to what the budget and the free pages allow.  The
reference runs prompts whole and never beside decoding (ginfer/engine/scheduler.cc:20-71); its queues,
its finishing rule (:83-99) and its answer to a full cache are kept.  A request is admitted with its tokens:
where the cache shares prefixes it starts behind the part that the cache already holds
(ginfer/engine/block_manager.cc:83-96), an evicted request behind what is left of its own pages.

When pages run out for a decoding request, the newest running request is evicted: its pages are given
back, it keeps its tokens, returns to the FRONT of the waiting queue and is later fed again from its
first token, prompt and output alike (recompute; ginfer/engine/scheduler.cc:47-56 and :73-77, where the
evicted sequence goes to the back of the queue instead).  If the request that cannot grow is the only
one running, it is evicted itself.  A request that could never fit the pool alone is refused when it
is added, so eviction always ends.
"""
from collections import deque
from dataclasses import dataclass
from typing import List

from ..cache import OutOfPages
from .sequence import Sequence, State


@dataclass
class Scheduled:
    seq: Sequence
    num_tokens: int          # tokens of seq.token_ids[num_computed:] that run in this step
    samples: bool            # the portion reaches the end of the known tokens: a token is sampled


class Scheduler:
    def __init__(self, cache, max_num_seqs, max_num_batched_tokens, eos_token_ids, max_model_len):
        if max_num_batched_tokens < 1 or max_num_seqs < 1:
            raise ValueError("max_num_seqs and max_num_batched_tokens must be positive")
        if max_num_batched_tokens < max_num_seqs:
            raise ValueError("max_num_batched_tokens (%d) must be at least max_num_seqs (%d): every running "
                             "request decodes one token a step" % (max_num_batched_tokens, max_num_seqs))
        self.cache = cache
        self.max_num_seqs, self.max_num_batched_tokens = int(max_num_seqs), int(max_num_batched_tokens)
        self.eos_token_ids = set(eos_token_ids)
        self.max_model_len = int(max_model_len)
        self.waiting = deque()
        self.running: List[Sequence] = []
        self.num_evictions = 0

    # ---- requests
    def add(self, seq):
        total = seq.num_prompt_tokens + seq.params.max_tokens
        if seq.num_prompt_tokens < 1:
            raise ValueError("request %r has an empty prompt" % (seq.request_id,))
        if seq.num_prompt_tokens + 1 > self.max_model_len:
            raise ValueError("request %r: prompt of %d tokens leaves no room under max_model_len %d"
                             % (seq.request_id, seq.num_prompt_tokens, self.max_model_len))
        ps = self.cache.page_size
        grown = min(total, self.max_model_len)
        for gi, g in enumerate(self.cache.groups):
            need = -(-grown // ps)
            if g.window is not None:         # token by token a window holds the pages that `window` positions can touch
                need = min(need, self.cache.window_span_pages(g.window, ps))
            if need > g.pool.num_pages:
                raise ValueError("request %r can grow to %d tokens (%d pages%s) but cache group %d has %d pages; "
                                 "it could never finish" % (seq.request_id, grown, need,
                                                            "" if g.window is None else " of a window of %d" % g.window,
                                                            gi, g.pool.num_pages))
        seq.state = State.WAITING
        self.waiting.append(seq)

    def is_finished(self):
        return not self.waiting and not self.running

    def abort(self, request_id, now=None):
        """Takes a request out, waiting or running: its pages and its state slot are given back at once and it
        finishes with the reason "aborted", keeping the tokens it has.  Returns the sequence, or None when no
        such request is alive.  A step that is already on the device may still hold the request: its token is
        passed over by absorb(), and what it writes lies in pages that nobody reads before they are written anew."""
        for seq in list(self.waiting) + self.running:
            if seq.request_id == request_id:
                break
        else:
            return None
        if seq.state is State.RUNNING:
            self.running.remove(seq)
        else:
            self.waiting.remove(seq)
        if self.cache.has(request_id):
            self.cache.release(request_id, seq.token_ids)
        seq.state, seq.finish_reason, seq.finish_ts = State.FINISHED, "aborted", now
        return seq

    # ---- one step
    def schedule(self) -> List[Scheduled]:
        cache = self.cache
        budget = self.max_num_batched_tokens
        out: List[Scheduled] = []

        # 1. decoding requests, oldest first; evict the newest when pages run out
        decoding = [s for s in self.running if s.remaining == 1 and s.num_computed > 0]
        i = 0
        while i < len(decoding) and budget > 0:
            seq = decoding[i]
            if seq.state is not State.RUNNING:      # evicted earlier in this loop
                i += 1
                continue
            try:
                cache.append(seq.request_id, 1)
            except OutOfPages:
                victim = self.running[-1]
                if any(sc.seq is victim for sc in out):
                    # the newest already holds its reservation for this step: undo it
                    out = [sc for sc in out if sc.seq is not victim]
                    budget += 1
                self._evict(victim)
                if victim is seq:
                    i += 1
                continue
            out.append(Scheduled(seq, 1, True))
            budget -= 1
            i += 1

        # 2. prompt portions of running requests (prompts not yet through)
        for seq in self.running:
            if budget <= 0:
                break
            if seq.remaining > 1 or seq.num_computed == 0:
                if any(sc.seq is seq for sc in out):
                    continue
                n = self._portion(seq, budget)
                if n > 0:
                    out.append(Scheduled(seq, n, n == seq.remaining))
                    budget -= n

        # 3. admissions in arrival order; no skipping ahead of the head of the queue
        while self.waiting and budget > 0 and len(self.running) < self.max_num_seqs and cache.can_admit():
            seq = self.waiting[0]
            cache.admit(seq.request_id, seq.token_ids)
            seq.num_computed = cache.length(seq.request_id)     # a known prefix is in the cache already
            n = self._portion(seq, budget)
            if n == 0:
                cache.release(seq.request_id)
                seq.num_computed = 0
                break
            self.waiting.popleft()
            seq.state = State.RUNNING
            self.running.append(seq)
            out.append(Scheduled(seq, n, n == seq.remaining))
            budget -= n

        if not out and not self.is_finished():
            # nothing fits: only possible when running prompts hold every page among them
            victim = self.running[-1] if self.running else None
            if victim is None or len(self.running) == 1:
                raise OutOfPages("no request can take a step: the cache is too small for the work in flight")
            self._evict(victim)
            return self.schedule()
        return out

    def _portion(self, seq, budget):
        """Reserves the largest portion of the request's remaining tokens that budget and pages allow."""
        n = min(seq.remaining, budget, self.cache.free_tokens(seq.request_id))
        while n > 0:
            try:
                self.cache.append(seq.request_id, n)
                return n
            except OutOfPages:
                n -= 1
        return 0

    def _evict(self, seq):
        self.cache.release(seq.request_id, seq.token_ids)
        self.running.remove(seq)
        seq.state = State.WAITING
        seq.num_computed = 0
        seq.decoding = False
        seq.evictions += 1
        self.num_evictions += 1
        self.waiting.appendleft(seq)

    # ---- after the step
    def postprocess(self, scheduled: List[Scheduled], tokens: List[int], now=None) -> List[Sequence]:
        """tokens: one sampled token for every scheduled item that samples, in order.  Appends them,
        finishes what is done (end-of-sequence id unless ignore_eos, max_tokens, max_model_len), frees
        their pages.  Returns the sequences that finished."""
        self.advance(scheduled)
        return self.absorb(scheduled, tokens, now)

    def advance(self, scheduled: List[Scheduled]):
        """The step has been handed to the device: its tokens count as computed."""
        cache = self.cache
        for sc in scheduled:
            rid = sc.seq.request_id
            if cache.pending(rid):
                cache.commit(rid, sc.seq.token_ids)
            sc.seq.num_computed += sc.num_tokens
            if sc.samples:
                sc.seq.decoding = True

    def absorb(self, scheduled: List[Scheduled], tokens: List[int], now=None) -> List[Sequence]:
        """The step's sampled tokens have arrived (one for every item that samples, in order): appends them and
        finishes what is done.  An item whose request finished meanwhile (a step launched ahead of the token that
        ended it) is passed over."""
        finished = []
        it = iter(tokens)
        for sc in scheduled:
            seq = sc.seq
            if not sc.samples:
                continue
            tok = int(next(it))
            if seq.state is not State.RUNNING:
                continue
            seq.token_ids.append(tok)
            if seq.first_token_ts is None:
                seq.first_token_ts = now
            stops = self.eos_token_ids if seq.params.stop_token_ids is None else set(seq.params.stop_token_ids)
            reason = None
            if not seq.params.ignore_eos and tok in stops:
                reason = "eos"
            elif seq.num_output_tokens >= seq.params.max_tokens:
                reason = "max_tokens"
            elif seq.num_tokens >= self.max_model_len:
                reason = "max_model_len"
            if reason:
                seq.state, seq.finish_reason, seq.finish_ts = State.FINISHED, reason, now
                self.cache.release(seq.request_id, seq.token_ids)
                self.running.remove(seq)
                finished.append(seq)
        return finished

    # ---- a step launched before the tokens of the step before it are known
    def schedule_ahead(self, scheduled: List[Scheduled]):
        """`scheduled` has been launched (and advanced) but its tokens have not been read yet.  If the step
        after it is certain to be one more token for every request that is still running, and nothing else,
        reserves that step and returns (its items, for each the index of its request in `scheduled`); else None,
        with nothing changed.  Certain means: every running request is in `scheduled` and samples there, none of
        them reaches max_tokens or max_model_len with the token it is about to get, no waiting request could be
        admitted, and the pages are there.  A request that ends on an end-of-sequence token nobody has seen yet
        runs one step too many; its result is dropped by absorb()."""
        alive = [(i, sc) for i, sc in enumerate(scheduled) if sc.seq.state is State.RUNNING]
        if not alive or len(alive) != len(self.running) or len(alive) > self.max_num_batched_tokens:
            return None
        if self.waiting and len(self.running) < self.max_num_seqs and self.cache.can_admit():
            return None
        for _, sc in alive:
            seq = sc.seq
            # every known token is computed and the next one is on its way: the request will hold `known` tokens
            known = len(seq.token_ids) + 1
            if not sc.samples or seq.num_computed != len(seq.token_ids) \
                    or known - seq.num_prompt_tokens >= seq.params.max_tokens or known >= self.max_model_len:
                return None
        reserved = []
        for _, sc in alive:
            try:
                self.cache.append(sc.seq.request_id, 1)
                reserved.append(sc.seq.request_id)
            except OutOfPages:
                for rid in reserved:
                    self.cache.cancel(rid)
                return None
        return [Scheduled(sc.seq, 1, True) for _, sc in alive], [i for i, _ in alive]
