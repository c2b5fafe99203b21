"""The cache manager: keys and values in pages with a block table per request, and slots for
per-request state of fixed size.

What a schedule entry of the model keeps per request is a list of caches: any number of paged ones (keys and values,
`KVCacheSpec`, or any per-token tensors, `PagedSpec`) and of state slots (`StateSpec`); most entries keep one.  The
paged caches fall into *groups* by what they need (their spec: widths, window).  A group has a page pool of its own and
every request has one block table per group; all caches of a group share the table (page p means page p of every
cache's tensors).  Block table entry i covers positions [i * page_size, (i + 1) * page_size) of the request.
A group with a window gives a page back as soon as every position in it lies behind the window of the
next token to be computed; its table keeps a -1 there.  Pages return to the pool when a request is
released and are used again by later requests.  The reference has one pool, one table per sequence,
no window and no state (ginfer/engine/block_manager.cc:63-148, ginfer/engine/model_runner.cc:52-87).

Shared prefixes (optional; the reference always does it, block_manager.cc:63-110): a page that is full and
whose tokens are known is remembered under (what came before it, its tokens).  A request that is admitted
with its tokens takes over the remembered pages of its longest known prefix, as one more holder of each, and
starts behind them; at least its last token is left to run.  A remembered page that nobody holds lies in the
free queue like any other and is forgotten when it is taken for something else.  What came before a page is
named by a number that is never used twice, so a hit is exact: it compares tokens, not hashes of them (the
reference compares a 64-bit chain hash and the page's own tokens).  Only for models whose every cache group
keeps all keys and that have no per-request state: a window gives pages of a prefix back, and state has to
see every token.

Device layout of one group: for each tensor of its spec one allocation [caches_in_group, pages, page_size * elements
per token]; keys are viewed [pages, nkv, page_size, hd] and values [pages, nkv, value_dim, page_size] (transposed
inside a page, which is what the matrix-core attention kernels read fastest).
"""
from array import array
from dataclasses import dataclass, field
from typing import Dict, List, Optional

import numpy as np

from ..parts.base import KVCacheSpec, PagedSpec, StateSpec
from .pages import PagePool, SlotPool, OutOfPages


@dataclass
class _Request:
    slot: int
    length: int = 0                      # tokens whose keys/values (or state) are in the cache
    pending: int = 0                     # tokens reserved by append() and not yet committed
    tables: List[List[int]] = field(default_factory=list)   # per group: logical block -> page or -1
    contents: List[List[int]] = field(default_factory=list) # per group: content number of each remembered block
    gone: List[int] = field(default_factory=list)           # per group: every block before this one was given back
    hit: int = 0                         # tokens taken over from a remembered prefix, not yet counted as a hit


def _block_tokens(token_ids, block, page_size):
    """The tokens of one full block as a key: their 32-bit values as bytes (compact, and compared exactly)."""
    return array("i", token_ids[block * page_size:(block + 1) * page_size]).tobytes()


def _is_paged(spec):
    return isinstance(spec, (KVCacheSpec, PagedSpec))


def caches_of(entry_spec):
    """What a schedule entry keeps, as a list: a single spec stands for a list of one, None for none."""
    if entry_spec is None:
        return []
    if isinstance(entry_spec, (list, tuple)):
        return list(entry_spec)
    return [entry_spec]


class CacheGroup:
    def __init__(self, spec, units, num_pages, page_size):
        """units: the caches of the group as (schedule entry, place in the entry's list)."""
        self.spec, self.units, self.page_size = spec, list(units), page_size
        self.entries = [e for e, _ in self.units]
        self.pool = PagePool(num_pages)
        self.tensors = None              # device tensors by name [caches, pages, page_size * elements], set by allocate_device
        # full pages whose tokens are known, for requests that share a prefix
        self._page_of = {}               # (content number of the block before or 0, the block's tokens) -> page
        self._key_of = {}                # page -> its key in _page_of
        self._content_of = {}            # page -> content number, never used twice
        self._contents = 0

    def lookup(self, before, tokens):
        """(page, content number) of the remembered block with these tokens after the content `before`, or None."""
        page = self._page_of.get((before, tokens))
        return None if page is None else (page, self._content_of[page])

    def remember(self, before, tokens, page):
        """The page holds the block with these tokens after `before`.  Returns the block's content number: a new
        one, or that of a page remembered earlier for the same content (this page then stays unknown)."""
        known = self._page_of.get((before, tokens))
        if known is not None:
            return self._content_of[known]
        self.forget(page)
        self._contents += 1
        self._page_of[(before, tokens)] = page
        self._key_of[page] = (before, tokens)
        self._content_of[page] = self._contents
        return self._contents

    def forget(self, page):
        key = self._key_of.pop(page, None)
        if key is not None:
            del self._page_of[key]
            del self._content_of[page]

    @property
    def window(self):
        return self.spec.window

    def first_needed_block(self, next_pos):
        """Blocks before this one hold only positions that no query at or after next_pos can see."""
        if self.window is None:
            return 0
        lo = next_pos - self.window + 1
        return max(lo, 0) // self.page_size


class CacheManager:
    def __init__(self, cache_specs, page_size, num_pages, max_requests, prefix_caching=False):
        """cache_specs: per schedule entry KVCacheSpec | PagedSpec | StateSpec | None, or a list of them (None: keeps
        nothing, or reads another entry's cache).  num_pages: pages of every group's pool, or a list with one count per group (in the
        order of `group_specs(cache_specs)`; a group with a window needs few, see `plan_pages`).  prefix_caching:
        requests admitted with their tokens share the pages of a known prefix."""
        if prefix_caching and not self.supports_prefix_caching(cache_specs):
            raise ValueError("prefixes cannot be shared in a model with a window or with per-request state")
        self.prefix_caching = bool(prefix_caching)
        self.prefix_hit_tokens = 0
        if page_size < 1:
            raise ValueError("page_size must be positive")
        self.page_size, self.max_requests = int(page_size), int(max_requests)
        self.cache_specs = list(cache_specs)
        by_key = self.group_specs(self.cache_specs)
        if isinstance(num_pages, (list, tuple)):
            if len(num_pages) != len(by_key):
                raise ValueError("%d page counts for %d cache groups" % (len(num_pages), len(by_key)))
            counts = [int(n) for n in num_pages]
        else:
            counts = [int(num_pages)] * len(by_key)
        self.groups = [CacheGroup(k, v, n, self.page_size) for (k, v), n in zip(by_key.items(), counts)]
        self.group_of = {}               # (schedule entry, place in its list) -> (group index, index inside the group)
        for gi, g in enumerate(self.groups):
            for j, unit in enumerate(g.units):
                self.group_of[unit] = (gi, j)
        self.state_units = [(i, k) for i, s in enumerate(self.cache_specs) for k, c in enumerate(caches_of(s))
                            if isinstance(c, StateSpec)]
        self.slots = SlotPool(self.max_requests)
        # one more slot than requests: the rows that pad a recorded step read and write the state of this slot, which
        # no request ever holds
        self.pad_slot = self.max_requests
        self.state_tensors = {}          # (schedule entry, place in its list) -> device tensor [max_requests + 1, *shape]
        self.requests: Dict[object, _Request] = {}
        # host mirrors for building a step without a Python loop per request: per group the block tables
        # by state slot (int32, -1 where there is no page), and the lengths by state slot
        self._table_np = [np.full((self.max_requests, 16), -1, dtype=np.int32) for _ in self.groups]
        self._length_np = np.zeros(self.max_requests, dtype=np.int64)
        self._any_window = any(g.window is not None for g in self.groups)

    @staticmethod
    def group_specs(cache_specs):
        """{paged spec: [(schedule entry, place in its list)]} in the order in which the groups are made."""
        by_key = {}
        for i, s in enumerate(cache_specs):
            for k, c in enumerate(caches_of(s)):
                if _is_paged(c):
                    by_key.setdefault(c, []).append((i, k))
        return by_key

    @staticmethod
    def state_bytes(cache_specs, max_requests):
        """Device bytes of the per-request state: every state tensor has a slot for each request and one more."""
        import torch
        total = 0
        for s in cache_specs:
            for c in caches_of(s):
                if isinstance(c, StateSpec):
                    n = 1
                    for d in c.shape:
                        n *= int(d)
                    total += (max_requests + 1) * n * torch.empty(0, dtype=c.dtype).element_size()
        return total

    @staticmethod
    def window_span_pages(window, page_size):
        """Pages that `window` consecutive positions can touch: what a request of a group with this window holds between
        steps (`commit` gives back what lies behind the window of the next token) and while one more token runs."""
        return (window - 1) // page_size + 2

    @classmethod
    def window_pages(cls, window, page_size, max_requests, max_step_tokens, max_model_len):
        """Pages that a group with this window can hold at most.  While a request runs n tokens of a step it holds the
        pages of the positions [length - window + 1, length + n): at most `window_span_pages` + 1 + (n - 1) // page; over
        the requests of a step the n add up to the step's token budget.  Never more than all keys of every request."""
        per_request_all = -(-max_model_len // page_size)
        per_request = min(cls.window_span_pages(window, page_size) + 1, per_request_all)
        return min(max_requests * per_request + -(-max_step_tokens // page_size), max_requests * per_request_all)

    @classmethod
    def plan_pages(cls, cache_specs, page_size, element_size, pool_bytes, max_requests, max_step_tokens, max_model_len):
        """Page counts per group for a pool of pool_bytes: a group with a window gets what it can ever hold
        (`window_pages`), the groups that keep all keys share the rest alike (every one of them holds the same number
        of pages per token).  Raises if the bytes do not give every group a page."""
        groups = cls.group_specs(cache_specs)
        if not groups:
            return []
        page_bytes = [len(units) * sum(w for _, w in spec.page_tensors()) * page_size * element_size
                      for spec, units in groups.items()]
        counts, left = [None] * len(groups), int(pool_bytes)
        for gi, spec in enumerate(groups):
            if spec.window is not None:
                counts[gi] = cls.window_pages(spec.window, page_size, max_requests, max_step_tokens, max_model_len)
                left -= counts[gi] * page_bytes[gi]
        rest = [gi for gi, c in enumerate(counts) if c is None]
        if rest:
            per = left // sum(page_bytes[gi] for gi in rest) if left > 0 else 0
            for gi in rest:
                counts[gi] = per
        elif left < 0:       # windows only and too little memory: shrink them alike
            total = sum(c * b for c, b in zip(counts, page_bytes))
            counts = [c * int(pool_bytes) // total for c in counts]
        if min(counts) < 1:
            raise RuntimeError("no memory left for the cache: %d bytes give the groups %s pages (a page of each takes %s bytes)"
                               % (pool_bytes, counts, page_bytes))
        return counts

    @staticmethod
    def supports_prefix_caching(cache_specs):
        flat = [c for s in cache_specs for c in caches_of(s)]
        return (any(_is_paged(c) for c in flat)
                and not any(isinstance(c, StateSpec) or (_is_paged(c) and c.window is not None) for c in flat))

    # ---- device memory
    def pool_bytes(self, element_size):
        return sum(g.pool.num_pages * len(g.units) * sum(w for _, w in g.spec.page_tensors()) * self.page_size
                   * element_size for g in self.groups)

    def allocate_device(self, dtype, device):
        import torch
        for g in self.groups:
            g.tensors = {name: torch.zeros((len(g.units), g.pool.num_pages, self.page_size * width), dtype=dtype,
                                           device=device) for name, width in g.spec.page_tensors()}
        for unit in self.state_units:
            s = caches_of(self.cache_specs[unit[0]])[unit[1]]
            self.state_tensors[unit] = torch.zeros((self.max_requests + 1,) + tuple(s.shape), dtype=s.dtype, device=device)

    def page_views(self, entry, place=0):
        """{name: [pages, page_size * elements per token]} of one paged cache of a schedule entry."""
        gi, j = self.group_of[(entry, place)]
        return {name: t[j] for name, t in self.groups[gi].tensors.items()}

    def kv_views(self, entry, place=0):
        """(k_pages [pages, nkv, page_size, hd], v_pages [pages, nkv, value_dim, page_size]) of a cache of keys and values."""
        gi, j = self.group_of[(entry, place)]
        g = self.groups[gi]
        n, nkv = g.pool.num_pages, g.spec.num_kv_heads
        return (g.tensors["k"][j].view(n, nkv, self.page_size, g.spec.head_dim),
                g.tensors["v"][j].view(n, nkv, g.spec.v_dim, self.page_size))

    # ---- requests
    def has(self, rid):
        return rid in self.requests

    def can_admit(self):
        return self.slots.num_free > 0

    def admit(self, rid, token_ids=None):
        """A state slot and empty block tables for the request.  With token_ids (and prefix caching): the pages of
        the longest remembered prefix are taken over, and length(rid) tells how many tokens they hold."""
        if rid in self.requests:
            raise ValueError("request %r is already in the cache" % (rid,))
        req = self.requests[rid] = _Request(slot=self.slots.take(), tables=[[] for _ in self.groups],
                                            contents=[[] for _ in self.groups], gone=[0] * len(self.groups))
        slot = req.slot
        for t in self._table_np:
            t[slot, :] = -1
        self._length_np[slot] = 0
        if self.prefix_caching and token_ids is not None:
            self._share_prefix(req, token_ids)
        return slot

    def _share_prefix(self, req, token_ids):
        ps = self.page_size
        blocks = (len(token_ids) - 1) // ps          # the last token at least is left to run
        chains = []
        for g in self.groups:
            chain, before = [], 0
            for i in range(blocks):
                hit = g.lookup(before, _block_tokens(token_ids, i, ps))
                if hit is None:
                    break
                chain.append(hit)
                before = hit[1]
            chains.append(chain)
            blocks = len(chain)
        if blocks == 0:
            return
        for gi, g in enumerate(self.groups):
            for page, content in chains[gi][:blocks]:
                g.pool.share(page)
                req.tables[gi].append(page)
                req.contents[gi].append(content)
            self._mirror_table(gi, req)
        req.length = blocks * ps
        self._length_np[req.slot] = req.length
        req.hit = req.length             # counted once the request's first tokens are reserved: an admission that is
                                         # taken back for lack of pages, and tried again step after step, is no hit

    def _remember(self, req, token_ids):
        """Remembers the request's full pages whose tokens are known and whose keys and values are committed."""
        ps = self.page_size
        full = min(req.length, len(token_ids)) // ps
        for gi, g in enumerate(self.groups):
            chain, table = req.contents[gi], req.tables[gi]
            for i in range(len(chain), full):
                chain.append(g.remember(chain[i - 1] if i else 0, _block_tokens(token_ids, i, ps), table[i]))

    def _mirror_table(self, gi, req, changed=None):
        """Copies the request's table of a group into the host mirror: all of it, or the blocks named."""
        table, mirror = req.tables[gi], self._table_np[gi]
        if len(table) > mirror.shape[1]:
            wider = np.full((self.max_requests, max(len(table), 2 * mirror.shape[1])), -1, dtype=np.int32)
            wider[:, :mirror.shape[1]] = mirror
            self._table_np[gi] = mirror = wider
        if changed is None:
            mirror[req.slot, :len(table)] = table
        else:
            for i in changed:
                mirror[req.slot, i] = table[i]

    def length(self, rid):
        return self.requests[rid].length

    def pending(self, rid):
        return self.requests[rid].pending

    def slot(self, rid):
        return self.requests[rid].slot

    def table(self, rid, group):
        return self.requests[rid].tables[group]

    def _plan(self, req, n_new):
        """Per group: (blocks to give back, pages to take) for n_new more tokens."""
        plan = []
        start, end = req.length, req.length + n_new
        need_blocks = -(-end // self.page_size)
        for gi, g in enumerate(self.groups):
            table = req.tables[gi]
            if g.window is None:         # a table without a window has no gaps: what is missing lies at its end
                plan.append(([], max(0, need_blocks - len(table)), 0, need_blocks))
                continue
            first = g.first_needed_block(start)
            give = [i for i in range(req.gone[gi], min(first, len(table))) if table[i] >= 0]
            take = 0
            for i in range(max(first, 0), need_blocks):
                if i >= len(table) or table[i] < 0:
                    take += 1
            plan.append((give, take, first, need_blocks))
        return plan

    def pages_short(self, rid, n_new, reserved=None):
        """How many pages the fullest group lacks to take n_new more tokens of this request (0: fits).
        `reserved`: per group, pages already promised to other requests of the same step."""
        req = self.requests[rid]
        short = 0
        for gi, (give, take, _, _) in enumerate(self._plan(req, n_new)):
            free = self.groups[gi].pool.num_free + len(give) - (reserved[gi] if reserved else 0)
            short = max(short, take - free)
        return max(short, 0)

    def can_append(self, rid, n_new):
        return self.pages_short(rid, n_new) == 0

    def free_tokens(self, rid):
        """How many more tokens of this request fit into the pages that are free now."""
        req = self.requests[rid]
        best = None
        for gi, g in enumerate(self.groups):
            table = req.tables[gi]
            first = g.first_needed_block(req.length)
            give = sum(1 for i in range(req.gone[gi], min(first, len(table))) if table[i] >= 0)
            have_blocks = len(table)
            room = have_blocks * self.page_size - req.length if have_blocks * self.page_size > req.length else 0
            cap = room + (g.pool.num_free + give) * self.page_size
            best = cap if best is None else min(best, cap)
        return best if best is not None else 1 << 60

    def append(self, rid, n_new):
        """Reserves room for the request's next n_new tokens: gives back pages behind the window, takes
        pages for the new positions.  All or nothing: raises OutOfPages and changes nothing if any group
        lacks pages.  Returns the position of the first new token."""
        req = self.requests[rid]
        if req.pending:
            raise ValueError("request %r has %d reserved tokens that were not committed" % (rid, req.pending))
        if n_new < 1:
            raise ValueError("append needs at least one token")
        hit, req.hit = req.hit, 0
        try:
            first = self._append(req, rid, n_new)
        except OutOfPages:
            req.hit = hit
            raise
        self.prefix_hit_tokens += hit
        return first

    def _append(self, req, rid, n_new):
        if n_new == 1 and not self._any_window and req.length % self.page_size:
            req.pending = 1              # the common decode step: room is left in the last page
            return req.length
        plan = self._plan(req, n_new)
        for gi, (give, take, _, _) in enumerate(plan):
            if take > self.groups[gi].pool.num_free + len(give):
                raise OutOfPages("request %r needs %d more pages of group %d, %d free"
                                 % (rid, take - len(give), gi, self.groups[gi].pool.num_free))
        for gi, (give, take, first, need_blocks) in enumerate(plan):
            g, table = self.groups[gi], req.tables[gi]
            g.pool.give_back([table[i] for i in give])
            for i in give:
                table[i] = -1
            req.gone[gi] = max(req.gone[gi], min(first, len(table)))
            scan_from = max(first, 0) if g.window is not None else len(table)
            while len(table) < need_blocks:
                table.append(-1)
            taken = g.pool.take(take)
            for p in taken:
                g.forget(p)              # what the page held for requests to come is gone
            new_pages = iter(taken)
            changed = list(give)
            for i in range(scan_from, need_blocks):
                if table[i] < 0:
                    table[i] = next(new_pages)
                    changed.append(i)
            self._mirror_table(gi, req, changed)
        req.pending = n_new
        return req.length

    def cancel(self, rid):
        """The reserved tokens will not run after all.  Pages that the reservation took stay in the request's table, where
        its next reservation finds them."""
        self.requests[rid].pending = 0

    def tables_array(self, group, slots, width):
        """int32 [len(slots), width]: the block tables of the requests in these state slots."""
        mirror = self._table_np[group]
        if width > mirror.shape[1]:
            out = np.full((len(slots), width), -1, dtype=np.int32)
            out[:, :mirror.shape[1]] = mirror[slots]
            return out
        return mirror[slots, :width]

    def lengths_array(self, slots):
        return self._length_np[slots]

    def commit(self, rid, token_ids=None):
        """The reserved tokens are in the cache (or on their way there, in stream order).  token_ids: the
        request's tokens as far as they are known, for remembering pages that are full now."""
        req = self.requests[rid]
        req.length += req.pending
        req.pending = 0
        self._length_np[req.slot] = req.length
        if self.prefix_caching and token_ids is not None:
            self._remember(req, token_ids)
        if self._any_window:
            # what lies behind the window of the next token goes back now: whoever takes such a page writes it in a
            # later step, behind this step's reads in stream order.  Between steps a request then holds the pages of
            # one window only, which is what `window_pages` counts on.
            for gi, g in enumerate(self.groups):
                if g.window is None:
                    continue
                table = req.tables[gi]
                first = min(g.first_needed_block(req.length), len(table))
                give = [i for i in range(req.gone[gi], first) if table[i] >= 0]
                if give:
                    g.pool.give_back([table[i] for i in give])
                    for i in give:
                        table[i] = -1
                    self._mirror_table(gi, req, give)
                req.gone[gi] = max(req.gone[gi], first)

    def release(self, rid, token_ids=None):
        """The request ends (or is evicted): every page and its slot go back, the pages of its end first, so
        that the start of what it held is the last to be taken for something else."""
        req = self.requests.pop(rid)
        if self.prefix_caching and token_ids is not None:
            self._remember(req, token_ids)
        for gi, g in enumerate(self.groups):
            g.pool.give_back([p for p in reversed(req.tables[gi]) if p >= 0])
        self.slots.give_back(req.slot)

    # ---- checks (tests call this after every operation)
    def check(self):
        for gi, g in enumerate(self.groups):
            seen = {}
            for rid, req in self.requests.items():
                for p in req.tables[gi]:
                    if p < 0:
                        continue
                    if p in seen and not self.prefix_caching:
                        raise AssertionError("page %d of group %d is held by %r and %r" % (p, gi, seen[p][0], rid))
                    seen.setdefault(p, []).append(rid)
                if len(set(p for p in req.tables[gi] if p >= 0)) != sum(1 for p in req.tables[gi] if p >= 0):
                    raise AssertionError("group %d: %r holds a page twice" % (gi, rid))
            for p, rids in seen.items():
                if g.pool.holders(p) != len(rids):
                    raise AssertionError("page %d of group %d has %d holders, tables say %r"
                                         % (p, gi, g.pool.holders(p), rids))
                if len(rids) > 1 and p not in g._key_of:
                    raise AssertionError("page %d of group %d is shared by %r but not remembered" % (p, gi, rids))
            for key, p in g._page_of.items():
                if g._key_of.get(p) != key or p not in g._content_of:
                    raise AssertionError("group %d: the records of remembered page %d disagree" % (gi, p))
            if len(g._key_of) != len(g._page_of) or len(g._content_of) != len(g._page_of):
                raise AssertionError("group %d: records of remembered pages left over" % gi)
            held = set(g.pool.held())
            if held != set(seen):
                raise AssertionError("group %d: pool holds %s, tables hold %s" % (gi, sorted(held), sorted(seen)))
            for rid, req in self.requests.items():
                row = self._table_np[gi][req.slot]
                t = req.tables[gi]
                if list(row[:len(t)]) != t or (row[len(t):] >= 0).any():
                    raise AssertionError("group %d: the host mirror of %r's table differs from the table" % (gi, rid))
                if self._length_np[req.slot] != req.length:
                    raise AssertionError("the host mirror of %r's length differs" % (rid,))
            if len(held) + g.pool.num_free != g.pool.num_pages:
                raise AssertionError("group %d: %d held + %d free != %d pages"
                                     % (gi, len(held), g.pool.num_free, g.pool.num_pages))
        slots = [r.slot for r in self.requests.values()]
        if len(set(slots)) != len(slots):
            raise AssertionError("a state slot is held twice: %s" % slots)
        if len(slots) + self.slots.num_free != self.slots.num_slots:
            raise AssertionError("state slots lost: %d held + %d free != %d"
                                 % (len(slots), self.slots.num_free, self.slots.num_slots))
