"""The cache manager: keys and values in pages with a block table per request, and slots for
per-request state of fixed size.

Schedule entries of the model that keep keys and values fall into *groups* by what they need
(num_kv_heads, head_dim, window).  A group has a page pool of its own and every request has one block
table per group; all entries of a group share the table (page p means page p of every entry's
tensor).  Block table entry i covers positions [i * page_size, (i + 1) * page_size) of the request.
A group with a window gives a page back as soon as every position in it lies behind the window of the
next token to be computed; its table keeps a -1 there.  Pages return to the pool when a request is
released and are used again by later requests.  The reference has one pool, one table per sequence,
no window and no state (ginfer/engine/block_manager.cc:63-148, ginfer/engine/model_runner.cc:52-87).

Device layout of one group: one allocation [entries_in_group, 2 (k, v), pages, nkv * page_size * hd]; an
entry's keys are viewed [pages, nkv, page_size, hd] and its values [pages, nkv, hd, page_size]
(transposed inside a page, which is what the matrix-core attention kernels read fastest).
"""
from dataclasses import dataclass, field
from typing import Dict, List, Optional

import numpy as np

from ..parts.base import KVCacheSpec, StateSpec
from .pages import PagePool, SlotPool, OutOfPages


@dataclass
class _Request:
    slot: int
    length: int = 0                      # tokens whose keys/values (or state) are in the cache
    pending: int = 0                     # tokens reserved by append() and not yet committed
    tables: List[List[int]] = field(default_factory=list)   # per group: logical block -> page or -1


class CacheGroup:
    def __init__(self, spec, entries, num_pages, page_size):
        self.spec, self.entries, self.page_size = spec, list(entries), page_size
        self.pool = PagePool(num_pages)
        self.tensor = None               # device tensor, set by allocate_device

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
    def __init__(self, cache_specs, page_size, num_pages, max_requests):
        """cache_specs: per schedule entry KVCacheSpec | StateSpec | None (None: keeps nothing, or reads
        another entry's cache).  num_pages: pages of every group's pool."""
        if page_size < 1:
            raise ValueError("page_size must be positive")
        self.page_size, self.max_requests = int(page_size), int(max_requests)
        self.cache_specs = list(cache_specs)
        by_key: Dict[KVCacheSpec, List[int]] = {}
        for i, s in enumerate(self.cache_specs):
            if isinstance(s, KVCacheSpec):
                by_key.setdefault(s, []).append(i)
        self.groups = [CacheGroup(k, v, num_pages, self.page_size) for k, v in by_key.items()]
        self.group_of = {}               # schedule entry -> (group index, index inside the group)
        for gi, g in enumerate(self.groups):
            for j, e in enumerate(g.entries):
                self.group_of[e] = (gi, j)
        self.state_entries = [i for i, s in enumerate(self.cache_specs) if isinstance(s, StateSpec)]
        self.slots = SlotPool(self.max_requests)
        self.state_tensors = {}          # schedule entry -> device tensor [max_requests, *shape]
        self.requests: Dict[object, _Request] = {}
        # host mirrors for building a step without a Python loop per request: per group the block tables
        # by state slot (int32, -1 where there is no page), and the lengths by state slot
        self._table_np = [np.full((self.max_requests, 16), -1, dtype=np.int32) for _ in self.groups]
        self._length_np = np.zeros(self.max_requests, dtype=np.int64)
        self._any_window = any(g.window is not None for g in self.groups)

    # ---- device memory
    def bytes_per_page(self, element_size):
        return sum(len(g.entries) * 2 * g.spec.num_kv_heads * self.page_size * g.spec.head_dim * element_size
                   for g in self.groups)

    def allocate_device(self, dtype, device):
        import torch
        for g in self.groups:
            g.tensor = torch.zeros((len(g.entries), 2, g.pool.num_pages,
                                    g.spec.num_kv_heads * self.page_size * g.spec.head_dim), dtype=dtype, device=device)
        for e in self.state_entries:
            s = self.cache_specs[e]
            self.state_tensors[e] = torch.zeros((self.max_requests,) + tuple(s.shape), dtype=s.dtype, device=device)

    def kv_views(self, entry):
        """(k_pages [pages, nkv, page_size, hd], v_pages [pages, nkv, hd, page_size]) of a schedule entry."""
        gi, j = self.group_of[entry]
        g = self.groups[gi]
        n, nkv, hd = g.pool.num_pages, g.spec.num_kv_heads, g.spec.head_dim
        return (g.tensor[j, 0].view(n, nkv, self.page_size, hd), g.tensor[j, 1].view(n, nkv, hd, self.page_size))

    # ---- requests
    def has(self, rid):
        return rid in self.requests

    def can_admit(self):
        return self.slots.num_free > 0

    def admit(self, rid):
        if rid in self.requests:
            raise ValueError("request %r is already in the cache" % (rid,))
        self.requests[rid] = _Request(slot=self.slots.take(), tables=[[] for _ in self.groups])
        slot = self.requests[rid].slot
        for t in self._table_np:
            t[slot, :] = -1
        self._length_np[slot] = 0
        return slot

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
            first = g.first_needed_block(start)
            give = [i for i in range(min(first, len(table))) if table[i] >= 0]
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
            give = sum(1 for i in range(min(first, len(table))) if table[i] >= 0)
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
            while len(table) < need_blocks:
                table.append(-1)
            new_pages = iter(g.pool.take(take))
            for i in range(max(first, 0), need_blocks):
                if table[i] < 0:
                    table[i] = next(new_pages)
            mirror = self._table_np[gi]
            if len(table) > mirror.shape[1]:
                wider = np.full((self.max_requests, max(len(table), 2 * mirror.shape[1])), -1, dtype=np.int32)
                wider[:, :mirror.shape[1]] = mirror
                self._table_np[gi] = mirror = wider
            mirror[req.slot, :len(table)] = table
        req.pending = n_new
        return req.length

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

    def commit(self, rid):
        req = self.requests[rid]
        req.length += req.pending
        req.pending = 0
        self._length_np[req.slot] = req.length

    def release(self, rid):
        """The request ends (or is evicted): every page and its slot go back."""
        req = self.requests.pop(rid)
        for gi, g in enumerate(self.groups):
            g.pool.give_back([p for p in req.tables[gi] if p >= 0])
        self.slots.give_back(req.slot)

    # ---- checks (tests call this after every operation)
    def check(self):
        for gi, g in enumerate(self.groups):
            seen = {}
            for rid, req in self.requests.items():
                for p in req.tables[gi]:
                    if p < 0:
                        continue
                    if p in seen:
                        raise AssertionError("page %d of group %d is held by %r and %r" % (p, gi, seen[p], rid))
                    seen[p] = rid
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
