"""A pool of cache pages and a pool of state slots: plain bookkeeping, no device memory."""
from collections import deque


class OutOfPages(RuntimeError):
    pass


class PagePool:
    """Pages 0..num_pages-1.  Taken from the front of the free queue and given back to its end, as the
    reference's free deque (ginfer/engine/block_manager.cc:28-61), so a freed page is used again only
    after the pages that were free before it."""

    def __init__(self, num_pages):
        if num_pages < 0:
            raise ValueError("a pool cannot hold %d pages" % num_pages)
        self.num_pages = int(num_pages)
        self._free = deque(range(self.num_pages))
        self._held = [False] * self.num_pages

    @property
    def num_free(self):
        return len(self._free)

    def take(self, n):
        if n > len(self._free):
            raise OutOfPages("asked for %d pages, %d free of %d" % (n, len(self._free), self.num_pages))
        out = []
        for _ in range(n):
            p = self._free.popleft()
            self._held[p] = True
            out.append(p)
        return out

    def give_back(self, pages):
        for p in pages:
            if not 0 <= p < self.num_pages:
                raise ValueError("page %r is not of this pool" % (p,))
            if not self._held[p]:
                raise ValueError("page %d is given back but not held" % p)
            self._held[p] = False
            self._free.append(p)

    def held(self):
        return [p for p, h in enumerate(self._held) if h]


class SlotPool:
    """Slots for per-request state of fixed size; the lowest free slot is taken first."""

    def __init__(self, num_slots):
        self.num_slots = int(num_slots)
        self._free = list(range(self.num_slots - 1, -1, -1))
        self._held = [False] * self.num_slots

    @property
    def num_free(self):
        return len(self._free)

    def take(self):
        if not self._free:
            raise OutOfPages("no free state slot (%d slots)" % self.num_slots)
        s = self._free.pop()
        self._held[s] = True
        return s

    def give_back(self, s):
        if not 0 <= s < self.num_slots or not self._held[s]:
            raise ValueError("slot %r is given back but not held" % (s,))
        self._held[s] = False
        self._free.append(s)
        self._free.sort(reverse=True)
