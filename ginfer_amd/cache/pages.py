"""A pool of cache pages and a pool of state slots: plain bookkeeping, no device memory."""
from collections import OrderedDict


class OutOfPages(RuntimeError):
    pass


class PagePool:
    """Pages 0..num_pages-1 with a count of holders each.  Taken from the front of the free queue and given back
    to its end, as the reference's free deque (ginfer/engine/block_manager.cc:28-61), so a freed page is used
    again only after the pages that were free before it.  A page may have several holders (requests that share a
    prefix, block_manager.cc:83-96); it is free when the last one gives it back, and a free page can be taken out
    of the queue again by share() while nobody else has taken it."""

    def __init__(self, num_pages):
        if num_pages < 0:
            raise ValueError("a pool cannot hold %d pages" % num_pages)
        self.num_pages = int(num_pages)
        self._free = OrderedDict((p, None) for p in range(self.num_pages))    # an ordered set
        self._holders = [0] * self.num_pages

    @property
    def num_free(self):
        return len(self._free)

    def take(self, n):
        if n > len(self._free):
            raise OutOfPages("asked for %d pages, %d free of %d" % (n, len(self._free), self.num_pages))
        out = []
        for _ in range(n):
            p, _none = self._free.popitem(last=False)
            self._holders[p] = 1
            out.append(p)
        return out

    def share(self, p):
        """One more holder of page p, which is held already or still lies in the free queue with what it held."""
        if not 0 <= p < self.num_pages:
            raise ValueError("page %r is not of this pool" % (p,))
        if self._holders[p] == 0:
            del self._free[p]
        self._holders[p] += 1

    def give_back(self, pages):
        for p in pages:
            if not 0 <= p < self.num_pages:
                raise ValueError("page %r is not of this pool" % (p,))
            if self._holders[p] == 0:
                raise ValueError("page %d is given back but not held" % p)
            self._holders[p] -= 1
            if self._holders[p] == 0:
                self._free[p] = None

    def holders(self, p):
        return self._holders[p]

    def held(self):
        return [p for p, h in enumerate(self._holders) if h]


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
