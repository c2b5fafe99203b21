"""Counter-based uniform numbers: uniform(seed, n) is a pure function, so the n-th output token of a
request draws the same number however the request was batched, cut or evicted and recomputed."""
import struct

_MASK = (1 << 64) - 1


def _mix(z):
    # the finaliser of splitmix64
    z = (z + 0x9E3779B97F4A7C15) & _MASK
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    return z ^ (z >> 31)


def uniform(seed, n):
    """A float32-exact number in [0, 1) for output position n of a request with this seed."""
    z = _mix(_mix(seed & _MASK) ^ ((n + 1) * 0xD1342543DE82EF95 & _MASK))
    return (z >> 40) / float(1 << 24)


def request_seed(request_id):
    """The seed of a request that names none: a function of its id alone."""
    return _mix((int(request_id) & _MASK) ^ 0xA0761D6478BD642F)
