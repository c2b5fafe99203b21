"""How a layer's parts are arranged around the residual stream."""
from ..kernels import ops
from .registry import register_arrangement


class Arrangement:
    """How a layer's parts sit around the residual stream.  A kind of arrangement says which roles it has and of which
    family each is (`roles`: role -> "mixer" | "feed_forward" | "norm"); the model builds the parts that a layer names
    for exactly these roles and hands them over as a dictionary.  Every part becomes an attribute under its role's
    name.  forward(residual float32 [T, H], delta, step, cache) takes the output of the block before as a pending
    `delta` (it is added to the residual by the first norm that runs) and returns its own last output as the next one.
    cache_spec(): what one run of the block keeps per request; the mixer's, unless the kind says otherwise (a block with
    several parts that keep something returns the list of their specs and gets the list of views as `cache`)."""

    roles = {}

    def __init__(self, parts):
        self._parts = dict(parts)
        for role, part in self._parts.items():
            setattr(self, role, part)

    def parts(self):
        """(role, part) pairs; the roles are what `LayerSpec.names` gives tensor prefixes for."""
        return list(self._parts.items())

    def cache_spec(self):
        mixer = self._parts.get("mixer")
        return mixer.cache_spec() if mixer is not None else None

    def forward(self, residual, delta, step, cache):
        raise NotImplementedError


@register_arrangement("prenorm")
class PreNormBlock(Arrangement):
    """n = norm1(x); h = x + mixer(n); n = norm2(h); x = h + feed_forward(n)
    (ginfer/core/layer/transformer/encoder.cc:33-39).  The residual stream is kept in 32-bit and every add
    is fused into the norm that follows it, so a block takes the previous block's output as a pending
    `delta` and returns its own feed-forward output as the next one.  Where the mixer says `folds_norm`, the
    feed-forward `takes_scaled_rows` and the norm between them is `foldable`, the mixer may add its result to
    the residual itself and hand the norm's rows on in two factors (ops.ScaledRows): then the second norm makes
    no pass over memory of its own.  The same holds across blocks: a block whose feed-forward `folds_norm` may be
    given the first norm of the block that runs next (`into_norm`), if that block says `takes_folded_input()`;
    it then returns ops.ScaledRows in place of its delta, and the next block skips its first norm."""

    roles = {"mixer": "mixer", "feed_forward": "feed_forward", "mixer_norm": "norm", "feed_forward_norm": "norm"}

    def __init__(self, parts):
        super().__init__(parts)
        mixer, feed_forward, feed_forward_norm = self.mixer, self.feed_forward, self.feed_forward_norm
        self.folds = (getattr(mixer, "folds_norm", False) and getattr(feed_forward, "takes_scaled_rows", False)
                      and getattr(feed_forward_norm, "foldable", False))

    @property
    def folds_output(self):
        """Whether forward() takes `into_norm`."""
        return bool(getattr(self.feed_forward, "folds_norm", False))

    def takes_folded_input(self):
        """The norm whose rows this block takes in two factors (ops.ScaledRows) in place of a delta, or None."""
        if getattr(self.mixer, "takes_scaled_rows", False) and getattr(self.mixer_norm, "foldable", False):
            return self.mixer_norm
        return None

    def forward(self, residual, delta, step, cache, into_norm=None):
        if isinstance(delta, ops.ScaledRows):      # the block before has added its output and folded this norm
            n = delta
        else:
            n = self.mixer_norm.forward(residual, whole(delta, self.mixer_norm))
        if self.folds:
            a = self.mixer.forward(n, step, cache, into_norm=(residual, self.feed_forward_norm))
        else:
            a = self.mixer.forward(n, step, cache)
        if not isinstance(a, ops.ScaledRows):
            a = self.feed_forward_norm.forward(residual, whole(a, self.feed_forward_norm))
        if into_norm is not None:
            return self.feed_forward.forward(a, into_norm=(residual, into_norm))
        return self.feed_forward.forward(a)


def whole(delta, norm=None):
    """A mixer or feed-forward may hand on float32 partial sums [parts, T, H] of a K-split product.  A norm
    that says `accepts_partial_sums` adds them up itself; for any other (or for none) they are added up here."""
    if delta is not None and delta.dim() == 3 and not getattr(norm, "accepts_partial_sums", False):
        total = delta.sum(dim=0)
        return total.to(norm.dtype) if norm is not None else total
    return delta
