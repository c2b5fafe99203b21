"""Interfaces of the parts a model is put together from.

Every part
  * is constructed as `cls(dtype=..., device=..., **spec.params)` (a position encoding, where a mixer
    has one, arrives already built under the parameter `position`);
  * says which tensors it needs: `weight_specs() -> {local name: WeightSpec}`; local names are joined
    to the part's prefix by the model, e.g. "model.layers.3.self_attn" + "." + "q_proj.weight";
  * may name tensors that a checkpoint is allowed to carry although the part never reads them:
    `unread_weights() -> [local name, ...]` (a tied head's own copy of the table);
  * receives them, already on the device and in the right dtype: `bind_weights({local name: tensor})`;
  * names the kernel libraries it launches: `kernel_modules() -> [module, ...]`;
  * says whether its forward may be recorded into a HIP graph: `capturable` (False unless the part sets
    it).  A capturable forward launches the same kernels with the same arguments whatever the step's
    host-side numbers are: it reads sizes only from tensor shapes, does nothing that waits for the device,
    and takes everything that changes from step to step from the step's device arrays.

Mixer         forward(x [T, H], step, cache) -> [T, H], or float32 [parts, T, H]: partial sums that the
              norm which follows adds up in order (what a K-split matrix product leaves)
              cache_spec() -> KVCacheSpec | PagedSpec | StateSpec | None, or a list of them: what one run of
              this mixer keeps per request (pages and, or, a state slot); `cache` in forward is the matching
              view (`KVView`, `StateView` or None; a list of views for a list of specs) of the schedule entry
              that is running.  `step` is the `StepContext` of the batch.
FeedForward   forward(x [T, H]) -> [T, H] (or partial sums, as a mixer)
Norm          forward(residual float32 [T, H], delta [T, H] | None, rows=None) -> [R or T, H]; a norm that
              sets `accepts_partial_sums` also takes delta as float32 [parts, T, H] (else the block adds
              the parts up before it calls the norm); it keeps its compute dtype in `dtype`
              adds delta into the 32-bit residual stream and returns the normalised rows; with `rows`
              (int32 indices) only those rows are returned and the residual is left as it is.
Position      what the mixer's kernel needs to encode positions (for rotary kinds: `tables()`).
Embedding     forward(token_ids int32 [T], step) -> float32 [T, H] (the start of the residual stream; `step` is the
              batch's `StepContext`, for an embedding that adds something by position)
Head          forward(x [R, H]) -> float32 logits [R, V]
Arrangement   how a layer's parts are ordered around the residual stream (see block.py).
"""
from dataclasses import dataclass
from typing import Optional, Tuple

import torch


@dataclass(frozen=True)
class PagedSpec:
    """Anything kept per token, in pages: `tensors` lists (name, elements per token) of every tensor a page holds; a
    page of the group's pool is, for each of them, page_size * elements in a row, which the mixer views as it likes.
    window: None keeps every token; an integer w keeps only what a token at position p can still see (positions > p - w).
    Mixers with the same spec share a pool and a block table."""
    tensors: Tuple[Tuple[str, int], ...]
    window: Optional[int] = None

    def page_tensors(self):
        return tuple((str(n), int(w)) for n, w in self.tensors)


@dataclass(frozen=True)
class KVCacheSpec:
    """Keys and values in pages: per token and kv head a key of head_dim and a value of value_dim elements (the keys'
    width unless given).  window: None keeps all keys; an integer w keeps only what queries can still see
    (positions > p - w)."""
    num_kv_heads: int
    head_dim: int
    window: Optional[int] = None
    value_dim: Optional[int] = None

    @property
    def v_dim(self):
        return self.head_dim if self.value_dim is None else self.value_dim

    def page_tensors(self):
        return (("k", self.num_kv_heads * self.head_dim), ("v", self.num_kv_heads * self.v_dim))


@dataclass(frozen=True)
class StateSpec:
    """State of fixed size per request: one tensor of `shape` and `dtype` in a slot."""
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


class Part:
    capturable = False

    def weight_specs(self):
        return {}

    def unread_weights(self):
        return []

    def bind_weights(self, tensors):
        if tensors:
            raise ValueError("%s takes no weights, got %s" % (type(self).__name__, sorted(tensors)))

    def kernel_modules(self):
        return []
