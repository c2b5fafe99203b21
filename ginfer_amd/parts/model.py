"""The model: parts put together from a `ModelSpec`, and one forward over a step's tokens."""
from dataclasses import dataclass
from typing import List, Optional

import torch

from . import registry
from .base import KVCacheSpec, StateSpec
from .block import whole


@dataclass
class KVView:
    """What a mixer sees of one paged cache of the schedule entry that is running.  A cache of keys and values
    (`KVCacheSpec`) comes as k_pages and v_pages; any other paged cache (`PagedSpec`) as `pages`, its tensors by name,
    each [pages, page_size * elements per token], for the mixer to view as it likes."""
    k_pages: Optional[torch.Tensor]    # [pages, nkv, page_size, hd]
    v_pages: Optional[torch.Tensor]    # [pages, nkv, value_dim, page_size]: values are kept transposed
    block_table: torch.Tensor      # int32 [entries, width]; -1 where a page was given back
    slot_mapping: torch.Tensor     # int64 [T]: page * page_size + offset for every token of the step
    page_size: int
    owner: bool                    # False when this run reads another entry's cache and must not write
    pages: Optional[dict] = None


@dataclass
class StateView:
    """Per-request state of fixed size: `state[slots[e]]` belongs to entry e of the step."""
    state: torch.Tensor            # [num_slots, *shape]
    slots: torch.Tensor            # int64 [entries]
    owner: bool


@dataclass
class StepContext:
    """One batch of (request, its next tokens), flattened.  Entry e owns the tokens
    cu_tokens[e] .. cu_tokens[e+1]; they sit at positions q_start[e] .. q_start[e] + q_len[e] - 1 of their
    request.  Host copies of the per-entry numbers travel along for launch decisions."""
    token_ids: torch.Tensor        # int32 [T]
    positions: torch.Tensor        # int32 [T]
    token_entry: torch.Tensor      # int32 [T]: which entry a token belongs to
    cu_tokens: torch.Tensor        # int32 [entries + 1]
    q_start: torch.Tensor          # int32 [entries]: tokens of the request already in the cache
    logit_rows: torch.Tensor       # int32 [R]: token rows whose logits are wanted
    num_tokens: int
    num_entries: int
    host_q_start: List[int]
    host_q_len: List[int]
    caches: List[object]           # per schedule entry: KVView | StateView | None, or a list of views
    extra: Optional[dict] = None   # whatever a kernel dispatcher wants to remember within the step

    @property
    def max_q_len(self):
        return max(self.host_q_len) if self.host_q_len else 0

    @property
    def max_kv_len(self):
        return max((s + n for s, n in zip(self.host_q_start, self.host_q_len)), default=0)


class DecoderModel:
    """embedding -> scheduled blocks -> final norm on the wanted rows -> head
    (ginfer/model/model.cc:158-165 for the order, :210-220 for the head)."""

    def __init__(self, spec, dtype, device):
        spec.validate()
        self.spec, self.dtype, self.device = spec, dtype, device
        self._positions = {}
        kw = dict(dtype=dtype, device=device)
        self.embedding = registry.lookup("embedding", spec.embedding.kind)(**spec.embedding.params, **kw)
        self.final_norm = registry.lookup("norm", spec.final_norm.kind)(**spec.final_norm.params, **kw)
        self.head = registry.lookup("head", spec.head.kind)(**spec.head.params, **kw)
        self.blocks = []
        for i, ls in enumerate(spec.layers):
            arrangement = registry.lookup("arrangement", ls.arrangement)
            roles = arrangement.roles        # role -> family of parts
            if set(ls.parts) != set(roles):
                raise ValueError("layer %d: arrangement %r has the roles %s, the layer names %s"
                                 % (i, ls.arrangement, sorted(roles), sorted(ls.parts)))
            self.blocks.append(arrangement({role: self._build(roles[role], ls.parts[role]) for role in roles}))
        self.schedule = list(spec.schedule)
        # per run of the schedule: the first norm of the block that runs next, where this run's block can fold it
        # into its own last product and that block takes its input so (a matter of speed only)
        self._fold_into = []
        for i, e in enumerate(self.schedule):
            nxt = self.blocks[self.schedule[i + 1].layer] if i + 1 < len(self.schedule) else None
            takes = getattr(nxt, "takes_folded_input", None)
            norm = takes() if takes is not None else None
            self._fold_into.append(norm if getattr(self.blocks[e.layer], "folds_output", False) else None)

    def _build(self, role, part_spec):
        params = dict(part_spec.params)
        pos = params.get("position")
        if pos is not None and hasattr(pos, "kind"):
            key = pos.key()
            if key not in self._positions:   # layers with the same encoding share its tables
                self._positions[key] = registry.lookup("position", pos.kind)(
                    **pos.params, dtype=self.dtype, device=self.device)
            params["position"] = self._positions[key]
        return registry.lookup(role, part_spec.kind)(**params, dtype=self.dtype, device=self.device)

    # ---- weights
    def _named_parts(self):
        name_of = self.spec.name_of
        out = [(name_of("embedding"), self.embedding), (name_of("final_norm"), self.final_norm),
               (name_of("head"), self.head)]
        for ls, block in zip(self.spec.layers, self.blocks):
            for role, part in block.parts():
                out.append((ls.prefix + "." + ls.name_of(role), part))
        return out

    def weight_specs(self):
        specs = {}
        for prefix, part in self._named_parts():
            for local, ws in part.weight_specs().items():
                specs[prefix + "." + local] = ws
        return specs

    def unread_weights(self):
        """Full names of tensors that a checkpoint may carry although no part reads them."""
        return [prefix + "." + local for prefix, part in self._named_parts()
                for local in getattr(part, "unread_weights", list)()]

    def bind_weights(self, tensors):
        for prefix, part in self._named_parts():
            local = {n: tensors[prefix + "." + n] for n in part.weight_specs()}
            part.bind_weights(local)
        if getattr(self.head, "tied", False):
            self.head.tie(self.embedding.weight)

    def kernel_modules(self):
        mods = []
        for _, part in self._named_parts():
            for m in part.kernel_modules():     # a name, or (name, {macro: value})
                if m not in mods:
                    mods.append(m)
        return mods

    def capturable(self):
        """Whether a step of this model may be recorded into a HIP graph: every part must allow it."""
        return all(getattr(part, "capturable", False) for _, part in self._named_parts())

    def position_parts(self):
        return list(self._positions.values())

    # ---- cache
    def cache_specs(self):
        """Per schedule entry: what its run keeps per request (a spec or a list of specs), or None when it keeps nothing
        or reads another entry's cache."""
        out = []
        for e in self.schedule:
            out.append(None if e.cache_of is not None else self.blocks[e.layer].cache_spec())
        return out

    # ---- forward
    def forward(self, step):
        """Logits float32 [R, V] at `step.logit_rows`."""
        residual = self.embedding.forward(step.token_ids, step)
        delta = None
        for i, e in enumerate(self.schedule):
            cache = step.caches[i]
            if self._fold_into[i] is not None:
                delta = self.blocks[e.layer].forward(residual, delta, step, cache, into_norm=self._fold_into[i])
            else:
                delta = self.blocks[e.layer].forward(residual, delta, step, cache)
        n = self.final_norm.forward(residual, whole(delta, self.final_norm), rows=step.logit_rows)
        return self.head.forward(n)


def build_model(spec, dtype, device):
    return DecoderModel(spec, dtype, device)
