"""What a model is made of, as data.

An architecture's typed configuration turns into a `ModelSpec`: one `LayerSpec` per layer, each
naming its parts (mixer, feed-forward, norms, whatever roles its arrangement has) by registry kind with
every size and constant as a parameter, and a `schedule` that lists the order in which layers run.  The builder in
`ginfer_amd.parts.model` reads nothing but this; no part ever sees the architecture's name.
"""
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional


@dataclass
class PartSpec:
    """A part chosen by registry kind, with its sizes and constants."""
    kind: str
    params: Dict[str, Any] = field(default_factory=dict)

    def key(self):
        return (self.kind, tuple(sorted((k, _freeze(v)) for k, v in self.params.items())))


def _freeze(v):
    if isinstance(v, PartSpec):
        return v.key()
    if isinstance(v, dict):
        return tuple(sorted((k, _freeze(x)) for k, x in v.items()))
    if isinstance(v, (list, tuple)):
        return tuple(_freeze(x) for x in v)
    return v


@dataclass
class LayerSpec:
    """One block: its parts by role, how they are arranged around the residual stream, and the prefix of its tensors.
    Which roles a block has is the arrangement's matter (`roles` of the registered arrangement class: role -> family of
    parts, e.g. {"mixer": "mixer", "feed_forward": "feed_forward", "mixer_norm": "norm", ...}); a layer names exactly
    those.  `names` gives each role the prefix of its tensors inside the layer, as the checkpoint spells it (a role
    that is not listed is spelt as the role itself)."""
    prefix: str
    parts: Dict[str, PartSpec]
    arrangement: str = "prenorm"
    names: Dict[str, str] = field(default_factory=dict)

    def name_of(self, role):
        return self.names.get(role, role)


def prenorm_layer(prefix, mixer, feed_forward, mixer_norm, feed_forward_norm, names=None):
    """The usual block of four parts (norm, mixer, norm, feed-forward).  names: role -> the prefix of its tensors inside
    the layer as the architecture's checkpoints spell it (the architecture's configuration knows; a role that is not
    listed is spelt as the role itself)."""
    return LayerSpec(prefix=prefix, parts=dict(mixer=mixer, feed_forward=feed_forward, mixer_norm=mixer_norm,
                                               feed_forward_norm=feed_forward_norm),
                     arrangement="prenorm", names=dict(names or {}))


@dataclass
class ScheduleEntry:
    """One run of a layer.  Every entry owns a cache of its own (so a layer named twice keeps two),
    unless `cache_of` names an earlier entry of the schedule whose cache this run reads."""
    layer: int
    cache_of: Optional[int] = None


@dataclass
class ModelSpec:
    hidden_size: int
    vocab_size: int
    layers: List[LayerSpec]
    schedule: List[ScheduleEntry]
    embedding: PartSpec
    final_norm: PartSpec
    head: PartSpec
    max_positions: int
    eos_token_ids: List[int]
    # tensor-name prefixes of the parts outside the layers, as the architecture's checkpoints spell them (a part that is
    # not listed is spelt as its role: "embedding", "final_norm", "head")
    names: Dict[str, str] = field(default_factory=dict)

    def name_of(self, role):
        return self.names.get(role, role)

    def validate(self):
        for i, e in enumerate(self.schedule):
            if not 0 <= e.layer < len(self.layers):
                raise ValueError("schedule entry %d names layer %d of %d" % (i, e.layer, len(self.layers)))
            if e.cache_of is not None:
                if not 0 <= e.cache_of < i:
                    raise ValueError("schedule entry %d reads the cache of entry %s, which does not "
                                     "run before it" % (i, e.cache_of))
                if self.schedule[e.cache_of].cache_of is not None:
                    raise ValueError("schedule entry %d reads the cache of entry %d, which owns none"
                                     % (i, e.cache_of))
