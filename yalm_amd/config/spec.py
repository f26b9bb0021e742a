"""The description of a model as data: which parts make up each layer, with
which sizes and constants, and in which order the layers run.  A typed
configuration of an architecture (config/llama.py) produces a ModelSpec; the
model builder (engine/model.py) knows only ModelSpecs and the part registry.
"""
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional


@dataclass(frozen=True)
class PartSpec:
    """One part: the name it is registered under and its parameters.  `prefix` is
    the part's place in the tensor names of a model folder, relative to its layer."""
    kind: str
    params: Dict[str, Any] = field(default_factory=dict)
    prefix: str = ""

    def __hash__(self):
        return hash((self.kind, self.prefix, repr(sorted(self.params.items(), key=lambda kv: kv[0]))))


class LayerSpec:
    """A layer: the arrangement (block kind), the members it arranges, by the names that block
    kind knows, and the layer's place in the tensor names.  The reference's arrangement
    ("prenorm_residual") has the members mixer, feed_forward, mixer_norm and feed_forward_norm;
    another block kind has the members it needs (one norm in front of a mixer and a feed-forward
    that run side by side, no feed-forward at all, ...) and reads only those.  Members are given by
    name, `LayerSpec("prenorm_residual", prefix="model.layers.3.", mixer=..., ...)`, or as a
    dictionary `parts`, and read back as attributes or with `part(name)`.  The member called
    `mixer`, if there is one, is the one whose cache line the schedule speaks of."""

    def __init__(self, block, parts=None, prefix="", **members):
        merged = dict(parts or {})
        merged.update(members)
        for name, spec in merged.items():
            if not isinstance(spec, PartSpec):
                raise TypeError("member %r of a layer is a %s, not a PartSpec" % (name, type(spec).__name__))
        self.__dict__["block"] = block                 # e.g. "prenorm_residual"
        self.__dict__["parts"] = merged
        self.__dict__["prefix"] = prefix               # e.g. "model.layers.3."

    def part(self, name, default=None):
        return self.parts.get(name, default)

    def __getattr__(self, name):
        parts = self.__dict__.get("parts")
        if parts is not None and name in parts:
            return parts[name]
        raise AttributeError("this layer (%s) has no member %r" % (self.__dict__.get("block"), name))

    def __setattr__(self, name, value):
        raise AttributeError("a LayerSpec is not changed after it is made")

    def __eq__(self, other):
        return isinstance(other, LayerSpec) and (self.block, self.parts, self.prefix) == (other.block, other.parts, other.prefix)

    def __repr__(self):
        return "LayerSpec(%r, %r, prefix=%r)" % (self.block, self.parts, self.prefix)


@dataclass(frozen=True)
class ScheduleEntry:
    """One run of a layer.  `cache` names the cache line the mixer uses: by default
    the entry's own index in the schedule; an entry with `writes_cache=False`
    reads the line another entry wrote (it must come later in the schedule)."""
    layer: int
    cache: int
    writes_cache: bool = True


@dataclass
class ModelSpec:
    architecture: str
    dim: int
    vocab_size: int
    max_positions: int
    embedding: PartSpec
    layers: List[LayerSpec]
    final_norm: PartSpec
    head: PartSpec
    schedule: Optional[List[ScheduleEntry]] = None
    bos_token_id: Optional[int] = None
    eos_token_ids: List[int] = field(default_factory=list)

    def __post_init__(self):
        if self.schedule is None:
            self.schedule = [ScheduleEntry(layer=i, cache=i) for i in range(len(self.layers))]
        self.validate()

    def validate(self):
        if self.dim <= 0 or self.vocab_size <= 0 or self.max_positions <= 0:
            raise ValueError("dim, vocab_size and max_positions must be positive")
        writers = {}
        for i, e in enumerate(self.schedule):
            if not 0 <= e.layer < len(self.layers):
                raise ValueError("schedule entry %d names layer %d of %d" % (i, e.layer, len(self.layers)))
            if e.writes_cache:
                if e.cache in writers:
                    raise ValueError("cache line %d is written by schedule entries %d and %d"
                                     % (e.cache, writers[e.cache], i))
                writers[e.cache] = i
            elif e.cache not in writers:
                raise ValueError("schedule entry %d reads cache line %d before any entry wrote it" % (i, e.cache))
            else:
                a = self.layers[self.schedule[writers[e.cache]].layer].part("mixer")
                b = self.layers[e.layer].part("mixer")
                if a is None or b is None or a.kind != b.kind:
                    raise ValueError("schedule entry %d (%s) cannot read the cache line of a %s"
                                     % (i, getattr(b, "kind", "no mixer"), getattr(a, "kind", "layer without a mixer")))
