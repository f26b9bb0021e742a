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


@dataclass(frozen=True)
class LayerSpec:
    """A layer: the arrangement (block kind) and the parts it arranges."""
    block: str                      # e.g. "prenorm_residual"
    mixer: PartSpec
    feed_forward: PartSpec
    mixer_norm: PartSpec
    feed_forward_norm: PartSpec
    prefix: str                     # e.g. "model.layers.3."


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
                a = self.layers[self.schedule[writers[e.cache]].layer].mixer
                b = self.layers[e.layer].mixer
                if a.kind != b.kind:
                    raise ValueError("schedule entry %d (%s) cannot read the cache line of a %s" % (i, b.kind, a.kind))
