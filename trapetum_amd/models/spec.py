"""A model as data: which parts stand in which layer, under which tensor names, run in which order.

An architecture's `build_spec(config)` returns a ModelSpec; the engine builds
the parts from it through the registry.  Parts name their tensors locally
("q_proj.weight"); the spec gives each part's place in the checkpoint as a
prefix ("model.layers.3.self_attn."), so no part knows which model it is in.
"""
import dataclasses
from typing import Dict, List, Optional, Tuple

PartRef = Tuple[str, dict]          # (registered name, constructor parameters)


@dataclasses.dataclass
class TensorSpec:
    """One tensor a part needs: its shape and how a random model fills it."""
    shape: tuple
    init: str = "matrix"            # "matrix", "norm", "embedding": which sigma; "zeros"; "ones"
    dtype: str = "float"            # "float": kept as stored (bf16, or fp32 if stored so); "int": int32 table


@dataclasses.dataclass
class LayerSpec:
    """One layer: the arrangement (block) and the parts it arranges."""
    block: PartRef
    mixer: PartRef
    feed_forward: PartRef
    norm: PartRef                    # built once for every norm site the block declares ...
    prefixes: Dict[str, str]         # site name of the block -> checkpoint prefix
    norms: Optional[Dict[str, PartRef]] = None    # ... unless a site is named here with a norm of its own

    def norm_of(self, site):
        return (self.norms or {}).get(site, self.norm)


@dataclasses.dataclass
class ScheduleEntry:
    """One run of a layer.  `cache_of` names an earlier entry whose cache this run reads
    instead of keeping one of its own."""
    layer: int
    cache_of: Optional[int] = None


@dataclasses.dataclass
class ModelSpec:
    architecture: str
    hidden_size: int
    vocab_size: int
    embedding: PartRef
    embedding_prefix: str
    layers: List[LayerSpec]
    schedule: List[ScheduleEntry]
    final_norm: PartRef
    final_norm_prefix: str
    head: PartRef
    head_prefix: str                 # the embedding's prefix when the head is tied to it
    stop_ids: tuple = ()

    def validate(self):
        for i, e in enumerate(self.schedule):
            if not 0 <= e.layer < len(self.layers):
                raise ValueError(f"schedule entry {i} names layer {e.layer}; the model has {len(self.layers)}")
            if e.cache_of is not None:
                if not 0 <= e.cache_of < i:
                    raise ValueError(f"schedule entry {i} reads the cache of entry {e.cache_of}, which does not run before it")
                if self.schedule[e.cache_of].cache_of is not None:
                    raise ValueError(f"schedule entry {i} reads the cache of entry {e.cache_of}, which has none of its own")
