"""A model described as data: which parts make each layer, with which sizes and constants, and in
which order the layers run.  The architecture modules produce these from a typed configuration;
the generic model builder consumes them and knows no architecture.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional


@dataclass(frozen=True)
class PartSpec:
    """One part: `kind` names an entry of the part's registry, `params` are its sizes and constants."""
    kind: str
    params: Dict[str, Any] = field(default_factory=dict)


@dataclass
class LayerSpec:
    """One layer: an arrangement (how norms, mixer and feed-forward are wired around the residual
    stream) and the parts that fill its slots.  `names` maps each slot to the sub-prefix of its
    tensors under `prefix` in a checkpoint."""
    prefix: str
    arrangement: str
    parts: Dict[str, PartSpec]
    names: Dict[str, str]
    residual_scale: float = 1.0


@dataclass(frozen=True)
class LayerRun:
    """One entry of the execution order: run `layer` with cache entry `cache`.

    A layer may appear in several runs (its weights are shared).  Two runs may name the same cache
    entry: the one with `writes_cache` fills it, the others only read it."""
    layer: int
    cache: Optional[int]
    writes_cache: bool = True


@dataclass
class HeadSpec:
    """The output head: a part of kind `kind` built from (vocab_size, hidden_size, scale, **params), whose
    tensors lie under `name` in a checkpoint."""
    name: str = "lm_head"
    scale: float = 1.0
    tie_to_embedding_when_missing: bool = True
    kind: str = "linear"
    params: Dict[str, Any] = field(default_factory=dict)


@dataclass
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden_size: int
    max_positions: int
    embed_name: str
    embed_scale: float
    layers: List[LayerSpec]
    order: List[LayerRun]
    final_norm: PartSpec
    final_norm_name: str
    head: HeadSpec
    eos_token_ids: List[int] = field(default_factory=list)
    # the embedding: a part of kind `embed_kind` built from (vocab_size, hidden_size, scale=embed_scale, **embed_params)
    embed_kind: str = "scaled_lookup"
    embed_params: Dict[str, Any] = field(default_factory=dict)
    # axes of the positions a step carries for every token (1: the place in the sequence alone; a position encoding
    # over several axes, rows and columns of a picture beside the place in the text, reads `batch.position_axes`)
    position_axes: int = 1

    def num_cache_entries(self) -> int:
        ids = [r.cache for r in self.order if r.cache is not None]
        return (max(ids) + 1) if ids else 0

    def validate(self) -> None:
        n = len(self.layers)
        writers: Dict[int, int] = {}
        for i, run in enumerate(self.order):
            if not 0 <= run.layer < n:
                raise ValueError(f"order[{i}] names layer {run.layer}, but there are {n} layers")
            if run.cache is not None and run.writes_cache:
                if run.cache in writers:
                    raise ValueError(f"cache entry {run.cache} is written by order[{writers[run.cache]}] and order[{i}]")
                writers[run.cache] = i
        for i, run in enumerate(self.order):
            if run.cache is not None and not run.writes_cache:
                if run.cache not in writers or writers[run.cache] > i:
                    raise ValueError(f"order[{i}] reads cache entry {run.cache} before any run has written it")
