"""The description of a whole model as data.

``ModelPlan.layers`` are the distinct layers (each owns weights); ``ModelPlan.calls`` is the
order in which they run. A call may name a layer that an earlier call already ran (the
weights are used twice, each call keeps a cache of its own) and may read the cache that an
earlier call wrote instead of keeping one (``cache_from``).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Optional, Tuple

from .base import PartSpec


@dataclass(frozen=True)
class TensorLocation:
    """Where a tensor belongs: ``layer`` None for the model-level parts; ``role`` is
    "embedding", "head", "final_norm", "mixer", "ffn" or "norm.<slot>"; ``name`` is the part's
    logical tensor name."""
    layer: Optional[int]
    role: str
    name: str


@dataclass(frozen=True)
class LayerPlan:
    """One layer: the block arrangement and the parts it wires. A layer may go without a mixer or
    without a feed-forward (None); its block arrangement then gets None in that place."""
    block: PartSpec
    mixer: Optional[PartSpec]
    ffn: Optional[PartSpec]
    norms: Tuple[Tuple[str, PartSpec], ...]   # (slot, spec) pairs the block arrangement wires

    def norm_map(self) -> Dict[str, PartSpec]:
        return dict(self.norms)


@dataclass(frozen=True)
class Call:
    layer: int
    cache_from: Optional[int] = None


@dataclass(frozen=True)
class EmbeddingSpec(PartSpec):
    kind = "embedding"
    vocab_size: int = 0
    hidden_size: int = 0
    scale: float = 1.0


@dataclass(frozen=True)
class HeadSpec(PartSpec):
    kind = "linear_head"
    vocab_size: int = 0
    hidden_size: int = 0
    tied: bool = False


@dataclass(frozen=True)
class ModelPlan:
    hidden_size: int
    vocab_size: int
    max_positions: int
    embedding: PartSpec            # EmbeddingSpec, or the spec of another registered embedding
    layers: Tuple[LayerPlan, ...]
    calls: Tuple[Call, ...]
    final_norm: PartSpec
    head: PartSpec                 # HeadSpec, or the spec of another registered head

    def validate(self) -> None:
        if not self.layers:
            raise ValueError("a model plan needs at least one layer")
        for i, c in enumerate(self.calls):
            if not (0 <= c.layer < len(self.layers)):
                raise ValueError(f"call {i} names layer {c.layer}, the plan has {len(self.layers)}")
            if c.cache_from is not None:
                if not (0 <= c.cache_from < i):
                    raise ValueError(f"call {i} reads the cache of call {c.cache_from}, which does not run before it")
                if self.calls[c.cache_from].cache_from is not None:
                    raise ValueError(f"call {i} reads the cache of call {c.cache_from}, which keeps none itself")
