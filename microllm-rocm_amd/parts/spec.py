"""Data that describes a model: which parts each layer is made of, and in which order layers run.

A configuration is turned into a ``ModelSpec`` by its architecture's builder;
from then on nothing looks at the configuration again. Every part is named by
a ``PartSpec``: its kind (looked up in the part registries), its sizes and
constants, and the file names of the tensors it needs.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Mapping, Optional, Tuple


@dataclass(frozen=True)
class PartSpec:
    kind: str
    params: Mapping[str, Any] = field(default_factory=dict)
    names: Mapping[str, str] = field(default_factory=dict)  # role in the part -> tensor name in the files

    def param(self, key: str, default: Any = None) -> Any:
        return self.params.get(key, default)


@dataclass(frozen=True)
class LayerSpec:
    """One layer: a mixer and, usually, a feed-forward, each behind its norm, in an arrangement.

    A layer without a feed-forward leaves ``ffn`` and ``ffn_norm`` out. What an arrangement needs beyond these
    (a norm after the mixer, norms of queries and keys outside the mixer, a second mixer) goes into ``extra``:
    a name of the arrangement's choice -> (category, spec); the block builds each and finds it in
    ``Block.extra[name]``."""
    arrangement: str  # e.g. "pre_norm"
    mixer_norm: PartSpec
    mixer: PartSpec
    ffn_norm: Optional[PartSpec] = None
    ffn: Optional[PartSpec] = None
    extra: Mapping[str, Tuple[str, PartSpec]] = field(default_factory=dict)


@dataclass(frozen=True)
class RunEntry:
    """One element of the run order.

    ``layer`` indexes ``ModelSpec.layers`` and may appear in several entries
    (shared weights; each entry has a cache of its own). ``reads_cache_of`` names
    an earlier entry whose cache this entry's mixer reads instead of owning one.
    """
    layer: int
    reads_cache_of: Optional[int] = None


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden_size: int
    max_positions: int
    embedding: PartSpec
    layers: Tuple[LayerSpec, ...]
    order: Tuple[RunEntry, ...]
    final_norm: PartSpec
    head: PartSpec

    def validate(self) -> None:
        if not self.layers or not self.order:
            raise ValueError("a model needs at least one layer and one run entry")
        for index, entry in enumerate(self.order):
            if not 0 <= entry.layer < len(self.layers):
                raise ValueError(f"run entry {index} names layer {entry.layer}, which does not exist")
            if entry.reads_cache_of is not None:
                if not 0 <= entry.reads_cache_of < index:
                    raise ValueError(f"run entry {index} must read the cache of an earlier entry")
                if self.order[entry.reads_cache_of].reads_cache_of is not None:
                    raise ValueError(f"run entry {index} reads the cache of an entry that owns none")


def in_order(count: int) -> Tuple[RunEntry, ...]:
    """The usual order: every layer once, first to last."""
    return tuple(RunEntry(layer=index) for index in range(count))
