"""How a layer's parts are arranged around the residual stream.

``pre_norm`` is the reference's block: ``h' = h + Mixer(Norm1(h))``,
``h'' = h' + FFN(Norm2(h'))`` (src/model/model.cpp:851-860). The residual stream
``h`` is float32 and every sum into it is a float32 sum; the sum is fused with
the norm that follows it, so a block hands its last delta on instead of adding
it (the decode path of the reference does the same, src/model/model.cpp:867).
Where a step has few rows, the part before a norm and the part after it can
take the norm between them: the first adds its result to the stream in its last
product's epilogue and multiplies by the norm's weight, the second multiplies
its first product's rows by the norm's factors (``linear.UnscaledRows``).
"""
from __future__ import annotations

from typing import Dict, Mapping, Optional

import torch

from .base import Part, Runtime, TensorDecl
from .linear import Residual, UnscaledRows
from .registry import build_part, register_part
from .spec import LayerSpec


class Block:
    """One layer built from a ``LayerSpec``. ``forward`` returns the delta still to be added to ``h``."""

    def __init__(self, spec: LayerSpec, runtime: Runtime):
        self.spec = spec
        self.mixer_norm = build_part("norm", spec.mixer_norm, runtime)
        self.mixer = build_part("mixer", spec.mixer, runtime)
        if (spec.ffn is None) != (spec.ffn_norm is None):
            raise ValueError("a layer has a feed-forward and its norm, or neither")
        self.ffn_norm = build_part("norm", spec.ffn_norm, runtime) if spec.ffn_norm is not None else None
        self.ffn = build_part("ffn", spec.ffn, runtime) if spec.ffn is not None else None
        self.extra: Dict[str, Part] = {name: build_part(category, part_spec, runtime)
                                       for name, (category, part_spec) in spec.extra.items()}

    def parts(self):
        """Every part of the layer (the cache manager asks ``mixer`` alone for a cache)."""
        own = (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn)
        return tuple(part for part in own if part is not None) + tuple(self.extra.values())

    def tensors(self) -> Dict[str, TensorDecl]:
        decls: Dict[str, TensorDecl] = {}
        for part in self.parts():
            decls.update(part.tensors())
        return decls

    def bind(self, tensors: Mapping[str, torch.Tensor]) -> None:
        for part in self.parts():
            part.bind(tensors)

    def forward(self, h: torch.Tensor, pending, ctx, cache, next_block: Optional["Block"] = None):
        """``pending`` is the delta the block before left to be added, or that block's ``UnscaledRows``: then the
        sum and this block's first norm are done. ``next_block`` is the block that runs after this one."""
        raise NotImplementedError

    def first_norm_after(self, producer, rows: int, h: torch.Tensor) -> Optional[Residual]:
        """What ``producer`` needs to add its delta to ``h`` itself and begin this block's first norm, if the norm,
        the producer and this block's mixer can all do their part for this many rows; else None."""
        return residual_for(producer, self.mixer_norm, self.mixer, rows, h)


def residual_for(producer, norm, consumer, rows: int, h: torch.Tensor) -> Optional[Residual]:
    if not getattr(producer, "fuses_residual", False) or not consumer.takes_unscaled(rows):
        return None
    pieces = norm.weight_then_factor()
    if pieces is None:
        return None
    weight, width, eps = pieces
    return Residual(h, weight, width, eps)


class PreNormBlock(Block):
    def forward(self, h, pending, ctx, cache, next_block=None):
        rows = h.shape[0]
        x = pending if isinstance(pending, UnscaledRows) else self.mixer_norm.forward(h, delta=pending, write_h=True)
        if self.ffn is None:        # no feed-forward: the mixer's delta goes to whatever norm comes next
            residual = next_block.first_norm_after(self.mixer, rows, h) if next_block is not None else None
            return self.mixer.forward(x, ctx, cache, residual=residual) if residual is not None else self.mixer.forward(x, ctx, cache)
        residual = residual_for(self.mixer, self.ffn_norm, self.ffn, rows, h)
        mixed = self.mixer.forward(x, ctx, cache, residual=residual) if residual is not None else self.mixer.forward(x, ctx, cache)
        x = mixed if isinstance(mixed, UnscaledRows) else self.ffn_norm.forward(h, delta=mixed, write_h=True)
        residual = next_block.first_norm_after(self.ffn, rows, h) if next_block is not None else None
        return self.ffn.forward(x, ctx, residual=residual) if residual is not None else self.ffn.forward(x, ctx)


_ARRANGEMENTS = {"pre_norm": PreNormBlock}


def register_arrangement(name: str, block_class, replace: bool = False) -> None:
    if name in _ARRANGEMENTS and not replace:
        raise ValueError(f"arrangement {name!r} is already registered")
    _ARRANGEMENTS[name] = block_class


def build_block(spec: LayerSpec, runtime: Runtime) -> Block:
    if spec.arrangement not in _ARRANGEMENTS:
        raise KeyError(f"unknown arrangement {spec.arrangement!r}; registered: {', '.join(sorted(_ARRANGEMENTS))}")
    return _ARRANGEMENTS[spec.arrangement](spec, runtime)
