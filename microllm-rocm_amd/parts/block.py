"""How a layer's parts are arranged around the residual stream.

``pre_norm`` is the reference's block: ``h' = h + Mixer(Norm1(h))``,
``h'' = h' + FFN(Norm2(h'))`` (src/model/model.cpp:851-860). The residual stream
``h`` is float32 and every sum into it is a float32 sum; the sum is fused with
the norm that follows it, so a block hands its last delta on instead of adding
it (the decode path of the reference does the same, src/model/model.cpp:867).
"""
from __future__ import annotations

from typing import Dict, Mapping, Optional

import torch

from .base import Part, Runtime, TensorDecl
from .registry import build_part, register_part
from .spec import LayerSpec


class Block:
    """One layer built from a ``LayerSpec``. ``forward`` returns the delta still to be added to ``h``."""

    def __init__(self, spec: LayerSpec, runtime: Runtime):
        self.spec = spec
        self.mixer_norm = build_part("norm", spec.mixer_norm, runtime)
        self.mixer = build_part("mixer", spec.mixer, runtime)
        self.ffn_norm = build_part("norm", spec.ffn_norm, runtime)
        self.ffn = build_part("ffn", spec.ffn, runtime)

    def parts(self):
        return (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn)

    def tensors(self) -> Dict[str, TensorDecl]:
        decls: Dict[str, TensorDecl] = {}
        for part in self.parts():
            decls.update(part.tensors())
        return decls

    def bind(self, tensors: Mapping[str, torch.Tensor]) -> None:
        for part in self.parts():
            part.bind(tensors)

    def forward(self, h: torch.Tensor, pending: Optional[torch.Tensor], ctx, cache) -> torch.Tensor:
        raise NotImplementedError


class PreNormBlock(Block):
    def forward(self, h, pending, ctx, cache):
        x = self.mixer_norm.forward(h, delta=pending, write_h=True)
        mixed = self.mixer.forward(x, ctx, cache)
        x = self.ffn_norm.forward(h, delta=mixed, write_h=True)
        return self.ffn.forward(x, ctx)


_ARRANGEMENTS = {"pre_norm": PreNormBlock}


def register_arrangement(name: str, block_class, replace: bool = False) -> None:
    if name in _ARRANGEMENTS and not replace:
        raise ValueError(f"arrangement {name!r} is already registered")
    _ARRANGEMENTS[name] = block_class


def build_block(spec: LayerSpec, runtime: Runtime) -> Block:
    if spec.arrangement not in _ARRANGEMENTS:
        raise KeyError(f"unknown arrangement {spec.arrangement!r}; registered: {', '.join(sorted(_ARRANGEMENTS))}")
    return _ARRANGEMENTS[spec.arrangement](spec, runtime)
