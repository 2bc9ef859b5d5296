from . import attention, block, feedforward, model, norm, position  # noqa: F401  (register the built-in kinds)
from .base import (CacheNeed, FeedForward, INT_TABLE, MATRIX, Mixer, Norm, PagedKVNeed, Part, PositionEncoding, Runtime,
                   StateNeed, TensorDecl, VECTOR)
from .block import Block, PreNormBlock, build_block, register_arrangement
from .model import Model
from .registry import build_part, register_part, registered_kinds, unregister_part
from .spec import LayerSpec, ModelSpec, PartSpec, RunEntry, in_order

__all__ = ["CacheNeed", "FeedForward", "INT_TABLE", "MATRIX", "Mixer", "Norm", "PagedKVNeed", "Part", "PositionEncoding",
           "Runtime", "StateNeed", "TensorDecl", "VECTOR", "Block", "PreNormBlock", "build_block",
           "register_arrangement", "Model", "build_part", "register_part", "registered_kinds",
           "unregister_part", "LayerSpec", "ModelSpec", "PartSpec", "RunEntry", "in_order"]
