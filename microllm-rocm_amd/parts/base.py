"""What every part is: sizes and constants in, tensor declarations out, one forward.

A part is built from a ``PartSpec`` and a ``Runtime`` and knows nothing of the
model it sits in: its sizes, constants and the names of its tensors all come
with the spec. Categories are ``norm``, ``position``, ``mixer``, ``ffn``,
``block``, ``embedding`` and ``head``; each has a registry in ``parts.registry``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Mapping, Optional, Sequence, Tuple, Union

import torch

from ..cache.needs import CacheNeed, PagedKVNeed, StateNeed
from .spec import PartSpec

MATRIX = "matrix"   # a float matrix or table: float32 stays float32, bfloat16 stays bfloat16 in a bfloat16 engine
VECTOR = "vector"   # a float vector read by kernels as float32 (norm weights, biases)
INT_TABLE = "int_table"  # integers, held as int32


@dataclass(frozen=True)
class TensorDecl:
    shape: Tuple[int, ...]
    kind: str = MATRIX


@dataclass(frozen=True)
class Runtime:
    """What a part needs of the engine: the element type of activations and pages, the device, and whether a
    bfloat16 weight keeps its copy as stored beside the packed one (False: one copy, where memory is short;
    steps with many rows then go through the streaming products 64 rows at a time)."""
    dtype: torch.dtype
    device: torch.device
    keep_plain_weights: bool = True


class Part:
    category = "part"
    # True for a part whose forward launches the same kernels on the same addresses whatever the step's
    # contents, reads the step's metadata on the device only, and may run twice without changing the
    # result: the engine replays decode steps from HIP graphs only if every part of the model says so.
    graph_safe = False

    def __init__(self, spec: PartSpec, runtime: Runtime):
        self.spec = spec
        self.runtime = runtime

    def tensors(self) -> Dict[str, TensorDecl]:
        """File name of every tensor this part needs, with its shape and kind."""
        return {}

    def bind(self, tensors: Mapping[str, torch.Tensor]) -> None:
        """Take the loaded tensors (by file name); called once, before the first forward."""

    def sub_parts(self) -> Sequence["Part"]:
        """Parts that this part built for itself (an attention's position encoding): the model asks, so that it
        knows every part it runs without knowing how any is put together."""
        return ()

    def step_planner(self):
        """A ``StepPlanner`` (engine/batch.py) if this part's kernels need metadata of their own for every step
        (tiles of queries, work lists), made on the host from the batch's shape and copied to the device with
        the step's other metadata; None otherwise. ``ctx.plan_of(planner)`` gives the plan in ``forward``."""
        return None

    def flops(self, tokens: int) -> float:
        """Floating-point operations of this part over one request's prompt of ``tokens`` ids (2 per multiply-add);
        by default those of its matrix products: its attributes that are a ``linear.Weight``."""
        from .linear import Weight      # (linear imports nothing of this module)
        return sum(2.0 * value.out_features * value.in_features * tokens for value in vars(self).values()
                   if isinstance(value, Weight))

    def name(self, role: str) -> str:
        try:
            return self.spec.names[role]
        except KeyError:
            raise KeyError(f"{type(self).__name__} needs a tensor name for {role!r}") from None


class Mixer(Part):
    """Mixes information between the positions of one request (attention, or a layer with state)."""
    category = "mixer"
    fuses_residual = False

    def takes_unscaled(self, rows: int) -> bool:
        return False

    def cache_need(self) -> Optional[CacheNeed]:
        """What this mixer keeps between steps (``cache.needs``): ``PagedKVNeed``, ``StateNeed``, a need class of
        its own, or None."""
        return None

    def forward(self, x: torch.Tensor, ctx, cache) -> torch.Tensor:
        """``[tokens, hidden]`` -> the delta for the residual stream: ``[tokens, hidden]``, or float32 partial
        sums ``[parts, tokens, hidden]`` that the next norm adds in order.

        A part with ``fuses_residual`` also takes ``residual=`` (a ``linear.Residual``, or None) and may then add
        its delta to the stream itself and return the next norm's result as ``linear.UnscaledRows``; a part whose
        ``takes_unscaled(rows)`` says so takes such rows as ``x``. A block only uses either where both sides agree."""
        raise NotImplementedError


class FeedForward(Part):
    category = "ffn"
    fuses_residual = False

    def takes_unscaled(self, rows: int) -> bool:
        return False

    def forward(self, x: torch.Tensor, ctx) -> torch.Tensor:
        """``[tokens, hidden]`` -> the delta for the residual stream, as a mixer's."""
        raise NotImplementedError


class Norm(Part):
    category = "norm"

    def weight_then_factor(self):
        """``(weight, width, eps)`` if the norm is ``x * weight * (1 / sqrt(mean(x^2) + eps))``, so that a product
        before it can multiply by the weight and the product after it by the rows' factors; else None."""
        return None

    def forward(self, h: torch.Tensor, delta: Optional[torch.Tensor] = None, write_h: bool = True,
                rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Normalise ``h + delta`` (float32 residual stream); with ``write_h`` the sum replaces ``h``.

        ``delta`` is ``[tokens, hidden]`` or float32 partial sums ``[parts, tokens, hidden]``, added in order first."""
        raise NotImplementedError


class PositionEncoding(Part):
    category = "position"
    fused_split_half = False  # True: the mixer's fused kernels rotate by the split-half rule with ``table(ctx)``'s cos and sin

    def apply(self, qkv: torch.Tensor, positions: torch.Tensor, heads: int, kv_heads: int,
              head_dim: int) -> torch.Tensor:
        """Encode positions into the q and k parts of fused projections ``[tokens, (heads + 2 kv) * hd]``."""
        raise NotImplementedError
