"""Rotary position encoding in the split-half layout.

For pair ``i`` of a head: ``theta = p * base^(-2i/d)``;
``x'[i] = x[i] cos - x[i+d/2] sin``; ``x'[i+d/2] = x[i] sin + x[i+d/2] cos``
(src/ops/ops.cpp:863-878). The part owns the table of inverse frequencies, held
in float64 so that the angle of any position is exact before cos and sin are
rounded to float32. cos and sin of a step's positions are computed once and
shared by the layers whose encoding has the same parameters; the attention
mixer's fused kernels apply the rotation.
"""
from __future__ import annotations

import torch

from ..ops import kernels
from .base import PositionEncoding, Runtime
from .registry import register_part
from .spec import PartSpec


class RopeSplitHalf(PositionEncoding):
    graph_safe = True
    fused_split_half = True

    def __init__(self, spec: PartSpec, runtime: Runtime):
        super().__init__(spec, runtime)
        self.theta = float(spec.params["theta"])
        self.head_dim = int(spec.params["head_dim"])
        self.rotary_dim = int(spec.params.get("rotary_dim", self.head_dim))
        if self.rotary_dim % 2 != 0 or not 0 < self.rotary_dim <= self.head_dim:
            raise ValueError("rotary_dim must be even and at most head_dim")
        exponents = torch.arange(0, self.rotary_dim, 2, dtype=torch.float64) / self.rotary_dim
        self.inv_freq = (self.theta ** -exponents).to(runtime.device)

    def table(self, ctx) -> torch.Tensor:
        """``[tokens, rotary_dim / 2, 2]`` float32: cos and sin for the step's tokens."""
        key = ("rope_split_half", self.theta, self.rotary_dim)
        if key not in ctx.memo:
            ctx.memo[key] = kernels.rope_table(ctx.positions, self.inv_freq)
        return ctx.memo[key]


register_part("position", "rope_split_half", RopeSplitHalf)
