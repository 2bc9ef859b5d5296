"""The SwiGLU feed-forward: ``down(silu(gate(x)) * up(x))``, no biases.

``z = g * sigmoid(g) * u`` with the sigmoid evaluated branch-stably
(src/ops/ops.cpp:72-76, 779-783; src/model/model.cpp:787-789). Gate and up are
stacked into one weight at bind time so the input is read once.
"""
from __future__ import annotations

from typing import Dict, Mapping, Optional

import torch

from ..ops import kernels
from .base import FeedForward, MATRIX, Runtime, TensorDecl
from .linear import Weight, linear, linear_into_stream, takes_unscaled
from .registry import register_part
from .spec import PartSpec


class SwiGLU(FeedForward):
    graph_safe = True
    fuses_residual = True
    def __init__(self, spec: PartSpec, runtime: Runtime):
        super().__init__(spec, runtime)
        self.hidden = int(spec.params["hidden_size"])
        self.intermediate = int(spec.params["intermediate_size"])
        self.gate_up_weight: Optional[torch.Tensor] = None
        self.down_weight: Optional[torch.Tensor] = None

    def tensors(self) -> Dict[str, TensorDecl]:
        return {
            self.name("gate_proj.weight"): TensorDecl((self.intermediate, self.hidden), MATRIX),
            self.name("up_proj.weight"): TensorDecl((self.intermediate, self.hidden), MATRIX),
            self.name("down_proj.weight"): TensorDecl((self.hidden, self.intermediate), MATRIX),
        }

    def bind(self, tensors: Mapping[str, torch.Tensor]) -> None:
        gate = tensors[self.name("gate_proj.weight")]
        up = tensors[self.name("up_proj.weight")]
        if gate.dtype != up.dtype:
            raise TypeError("the gate and up weights of one layer must share a dtype to be stacked")
        self.gate_up_weight = Weight(torch.cat([gate, up], dim=0).contiguous(), gated=True, keep_plain=self.runtime.keep_plain_weights)
        del gate, up
        self.down_weight = Weight(tensors[self.name("down_proj.weight")], keep_plain=self.runtime.keep_plain_weights)

    def takes_unscaled(self, rows: int) -> bool:
        return takes_unscaled(self.gate_up_weight, rows)

    def forward(self, x, ctx, residual=None):
        z = linear(x, self.gate_up_weight, gated=True)
        if residual is not None:
            begun = linear_into_stream(z, self.down_weight, residual)
            if begun is not None:
                return begun
        return linear(z, self.down_weight, out_dtype=torch.float32, partials=True)


register_part("ffn", "swiglu", SwiGLU)
