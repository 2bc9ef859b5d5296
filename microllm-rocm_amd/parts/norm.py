"""RMSNorm over the float32 residual stream.

``y = x * (1 / sqrt(mean(x^2) + eps)) * w`` with eps inside the root and the
weight multiplied last (src/ops/ops.cpp:687-698); fused with the residual sum as
the reference's ``add_rms_norm`` is (src/ops/hip/basic_kernels.hip:393-418).
"""
from __future__ import annotations

from typing import Dict, Mapping, Optional

import torch

from ..ops import kernels
from .base import Norm, Runtime, TensorDecl, VECTOR
from .registry import register_part
from .spec import PartSpec


class RMSNorm(Norm):
    graph_safe = True
    def __init__(self, spec: PartSpec, runtime: Runtime):
        super().__init__(spec, runtime)
        self.size = int(spec.params["size"])
        self.eps = float(spec.params["eps"])
        self.weight: Optional[torch.Tensor] = None

    def tensors(self) -> Dict[str, TensorDecl]:
        return {self.name("weight"): TensorDecl((self.size,), VECTOR)}

    def bind(self, tensors: Mapping[str, torch.Tensor]) -> None:
        self.weight = tensors[self.name("weight")]

    def weight_then_factor(self):
        return (self.weight, self.size, self.eps) if self.weight is not None and self.weight.dtype == torch.float32 else None

    def forward(self, h, delta=None, write_h=True, rows=None):
        return kernels.rms_norm(h, self.weight, self.eps, self.runtime.dtype, delta=delta, rows=rows,
                                write_h=write_h and delta is not None and rows is None)


register_part("norm", "rms_norm", RMSNorm)
