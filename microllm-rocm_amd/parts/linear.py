"""A matrix product ``x @ W.T`` with the weight kept in the file's ``[out, in]`` layout.

The reference stores ``[in, out]`` and transposes every linear at load
(src/model/model.cpp:285, 1939-1973); keeping ``[out, in]`` removes that pass and
lets several weights that share an input be stacked along ``out``.
"""
from __future__ import annotations

from typing import Optional

import torch

from ..ops import kernels


def linear(x: torch.Tensor, weight: torch.Tensor, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """``x @ weight.T`` with float32 accumulation; the result has ``out_dtype`` (default: x's)."""
    out_dtype = out_dtype or x.dtype
    if weight.dtype == torch.float32:
        # True 32-bit product, also for a 32-bit weight inside a bfloat16 engine.
        a = x if x.dtype == torch.float32 else x.to(torch.float32)
        y = kernels.gemm_f32(a, weight)
        return y if out_dtype == torch.float32 else y.to(out_dtype)
    if x.dtype != weight.dtype:
        raise TypeError(f"cannot multiply {x.dtype} activations with a {weight.dtype} weight")
    return kernels.gemm_bf16(x, weight, out_dtype)
