"""A matrix product ``x @ W.T`` with the weight kept in the file's ``[out, in]`` layout.

The reference stores ``[in, out]`` and transposes every linear at load
(src/model/model.cpp:285, 1939-1973); keeping ``[out, in]`` removes that pass and
lets several weights that share an input be stacked along ``out``. A bfloat16
weight is held twice on the GPU: as stored, for the library product that steps
with many rows use, and packed in the order the MFMA consumes it, for the two
kernels that stream it once when a step has few rows (decoding): one for up to
16 rows, one that shares the activations between waves for up to 64.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Union

import torch

from ..ops import kernels


class Weight:
    """A linear's weight ``[out, in]`` and, for bfloat16, its packed copy."""

    def __init__(self, tensor: torch.Tensor, gated: bool = False, pack: bool = True,
                 row_order: Optional[torch.Tensor] = None, keep_plain: bool = True):
        self.tensor: Optional[torch.Tensor] = tensor
        self.dtype = tensor.dtype
        self.out_features, self.in_features = tensor.shape
        self.gated = gated   # rows are [gate; up]: the packed copy interleaves them for the fused epilogue
        self.row_order = row_order   # the packed copy's rows in another order: its products' columns come in that order
        self.packed: Optional[torch.Tensor] = None
        if pack and tensor.is_cuda and tensor.dtype == torch.bfloat16 and self.in_features % 8 == 0:
            self.packed = kernels.pack_weight(tensor, interleave_halves=gated, row_order=row_order)
            if not keep_plain:
                self.tensor = None   # the packed copy serves every number of rows


MAX_FACTOR_WIDTH = 8192   # the widest norm whose rows' factors the streaming product applies (its sums sit in LDS)
SKINNY_ROWS = 16        # up to this many rows gemm_skinny beats the library on MI355X for every weight
MEDIUM_ROWS = 64        # and up to this many gemm_medium does, except for
MEDIUM_WIDE_TILES = 2048   # weights with this many tiles of 16 rows or more (gate/up, the head), where the
MEDIUM_WIDE_ROWS = 40      # library is as fast from about this many rows on
MEDIUM_GATED_ROWS = 48     # a gated product (silu(gate) * up in the epilogue) is gemm_medium's up to this many rows: in the
                           # decode step against the tuned library product and the SiLU kernel, 7B sizes +2.5 % at 17 to 32
                           # rows, +1 % at 48, -0.6 % at 56 and 64; 0.5B sizes +9 % at 17, +7 % at 32, the same at 64


@dataclass
class UnscaledRows:
    """A norm's result but for the rows' factors: ``values`` is ``(h * norm weight)`` rounded to bfloat16, and a
    product that takes it multiplies its own rows by ``scale``'s factors (the product is linear in them).
    ``linear_into_stream`` makes these; ``linear`` takes them where ``takes_unscaled`` says so."""
    values: torch.Tensor
    scale: kernels.RowScale

    @property
    def shape(self):
        return self.values.shape

    @property
    def dtype(self):
        return self.values.dtype


@dataclass
class Residual:
    """What the last product of a mixer or feed-forward needs to add its result to the residual stream itself
    and begin the norm that follows: the stream and that norm's weight, width and eps."""
    h: torch.Tensor
    norm_weight: torch.Tensor
    width: int
    eps: float


def takes_unscaled(weight: "Weight", rows: int) -> bool:
    """Whether ``linear`` (and the q/k/v product) can apply rows' factors for this weight and this many rows."""
    return weight.packed is not None and rows <= SKINNY_ROWS


def linear_into_stream(x: torch.Tensor, weight: "Weight", residual: Residual) -> Optional[UnscaledRows]:
    """``residual.h += x @ W.T`` and the next norm begun, in the product's epilogue; None where that cannot be
    done (then nothing was changed and the caller returns its delta as usual)."""
    if not isinstance(x, torch.Tensor) or x.dtype != torch.bfloat16 or not takes_unscaled(weight, x.shape[0]):
        return None
    if weight.row_order is not None or residual.norm_weight.dtype != torch.float32 or residual.width > MAX_FACTOR_WIDTH:
        return None
    values, scale = kernels.gemm_skinny_residual(x, weight.packed, residual.h, residual.norm_weight, residual.width, residual.eps)
    return UnscaledRows(values, scale)


def takes_packed(weight: "Weight", rows: int, gated: bool = False) -> bool:
    """Whether ``linear`` multiplies this many rows with the packed copy (whose rows may be in ``row_order``)."""
    if weight.packed is None:
        return False
    if rows <= SKINNY_ROWS or weight.tensor is None:
        return True
    if gated:
        return rows <= MEDIUM_GATED_ROWS
    wide = -(-weight.out_features // 16) >= MEDIUM_WIDE_TILES
    return rows <= (MEDIUM_WIDE_ROWS if wide else MEDIUM_ROWS)


def linear(x: Union[torch.Tensor, UnscaledRows], weight, out_dtype: Optional[torch.dtype] = None, gated: bool = False,
           partials: bool = False) -> torch.Tensor:
    """``x @ W.T`` with float32 accumulation; the result has ``out_dtype`` (default: x's).

    With ``gated`` the weight's rows are [gate; up] and the result is ``silu(gate) * up`` of half the
    width, in x's dtype. With ``partials`` a float32 result may come as ``[parts, rows, out]``: sums over
    ranges of ``in`` that the caller adds in order (the norms and ``qkv_rope_store`` do). For a weight with a
    ``row_order`` the columns of the result are in that order whenever ``takes_packed`` says so.
    """
    if isinstance(weight, torch.Tensor):
        weight = Weight(weight, pack=False)
    out_dtype = out_dtype or x.dtype
    scale = None
    if isinstance(x, UnscaledRows):
        if not takes_unscaled(weight, x.shape[0]) or x.dtype != weight.dtype:
            raise TypeError("this product cannot apply the rows' factors; see takes_unscaled")
        x, scale = x.values, x.scale
    w = weight.tensor
    if weight.dtype == torch.float32:
        # True 32-bit product, also for a 32-bit weight inside a bfloat16 engine.
        a = x if x.dtype == torch.float32 else x.to(torch.float32)
        y = kernels.gemm_f32(a, w, partials=partials and not gated and out_dtype == torch.float32)
        if gated:
            return kernels.silu_mul(y if x.dtype == torch.float32 else y.to(x.dtype))
        return y if out_dtype == torch.float32 else y.to(out_dtype)
    if x.dtype != weight.dtype:
        raise TypeError(f"cannot multiply {x.dtype} activations with a {weight.dtype} weight")
    rows = x.shape[0]
    if weight.packed is not None and rows <= SKINNY_ROWS:
        if gated:
            return kernels.gemm_skinny(x, weight.packed, weight.out_features, "gated", scale=scale)
        return kernels.gemm_skinny(x, weight.packed, weight.out_features, "bf16" if out_dtype == torch.bfloat16 else "f32",
                                   scale=scale)
    if w is None and rows > MEDIUM_ROWS:
        # Only the packed copy is kept: many rows go through this package's tiled product, or, where the
        # reduction is no multiple of 32, through the product for 64 rows, a piece at a time.
        epilogue = "gated" if gated else ("f32" if out_dtype == torch.float32 else "bf16")
        if weight.in_features % 32 == 0:
            splits = kernels.tiled_splits(rows, weight.out_features, weight.in_features) if partials and epilogue == "f32" else 1
            return kernels.gemm_tiled(x, weight.packed, weight.out_features, epilogue, splits=splits)
        plan = kernels.medium_plan(weight.out_features, weight.in_features, may_split=False)
        pieces = [kernels.gemm_medium(x[first:first + MEDIUM_ROWS], weight.packed, weight.out_features, epilogue, plan=plan)
                  for first in range(0, rows, MEDIUM_ROWS)]
        return torch.cat(pieces)
    if w is None or takes_packed(weight, rows, gated):
        if gated:
            return kernels.gemm_medium(x, weight.packed, weight.out_features, "gated")
        if out_dtype == torch.float32:
            plan = kernels.medium_plan(weight.out_features, weight.in_features, may_split=partials)
            return kernels.gemm_medium(x, weight.packed, weight.out_features, "f32", plan=plan)
        return kernels.gemm_medium(x, weight.packed, weight.out_features, "bf16")
    if gated:
        return kernels.silu_mul(kernels.gemm_bf16(x, w, torch.bfloat16))
    if partials and out_dtype == torch.float32:
        parts = kernels.library_splits(rows, weight.out_features, weight.in_features)
        if parts > 1:
            return kernels.gemm_bf16_split(x, w, parts)
    return kernels.gemm_bf16(x, w, out_dtype)
