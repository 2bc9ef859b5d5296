"""Grouped-query attention over paged keys and values.

``q = x Wq + bq`` (likewise k, v), rotation of q and k after the bias, scores
``(q . k_j) * scale`` over the visible keys, softmax in float32, ``o = sum p_j v_j``,
then the output projection without bias (src/model/model.cpp:472-520;
src/ops/ops.cpp:2348-2383). Query head ``h`` uses kv head ``h // (heads / kv_heads)``.
With a window ``W`` key ``j`` is visible to a query at ``p`` iff ``j <= p`` and
``p - j < W``; the reference has no window (src/model/huggingface.cpp:159-161).
The three projections are stacked into one weight at bind time.
"""
from __future__ import annotations

import math
from typing import Dict, Mapping, Optional

import numpy as np
import torch

from ..ops import kernels
from .base import MATRIX, Mixer, PagedKVNeed, Runtime, TensorDecl, VECTOR
from .linear import MEDIUM_ROWS, SKINNY_ROWS, UnscaledRows, Weight, linear, linear_into_stream, takes_packed, takes_unscaled
from .registry import build_part, register_part
from .spec import PartSpec


class QueryTilePlanner:
    """The step metadata of the MFMA attention kernels (an ``engine.batch.StepPlanner``): requests that bring
    several tokens are cut into tiles of ``kernels.QUERY_TILE`` queries, which go to the prefill kernel's
    workgroups in twos (``kernels.pair_query_tiles``); requests that bring one token beside them are listed for the
    decode kernel. In a step of single tokens only there is nothing to plan: the decode kernel takes every row.

    Which two tiles share a workgroup: a late tile of a prompt with an early one, so that all workgroups walk about
    as many keys; under a window neighbours, which then read nearly the same keys. (Neighbours for long prompts
    without a window, the longest workgroups first, were measured too: a 16384-token prompt takes 3.0 instead of
    2.6 ms a layer that way.)

    Plan: ``tiles`` int32 [workgroups, 5]; ``single_tokens`` int32 [rows]; ``max_single_total``, the longest of
    the requests listed there."""
    padding = {"tiles": 0, "single_tokens": -1}      # an entry of two empty tiles; a row that is none: both passed over

    def __init__(self, windowed: bool):
        self.windowed = windowed
        self.key = ("paged_attention_query_tiles", windowed)

    def plan(self, host):
        counts, cu = host.counts, host.cu
        if host.single_tokens_only:
            return {"tiles": np.zeros((0, 5), np.int32), "single_tokens": np.zeros(0, np.int32)}, {"max_single_total": 0}
        mixed = any(count == 1 for count in counts)
        tile_list = [(index, int(cu[index]) + offset, min(kernels.QUERY_TILE, count - offset), host.starts[index] + offset)
                     for index, count in enumerate(counts) if not (mixed and count == 1)
                     for offset in range(0, count, kernels.QUERY_TILE)]
        tiles = np.asarray(kernels.pair_query_tiles(tile_list, adjacent=self.windowed), dtype=np.int32).reshape(-1, 5)
        single = np.asarray([cu[index] for index, count in enumerate(counts) if mixed and count == 1], dtype=np.int32)
        longest = max((host.totals[index] for index, count in enumerate(counts) if mixed and count == 1), default=0)
        return {"tiles": tiles, "single_tokens": single}, {"max_single_total": longest}


class PagedAttention(Mixer):
    fuses_residual = True
    graph_safe = True
    def __init__(self, spec: PartSpec, runtime: Runtime):
        super().__init__(spec, runtime)
        p = spec.params
        self.hidden = int(p["hidden_size"])
        self.heads = int(p["num_heads"])
        self.kv_heads = int(p["num_kv_heads"])
        self.head_dim = int(p["head_dim"])
        self.qkv_bias = bool(p.get("qkv_bias", False))
        self.window = p.get("window")
        self.scale = float(p.get("scale", 1.0 / math.sqrt(self.head_dim)))
        self.owns_kv = bool(p.get("owns_kv", True))  # False: only q is projected, another entry's pages are read
        if self.heads % self.kv_heads != 0:
            raise ValueError("num_heads must divide into num_kv_heads groups")
        position = p.get("position")
        self.position = build_part("position", position, runtime) if position is not None else None
        self.planner = QueryTilePlanner(bool(self.window))
        self.qkv_weight: Optional[torch.Tensor] = None
        self.qkv_bias_vector: Optional[torch.Tensor] = None
        self.o_weight: Optional[torch.Tensor] = None

    # ---- tensors -------------------------------------------------------------------------
    def _projections(self):
        out = [("q", self.heads * self.head_dim)]
        if self.owns_kv:
            out += [("k", self.kv_heads * self.head_dim), ("v", self.kv_heads * self.head_dim)]
        return out

    def tensors(self) -> Dict[str, TensorDecl]:
        decls = {}
        for role, width in self._projections():
            decls[self.name(f"{role}_proj.weight")] = TensorDecl((width, self.hidden), MATRIX)
            if self.qkv_bias:
                decls[self.name(f"{role}_proj.bias")] = TensorDecl((width,), VECTOR)
        decls[self.name("o_proj.weight")] = TensorDecl((self.hidden, self.heads * self.head_dim), MATRIX)
        return decls

    def bind(self, tensors: Mapping[str, torch.Tensor]) -> None:
        weights = [tensors[self.name(f"{role}_proj.weight")] for role, _ in self._projections()]
        if len({w.dtype for w in weights}) != 1:
            raise TypeError("the q, k and v weights of one layer must share a dtype to be stacked")
        # The packed copy of a weight whose heads rotate by the split-half rule holds the two dims of a rotary pair
        # side by side, so that the product for few rows can rotate and store in its epilogue.
        order = None
        if (self.position is None or self.position.fused_split_half) and self.head_dim % 16 == 0:
            n_freq = self.position.inv_freq.shape[0] if self.position is not None else 0
            order = kernels.rotary_pair_order(self.heads, self.kv_heads if self.owns_kv else 0, self.head_dim, n_freq)
        self.qkv_weight = Weight(torch.cat(weights, dim=0).contiguous() if len(weights) > 1 else weights[0], row_order=order,
                                 keep_plain=self.runtime.keep_plain_weights)
        del weights
        if self.qkv_bias:
            biases = [tensors[self.name(f"{role}_proj.bias")] for role, _ in self._projections()]
            self.qkv_bias_vector = torch.cat(biases, dim=0).contiguous() if len(biases) > 1 else biases[0]
        self.o_weight = Weight(tensors[self.name("o_proj.weight")], keep_plain=self.runtime.keep_plain_weights)

    def sub_parts(self):
        return (self.position,) if self.position is not None else ()

    def step_planner(self):
        return self.planner

    def cache_need(self):
        if not self.owns_kv:
            return None
        return PagedKVNeed(self.kv_heads, self.head_dim, self.window)

    def flops(self, tokens: int) -> float:
        """The projections', and 4 per (query, visible key, head, dim): scores and weighted values."""
        window = self.window or tokens
        pairs = sum(min(position + 1, window) for position in range(tokens))
        return super().flops(tokens) + 4.0 * self.heads * self.head_dim * pairs

    # ---- forward -------------------------------------------------------------------------
    def takes_unscaled(self, rows: int) -> bool:
        return self.qkv_weight.row_order is not None and takes_unscaled(self.qkv_weight, rows)

    TILED_FILL = 0.9     # with a copy of the weight as stored: the tiled product's workgroups must fill this much

    @classmethod
    def _tiled_whole(cls, weight: Weight, rows: int, cos_sin) -> bool:
        """Whether the tiled product with the q/k/v epilogue takes these rows: they are a prompt's, and the
        product's tiles fill the GPU without taking the reduction in parts (partial sums cannot be rotated and
        stored by the workgroup that made them). Where the weight is also kept as stored, only if the tiles fill
        the compute units' rounds: the product is then as fast as the library's and the epilogue is cheaper than
        the kernel it replaces (2048 rows at 7B sizes: 75 against 83 us; 512 rows: 59 against 38)."""
        if rows <= MEDIUM_ROWS or weight.in_features % 32 != 0 or (cos_sin is not None and cos_sin.shape[1] % 2 != 0):
            return False
        if kernels.tiled_splits(rows, weight.out_features, weight.in_features) != 1:
            return False
        return weight.tensor is None or kernels.tiled_fill(rows, weight.out_features) >= cls.TILED_FILL

    def forward(self, x, ctx, cache, residual=None):
        view = ctx.paged[cache.group]
        scale = None
        if isinstance(x, UnscaledRows):     # only where takes_unscaled said so: the q/k/v product applies the factors
            x, scale = x.values, x.scale
        kv_heads = cache.need.kv_heads
        stored_heads = self.kv_heads if self.owns_kv else 0
        slot_mapping = view.slot_mapping if self.owns_kv else None
        k_pages = cache.k if self.owns_kv else None
        v_pages = cache.v if self.owns_kv else None
        bias = self.qkv_bias_vector
        weight = self.qkv_weight
        fused = self.position is None or self.position.fused_split_half
        cos_sin = self.position.table(ctx) if self.position is not None and fused else None
        rotary_packed = weight.row_order is not None and weight.packed is not None and x.dtype == weight.dtype
        pair_order = rotary_packed and takes_packed(weight, x.shape[0])
        if pair_order and x.shape[0] <= SKINNY_ROWS:
            q = kernels.gemm_skinny_qkv(x, weight.packed, bias, slot_mapping, cos_sin, k_pages, v_pages,
                                        self.heads, stored_heads, self.head_dim, view.page_size, scale=scale)
        elif rotary_packed and scale is None and self._tiled_whole(weight, x.shape[0], cos_sin):
            q = kernels.gemm_tiled_qkv(x, weight.packed, bias, slot_mapping, cos_sin, k_pages, v_pages,
                                       self.heads, stored_heads, self.head_dim, view.page_size)
        else:
            if scale is not None:
                raise TypeError("rows without their factors reached a q/k/v product that cannot apply them")
            qkv = linear(x, weight, out_dtype=torch.float32, partials=fused)   # rounded once, after bias and rotation
            if not fused:
                if bias is not None:
                    qkv = qkv + bias
                    bias = None
                qkv = self.position.apply(qkv, ctx.positions, self.heads, stored_heads, self.head_dim).contiguous()
            q = kernels.qkv_rope_store(qkv, bias, ctx.positions, slot_mapping, None, k_pages, v_pages,
                                       self.heads, stored_heads, self.head_dim, view.page_size, self.runtime.dtype,
                                       pair_order=pair_order, cos_sin=cos_sin)
        window = int(self.window) if self.window else 0
        o = kernels.paged_attention(q, cache.k, cache.v, view, ctx, self.scale, window,
                                    self.heads, kv_heads, self.head_dim, planner=self.planner)
        if residual is not None:
            begun = linear_into_stream(o, self.o_weight, residual)
            if begun is not None:
                return begun
        return linear(o, self.o_weight, out_dtype=torch.float32, partials=True)   # summed into the residual stream in float32


register_part("mixer", "paged_attention", PagedAttention)
