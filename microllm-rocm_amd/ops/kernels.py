"""Python bindings of the HIP kernels: shape and type checks on the host, then one launch.

Every function takes torch tensors on the GPU, launches on torch's current HIP
stream and returns the output tensor. Checks happen here, before the launch, so
a kernel never sees operands that do not fit what its grid assumes.
"""
from __future__ import annotations

import ctypes
import os
from typing import List, NamedTuple, Optional, Sequence, Tuple

import torch

from . import library
from .library import KernelLibraryError

F32, BF16 = 0, 1
_CODES = {torch.float32: F32, torch.bfloat16: BF16}


def _code(dtype: torch.dtype) -> int:
    if dtype not in _CODES:
        raise KernelLibraryError(f"kernels take float32 or bfloat16, got {dtype}")
    return _CODES[dtype]


def _ptr(tensor: Optional[torch.Tensor]) -> ctypes.c_void_p:
    return ctypes.c_void_p(0 if tensor is None else tensor.data_ptr())


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", torch.cuda.current_device)


def _stream() -> ctypes.c_void_p:
    """The current stream of the current device (asked on every launch: a few microseconds through the public
    interface, a fraction of one through the call torch's own compiled code uses)."""
    if _raw_stream is not None:
        return ctypes.c_void_p(_raw_stream(_raw_device()))
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _check(status: int, lib) -> None:
    if status != 0:
        raise KernelLibraryError(lib.mll_last_error().decode("utf-8", "replace"))


def _need(condition: bool, text: str) -> None:
    if not condition:
        raise KernelLibraryError(text)


def _device_tensor(tensor: torch.Tensor, name: str, dtype: Optional[torch.dtype] = None) -> None:
    if tensor.is_cuda and tensor.is_contiguous() and (dtype is None or tensor.dtype == dtype):
        return
    _need(tensor.is_cuda, f"{name} must live on the GPU")
    _need(tensor.is_contiguous(), f"{name} must be contiguous")
    _need(tensor.dtype == dtype, f"{name} must be {dtype}, got {tensor.dtype}")


def embedding(table: torch.Tensor, ids: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    lib = library.load()
    _device_tensor(table, "embedding table")
    _device_tensor(ids, "token ids", torch.int32)
    _need(table.dim() == 2 and ids.dim() == 1, "embedding takes a [vocab, width] table and [tokens] ids")
    vocab, width = table.shape
    if out is None:
        out = torch.empty((ids.shape[0], width), dtype=torch.float32, device=table.device)
    _device_tensor(out, "embedding output", torch.float32)
    _need(tuple(out.shape) == (ids.shape[0], width), "embedding output has the wrong shape")
    _check(lib.mll_embedding(_ptr(table), _code(table.dtype), _ptr(ids), _ptr(out),
                             ids.shape[0], width, vocab, _stream()), lib)
    return out


def rms_norm(h: torch.Tensor, weight: torch.Tensor, eps: float, out_dtype: torch.dtype,
             delta: Optional[torch.Tensor] = None, rows: Optional[torch.Tensor] = None,
             write_h: bool = False, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``out = rms_norm(h[rows] + delta[rows]) * weight``; with ``write_h`` the sum replaces ``h``."""
    lib = library.load()
    _device_tensor(h, "residual stream", torch.float32)
    _device_tensor(weight, "norm weight", torch.float32)
    _need(h.dim() == 2 and weight.dim() == 1 and weight.shape[0] == h.shape[1],
          "rms_norm weight must match the last dimension")
    width = h.shape[1]
    delta_code, n_partials = F32, 1
    if delta is not None:
        _device_tensor(delta, "delta")
        _need(delta.dtype in (torch.float32, out_dtype), "delta must be float32 or have the output's dtype")
        if delta.dim() == 3:   # partial sums [parts, rows, width], added in order
            n_partials = delta.shape[0]
            _need(n_partials >= 1 and tuple(delta.shape[1:]) == tuple(h.shape), "delta parts must have the residual stream's shape")
        else:
            _need(tuple(delta.shape) == tuple(h.shape), "delta must have the residual stream's shape")
        delta_code = _code(delta.dtype)
    if rows is not None:
        _device_tensor(rows, "row selection", torch.int32)
        _need(not write_h, "cannot write h through a row selection")
        n_rows = rows.shape[0]
    else:
        n_rows = h.shape[0]
    if out is None:
        out = torch.empty((n_rows, width), dtype=out_dtype, device=h.device)
    _device_tensor(out, "norm output", out_dtype)
    _need(tuple(out.shape) == (n_rows, width), "norm output has the wrong shape")
    _check(lib.mll_rms_norm(_ptr(h), _ptr(delta), delta_code, n_partials, ctypes.c_int64(h.numel()), _ptr(rows),
                            _ptr(weight), ctypes.c_float(eps), _ptr(out),
                            _code(out_dtype), n_rows, width, int(write_h), _stream()), lib)
    return out


def residual_add(h: torch.Tensor, delta: torch.Tensor) -> torch.Tensor:
    lib = library.load()
    _device_tensor(h, "residual stream", torch.float32)
    _device_tensor(delta, "delta")
    _need(tuple(delta.shape) == tuple(h.shape) and h.dim() == 2, "delta must have the residual stream's shape")
    _check(lib.mll_residual_add(_ptr(h), _ptr(delta), _code(delta.dtype), h.shape[0], h.shape[1], _stream()), lib)
    return h


def rope_table(positions: torch.Tensor, inv_freq: torch.Tensor) -> torch.Tensor:
    """``[tokens, n_freq, 2]`` float32: cos and sin of ``position * inv_freq``, the angle taken in float64."""
    lib = library.load()
    _device_tensor(positions, "positions", torch.int32)
    _device_tensor(inv_freq, "inverse frequencies", torch.float64)
    _need(positions.dim() == 1 and inv_freq.dim() == 1 and inv_freq.shape[0] > 0, "rope_table takes [tokens] and [n_freq]")
    out = torch.empty((positions.shape[0], inv_freq.shape[0], 2), dtype=torch.float32, device=positions.device)
    _check(lib.mll_rope_table(_ptr(positions), _ptr(inv_freq), inv_freq.shape[0], positions.shape[0], _ptr(out), _stream()), lib)
    return out


def qkv_rope_store(qkv: torch.Tensor, bias: Optional[torch.Tensor], positions: torch.Tensor,
                   slot_mapping: Optional[torch.Tensor], inv_freq: Optional[torch.Tensor],
                   k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor],
                   heads: int, kv_heads: int, head_dim: int, page_size: int, out_dtype: torch.dtype,
                   q_out: Optional[torch.Tensor] = None, pair_order: bool = False,
                   cos_sin: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Bias, rotation and page write of fused projections ``[tokens, (heads + 2 kv_heads) * head_dim]``.

    ``qkv`` is float32 or ``out_dtype``; the rotated queries and the pages have ``out_dtype``. The rotation
    takes ``cos_sin`` (``rope_table``'s, for these tokens) or computes the same from ``inv_freq``. With
    ``pair_order`` the query and key heads of ``qkv`` come in ``rotary_pair_order``."""
    lib = library.load()
    _device_tensor(qkv, "qkv")
    _need(qkv.dtype in (torch.float32, out_dtype), "qkv must be float32 or have the output's dtype")
    total = (heads + 2 * kv_heads) * head_dim
    n_partials = 1
    if qkv.dim() == 3:   # partial sums [parts, tokens, total], added in order
        n_partials = qkv.shape[0]
        _need(n_partials >= 1, "qkv needs at least one part")
    n_tokens = qkv.shape[-2]
    _need(qkv.dim() in (2, 3) and qkv.shape[-1] == total, f"qkv must be [tokens, {total}]")
    if bias is not None:
        _device_tensor(bias, "qkv bias", torch.float32)
        _need(tuple(bias.shape) == (total,), "qkv bias has the wrong size")
    _device_tensor(positions, "positions", torch.int32)
    _need(tuple(positions.shape) == (n_tokens,), "positions must hold one entry per token")
    n_freq = 0
    if inv_freq is not None:
        _device_tensor(inv_freq, "inverse frequencies", torch.float64)
        n_freq = inv_freq.shape[0]
    if cos_sin is not None:
        _device_tensor(cos_sin, "cos/sin table", torch.float32)
        _need(cos_sin.dim() == 3 and cos_sin.shape[0] == n_tokens and cos_sin.shape[2] == 2, "the cos/sin table must be [tokens, n_freq, 2]")
        _need(inv_freq is None or cos_sin.shape[1] == n_freq, "the cos/sin table and inv_freq differ in size")
        n_freq = cos_sin.shape[1]
    if slot_mapping is not None:
        _device_tensor(slot_mapping, "slot mapping", torch.int32)
        _need(tuple(slot_mapping.shape) == (n_tokens,), "slot mapping must hold one entry per token")
        _need(k_cache is not None and v_cache is not None, "slot mapping needs both caches")
        _check_pages(k_cache, v_cache, out_dtype, kv_heads, head_dim, page_size)
    if q_out is None:
        q_out = torch.empty((n_tokens, heads * head_dim), dtype=out_dtype, device=qkv.device)
    _device_tensor(q_out, "q output", out_dtype)
    _need(tuple(q_out.shape) == (n_tokens, heads * head_dim), "q output has the wrong shape")
    _check(lib.mll_qkv_rope_store(_ptr(qkv), _code(qkv.dtype), n_partials, ctypes.c_int64(n_tokens * total),
                                  _code(out_dtype), _ptr(bias), _ptr(positions), _ptr(slot_mapping),
                                  _ptr(inv_freq), _ptr(cos_sin), n_freq, _ptr(q_out), _ptr(k_cache), _ptr(v_cache),
                                  n_tokens, heads, kv_heads, head_dim, page_size, int(pair_order), _stream()), lib)
    return q_out


def rotary_pair_order(heads: int, kv_heads: int, head_dim: int, n_freq: int) -> torch.Tensor:
    """Row order of a stacked q/k/v weight that puts the two dims of a rotary pair side by side.

    In every query and key head rows ``2p`` and ``2p + 1`` become dims ``p`` and ``p + n_freq`` for
    ``p < n_freq``; the dims beyond the rotary part and the value heads stay where they are. Returns the
    old row of every new row."""
    _need(0 <= 2 * n_freq <= head_dim, "more rotary pairs than dims")
    within = torch.arange(head_dim)
    pairs = torch.stack([torch.arange(n_freq), torch.arange(n_freq) + n_freq], dim=1).reshape(-1)
    within[: 2 * n_freq] = pairs
    rows = []
    for head in range(heads + 2 * kv_heads):
        rotated = head < heads + kv_heads
        rows.append(head * head_dim + (within if rotated else torch.arange(head_dim)))
    return torch.cat(rows)


class _RowScale(ctypes.Structure):
    _fields_ = [("sumsq", ctypes.c_void_p), ("groups", ctypes.c_int), ("stride", ctypes.c_int), ("width", ctypes.c_int),
                ("eps", ctypes.c_float)]


class _ResidualNorm(ctypes.Structure):
    _fields_ = [("h", ctypes.c_void_p), ("norm_weight", ctypes.c_void_p), ("x_out", ctypes.c_void_p),
                ("sumsq_out", ctypes.c_void_p), ("sumsq_stride", ctypes.c_int)]


class RowScale(NamedTuple):
    """The rows' factors of an RMS norm that a product applies to its result: row ``r`` is multiplied by
    ``1 / sqrt(sumsq[r, :groups].sum() / width + eps)``. ``gemm_skinny_residual`` makes these."""
    sumsq: torch.Tensor     # float32 [rows, stride]; stride is a multiple of 4
    groups: int
    width: int
    eps: float


def _scale_argument(scale: Optional[RowScale], rows: int):
    if scale is None:
        return None
    _device_tensor(scale.sumsq, "sums of squares", torch.float32)
    _need(scale.sumsq.dim() == 2 and scale.sumsq.shape[0] == rows and rows <= 16, "row factors are [rows <= 16, stride]")
    _need(scale.sumsq.shape[1] % 4 == 0 and 0 < scale.groups <= scale.sumsq.shape[1], "rows of sums must be a multiple of 4 long")
    return ctypes.byref(_RowScale(_ptr(scale.sumsq), int(scale.groups), scale.sumsq.shape[1], int(scale.width), float(scale.eps)))


class _QkvStore(ctypes.Structure):
    _fields_ = [("bias", ctypes.c_void_p), ("slot_mapping", ctypes.c_void_p),
                ("cos_sin", ctypes.c_void_p), ("n_freq", ctypes.c_int), ("q_out", ctypes.c_void_p),
                ("k_cache", ctypes.c_void_p), ("v_cache", ctypes.c_void_p), ("heads", ctypes.c_int),
                ("kv_heads", ctypes.c_int), ("head_dim", ctypes.c_int), ("page_size", ctypes.c_int)]


def gemm_skinny_qkv(x: torch.Tensor, packed: torch.Tensor, bias: Optional[torch.Tensor],
                    slot_mapping: Optional[torch.Tensor], cos_sin: Optional[torch.Tensor],
                    k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor],
                    heads: int, kv_heads: int, head_dim: int, page_size: int,
                    scale: Optional[RowScale] = None) -> torch.Tensor:
    """Queries, keys and values of at most 16 bfloat16 rows in one kernel: ``gemm_skinny`` finished by the work
    of ``qkv_rope_store``. ``packed`` is the stacked weight packed in ``rotary_pair_order``; ``cos_sin`` is
    ``rope_table``'s for these rows (none: no rotation). Returns the queries."""
    lib = library.load()
    _device_tensor(x, "gemm input", torch.bfloat16)
    _device_tensor(packed, "packed weight", torch.bfloat16)
    _need(x.dim() == 2 and x.shape[0] <= 16, "gemm_skinny_qkv takes [m <= 16, k] activations")
    m, k = x.shape
    total = (heads + 2 * kv_heads) * head_dim
    _need(k % 8 == 0 and head_dim % 16 == 0, "gemm_skinny_qkv needs k % 8 == 0 and head_dim % 16 == 0")
    _need(packed.dim() == 5 and tuple(packed.shape[2:]) == (4, 16, 8) and packed.shape[0] == total // 16
          and packed.shape[1] == -(-k // 32), "the packed weight does not fit the heads and k")
    if bias is not None:
        _device_tensor(bias, "qkv bias", torch.float32)
        _need(tuple(bias.shape) == (total,), "qkv bias has the wrong size")
    n_freq = 0
    if cos_sin is not None:
        _device_tensor(cos_sin, "cos/sin table", torch.float32)
        _need(cos_sin.dim() == 3 and cos_sin.shape[0] == m and cos_sin.shape[2] == 2, "the cos/sin table must be [rows, n_freq, 2]")
        n_freq = cos_sin.shape[1]
        _need(2 * n_freq <= head_dim, "more rotary pairs than dims")
    if slot_mapping is not None:
        _device_tensor(slot_mapping, "slot mapping", torch.int32)
        _need(tuple(slot_mapping.shape) == (m,), "slot mapping must hold one entry per token")
        _need(k_cache is not None and v_cache is not None, "slot mapping needs both caches")
        _check_pages(k_cache, v_cache, torch.bfloat16, kv_heads, head_dim, page_size)
    q_out = torch.empty((m, heads * head_dim), dtype=torch.bfloat16, device=x.device)
    store = _QkvStore(_ptr(bias), _ptr(slot_mapping), _ptr(cos_sin), n_freq, _ptr(q_out),
                      _ptr(k_cache), _ptr(v_cache), heads, kv_heads, head_dim, page_size)
    _check(lib.mll_gemm_skinny_qkv(_ptr(x), _ptr(packed), m, k, ctypes.byref(store), _scale_argument(scale, m), _stream()), lib)
    return q_out


def gemm_skinny_residual(x: torch.Tensor, packed: torch.Tensor, h: torch.Tensor, norm_weight: torch.Tensor,
                         width: int, eps: float, scale: Optional[RowScale] = None) -> Tuple[torch.Tensor, RowScale]:
    """``h += x @ W.T`` for at most 16 bfloat16 rows, and the RMS norm of the sum begun.

    Returns ``(h * norm_weight)`` in bfloat16, the norm's result but for the rows' factors, and those factors as
    a ``RowScale`` for the product that takes it."""
    lib = library.load()
    _device_tensor(x, "gemm input", torch.bfloat16)
    _device_tensor(packed, "packed weight", torch.bfloat16)
    _device_tensor(h, "residual stream", torch.float32)
    _device_tensor(norm_weight, "norm weight", torch.float32)
    _need(x.dim() == 2 and x.shape[0] <= 16, "gemm_skinny_residual takes [m <= 16, k] activations")
    m, k = x.shape
    _need(h.dim() == 2 and h.shape[0] == m and h.shape[1] == width, "the residual stream must be [m, n]")
    n = h.shape[1]
    _need(tuple(norm_weight.shape) == (n,), "the norm's weight must be [n]")
    _need(k % 8 == 0, "gemm_skinny_residual needs k to be a multiple of 8")
    _need(packed.dim() == 5 and tuple(packed.shape[2:]) == (4, 16, 8) and packed.shape[0] == -(-n // 16)
          and packed.shape[1] == -(-k // 32), "the packed weight does not fit n and k")
    groups = -(-n // 16)
    x_out = torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
    sumsq = torch.empty((m, -(-groups // 4) * 4), dtype=torch.float32, device=x.device)
    residual = _ResidualNorm(_ptr(h), _ptr(norm_weight), _ptr(x_out), _ptr(sumsq), sumsq.shape[1])
    _check(lib.mll_gemm_skinny_residual(_ptr(x), _ptr(packed), m, n, k, ctypes.byref(residual), _scale_argument(scale, m),
                                        _stream()), lib)
    return x_out, RowScale(sumsq, groups, width, eps)


def _check_pages(k_cache, v_cache, dtype, kv_heads, head_dim, page_size=None) -> int:
    """Key and value pages must have the tiled shapes of ``cache.layout``; returns the page size."""
    from ..cache.layout import key_page_shape, value_page_shape
    _device_tensor(k_cache, "key pages", dtype)
    _device_tensor(v_cache, "value pages", dtype)
    _need(k_cache.dim() == 6 and v_cache.dim() == 4, "key pages must have 6 dimensions and value pages 4 (tiled layout)")
    found = k_cache.shape[2] * 16
    _need(page_size is None or page_size == found, "the pages do not have the page size given")
    pages = k_cache.shape[0]
    _need(tuple(k_cache.shape) == key_page_shape(pages, kv_heads, found, head_dim), "key pages have the wrong shape")
    _need(tuple(v_cache.shape) == value_page_shape(pages, kv_heads, found, head_dim), "value pages have the wrong shape")
    return found


def _check_paged(q, k_cache, v_cache, block_table, heads, kv_heads, head_dim) -> int:
    _device_tensor(q, "queries")
    _need(q.dim() == 2 and q.shape[1] == heads * head_dim, "queries must be [tokens, heads * head_dim]")
    page_size = _check_pages(k_cache, v_cache, q.dtype, kv_heads, head_dim)
    _device_tensor(block_table, "block table", torch.int32)
    _need(block_table.dim() == 2, "block table must be [requests, pages]")
    return page_size


ROWWISE_SPLIT_BELOW = 2048      # (token, head) rows: with fewer, a row's chunks of keys get a wave each


def rowwise_heads_a_wave(count: int) -> int:
    """Forces how many query heads of a kv head one wave of the float32 row-wise attention takes (1 to 8; 0 gives
    the choice back to the launch, which goes by the waves the step then has); returns the value before. Every
    count gives the same bits."""
    return int(library.load().mll_rowwise_heads_a_wave(int(count)))


def rowwise_chunks(longest: int, window: int) -> int:
    """The most chunks of keys (at absolute positions) that a row's visible keys can span, for rows that see at
    most ``longest`` keys' positions (position < longest)."""
    chunk = library.load().mll_paged_attention_rowwise_chunk()
    if window > 0:
        return min(-(-longest // chunk), (window + chunk - 2) // chunk + 1)
    return max(1, -(-longest // chunk))


def paged_attention_rowwise(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                            block_table: torch.Tensor, seq_of_token: torch.Tensor, positions: torch.Tensor,
                            scale: float, window: int, heads: int, kv_heads: int, head_dim: int,
                            out: Optional[torch.Tensor] = None, longest: Optional[int] = None,
                            split: Optional[bool] = None, usual: Optional[int] = None) -> torch.Tensor:
    """The plain attention kernel (any dtype, any head size). ``longest``: no position of the step reaches it
    (default: what the block table can hold). ``split``: a wave per chunk of keys and a merge, or a wave per row;
    by default by the number of rows. Both give the same bits. ``usual``: how far the step's rows reach now
    (default ``longest``, which may leave room for later steps of the same shape): how many query heads a wave
    of the float32 kernel takes goes by it, nothing else."""
    lib = library.load()
    page_size = _check_paged(q, k_cache, v_cache, block_table, heads, kv_heads, head_dim)
    n_tokens = q.shape[0]
    _device_tensor(seq_of_token, "request of token", torch.int32)
    _device_tensor(positions, "positions", torch.int32)
    _need(seq_of_token.shape[0] == n_tokens and positions.shape[0] == n_tokens,
          "request-of-token and positions must hold one entry per token")
    if out is None:
        out = torch.empty_like(q)
    _device_tensor(out, "attention output", q.dtype)
    _need(out.shape == q.shape, "attention output must have the queries' shape")
    capacity = block_table.shape[1] * page_size
    longest = capacity if longest is None else min(int(longest), capacity)
    if split is None:
        split = n_tokens * heads < ROWWISE_SPLIT_BELOW
    chunks = rowwise_chunks(max(longest, 1), window) if split else 0
    usual_chunks = rowwise_chunks(max(min(int(usual), longest), 1), window) if split and usual is not None else 0
    part_o = part_ml = None
    if chunks > 1:
        part_o = torch.empty((n_tokens, heads, chunks, head_dim), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((n_tokens, heads, chunks, 2), dtype=torch.float32, device=q.device)
    else:
        chunks = 0      # one chunk a row: the wave per row is the wave per chunk
    _check(lib.mll_paged_attention_rowwise(_ptr(q), _code(q.dtype), _ptr(k_cache), _ptr(v_cache), _ptr(block_table),
                                           block_table.shape[1], _ptr(seq_of_token), _ptr(positions), _ptr(out),
                                           _ptr(part_o), _ptr(part_ml), chunks, usual_chunks, ctypes.c_float(scale), int(window),
                                           n_tokens, heads, kv_heads, head_dim, page_size, _stream()), lib)
    return out


def silu_mul(gate_up: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``silu(gate) * up`` of fused rows ``[tokens, 2 * width]`` (gate first)."""
    lib = library.load()
    _device_tensor(gate_up, "gate/up")
    _need(gate_up.dim() == 2 and gate_up.shape[1] % 2 == 0, "gate/up must be [tokens, 2 * width]")
    n_tokens, double = gate_up.shape
    width = double // 2
    if out is None:
        out = torch.empty((n_tokens, width), dtype=gate_up.dtype, device=gate_up.device)
    _device_tensor(out, "silu_mul output", gate_up.dtype)
    _need(tuple(out.shape) == (n_tokens, width), "silu_mul output has the wrong shape")
    element = gate_up.element_size()
    for start in range(0, n_tokens, 65535):
        count = min(65535, n_tokens - start)
        gate_ptr = gate_up.data_ptr() + start * double * element
        _check(lib.mll_silu_mul(ctypes.c_void_p(gate_ptr), ctypes.c_void_p(gate_ptr + width * element),
                                ctypes.c_int64(double), ctypes.c_void_p(out.data_ptr() + start * width * element),
                                _code(gate_up.dtype), count, width, _stream()), lib)
    return out


def f32_small_variant(variant: int) -> int:
    """For measurements and tests: which kernel ``gemm_f32`` takes for at most 16 rows: 1 (an element a thread), 2
    (2 x 2 elements) or 4 (1 x 4; at most 8 rows); 0 gives the choice back. Returns the value before. The same
    bits whichever."""
    return int(library.load().mll_gemm_f32_small_variant(int(variant)))


def f32_splits(n: int, k: int) -> int:
    """Into how many parts ``gemm_f32`` may cut the reduction of a weight ``[n, k]``: the weight's shape decides,
    never the rows of a call, so that a row's bits are the same in every batch."""
    return int(library.load().mll_gemm_f32_splits(int(n), int(k)))


def gemm_f32(a: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
             out: Optional[torch.Tensor] = None, partials: bool = False) -> torch.Tensor:
    """``a @ weight.T (+ bias)`` in true float32 with a fixed order of additions per element. With ``partials``
    the result may come as ``[parts, m, n]`` (``f32_splits`` parts): sums over consecutive ranges of k, which the
    caller adds in order."""
    lib = library.load()
    _device_tensor(a, "gemm input", torch.float32)
    _device_tensor(weight, "gemm weight", torch.float32)
    _need(a.dim() == 2 and weight.dim() == 2 and a.shape[1] == weight.shape[1],
          "gemm takes [m, k] and [n, k]")
    m, k = a.shape
    n = weight.shape[0]
    if bias is not None:
        _device_tensor(bias, "gemm bias", torch.float32)
        _need(tuple(bias.shape) == (n,), "gemm bias has the wrong size")
    step = 65535 * 16
    splits = f32_splits(n, k) if partials and m <= step else 1
    shape = (m, n) if splits == 1 else (splits, m, n)
    if out is None:
        out = torch.empty(shape, dtype=torch.float32, device=a.device)
    _device_tensor(out, "gemm output", torch.float32)
    _need(tuple(out.shape) == shape, "gemm output has the wrong shape")
    for start in range(0, max(m, 1), step):
        count = min(step, m - start)
        _check(lib.mll_gemm_f32(ctypes.c_void_p(a.data_ptr() + start * k * 4), _ptr(weight), _ptr(bias),
                                ctypes.c_void_p(out.data_ptr() + start * n * 4), count, n, k, splits, _stream()), lib)
    return out


def argmax(logits: torch.Tensor) -> torch.Tensor:
    lib = library.load()
    _device_tensor(logits, "logits", torch.float32)
    _need(logits.dim() == 2, "logits must be [rows, vocab]")
    rows, vocab = logits.shape
    out = torch.empty((rows,), dtype=torch.int32, device=logits.device)
    parts = torch.empty((rows, lib.mll_argmax_slices(vocab), 4), dtype=torch.int32, device=logits.device)
    _check(lib.mll_argmax(_ptr(logits), _ptr(out), _ptr(parts), rows, vocab, _stream()), lib)
    return out


def sample(logits: torch.Tensor, temperature: torch.Tensor, top_k: Optional[torch.Tensor],
           uniform: torch.Tensor) -> torch.Tensor:
    lib = library.load()
    _device_tensor(logits, "logits", torch.float32)
    _need(logits.dim() == 2, "logits must be [rows, vocab]")
    rows = logits.shape[0]
    _device_tensor(temperature, "temperature", torch.float32)
    _device_tensor(uniform, "uniform", torch.float32)
    _need(temperature.shape[0] == rows and uniform.shape[0] == rows, "one temperature and uniform per row")
    if top_k is not None:
        _device_tensor(top_k, "top_k", torch.int32)
        _need(top_k.shape[0] == rows, "one top_k per row")
    out = torch.empty((rows,), dtype=torch.int32, device=logits.device)
    workspace = torch.empty((lib.mll_sample_workspace(rows, logits.shape[1]) // 4,), dtype=torch.int32, device=logits.device)
    _check(lib.mll_sample(_ptr(logits), _ptr(temperature), _ptr(top_k), _ptr(uniform), _ptr(out), _ptr(workspace),
                          rows, logits.shape[1], _stream()), lib)
    return out


LIBRARY_TUNE_ROWS = 1024     # with library tuning on, bfloat16 products of this many rows or more are tuned,
LIBRARY_TUNE_DECODE_ROWS = 64     # and those of up to this many (the gate/up product of large decode batches); between
                                  # the two a serving engine meets too many shapes, and short tuning runs mislead
_library_tuning = {"on": False, "seen": set(), "plain": set()}


def set_library_tuning(on: bool, results_file: Optional[str] = None) -> None:
    """Let the library choose the algorithm of a large product by timing its candidates instead of by its
    heuristic (the reference has --bf16-algorithm-index for that, apps/hf_infer.cpp:73). This is PyTorch's
    TunableOp, and the switch is global to the process: the first bfloat16-result product of a new shape with
    ``LIBRARY_TUNE_ROWS`` rows or more (gate/up of a prompt), or with at most ``LIBRARY_TUNE_DECODE_ROWS``, then
    takes seconds; later ones of the shape run the fastest candidate (7B sizes, 2048 rows: 0.45 instead of
    0.52 ms), or the heuristic's choice where that proves faster when the two are timed by turns. Results are
    kept in ``results_file`` (default: a file of this user in the temporary folder) and found again by later
    processes."""
    import torch.cuda.tunable as tunable
    if on:
        if results_file is None:
            results_file = os.path.join(library.private_temporary_folder(), "tunableop_results.csv")
        tunable.set_filename(results_file)
        tunable.set_max_tuning_duration(30)
        tunable.set_max_tuning_iterations(10)
    tunable.enable(on)
    tunable.tuning_enable(False)     # switched on around the first product of a shape only
    _library_tuning["on"] = on


def library_tuning() -> bool:
    return _library_tuning["on"]


def _tune_product(x: torch.Tensor, transposed_weight: torch.Tensor, shape: Tuple[int, int, int]) -> None:
    """Tune one shape, then time the tuned choice and the heuristic's by turns: the tuner's own runs are short."""
    import torch.cuda.tunable as tunable
    _library_tuning["seen"].add(shape)
    tunable.tuning_enable(True)
    try:
        torch.mm(x, transposed_weight)
    finally:
        tunable.tuning_enable(False)
    times = {True: 0.0, False: 0.0}
    try:
        for _ in range(3):
            for tuned in (True, False):
                tunable.enable(tuned)
                torch.mm(x, transposed_weight)
                start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                start.record()
                for _ in range(10):
                    torch.mm(x, transposed_weight)
                stop.record()
                stop.synchronize()
                times[tuned] += start.elapsed_time(stop)
    finally:
        tunable.enable(True)
    if times[False] < times[True]:
        _library_tuning["plain"].add(shape)


def gemm_bf16(x: torch.Tensor, weight: torch.Tensor, out_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """``x @ weight.T`` for bfloat16 operands with float32 accumulation.

    The product itself is the library's (hipBLASLt through ``torch.mm``), as the
    reference uses the library for its large linears (src/ops/optimized.cpp:94-450).
    """
    _device_tensor(x, "gemm input", torch.bfloat16)
    _device_tensor(weight, "gemm weight", torch.bfloat16)
    _need(x.dim() == 2 and weight.dim() == 2 and x.shape[1] == weight.shape[1], "gemm takes [m, k] and [n, k]")
    if out_dtype != torch.bfloat16:
        return torch.mm(x, weight.t(), out_dtype=out_dtype)
    if _library_tuning["on"]:
        shape = (x.shape[0], weight.shape[0], x.shape[1])
        tuned_rows = shape[0] >= LIBRARY_TUNE_ROWS or 0 < shape[0] <= LIBRARY_TUNE_DECODE_ROWS
        if tuned_rows and shape not in _library_tuning["seen"] and not torch.cuda.is_current_stream_capturing():
            _tune_product(x, weight.t(), shape)
        if shape in _library_tuning["plain"]:
            import torch.cuda.tunable as tunable
            tunable.enable(False)
            try:
                return torch.mm(x, weight.t())
            finally:
                tunable.enable(True)
    return torch.mm(x, weight.t())


LIBRARY_TILE = 256          # the library's products of many rows work in tiles of about 256 x 256
LIBRARY_WORKGROUPS = 224    # splitting the reduction pays while tiles x parts stay at or under this (of 256 compute units)
LIBRARY_SPLIT_LENGTH = 2048  # and every part of the reduction keeps at least this many terms


def library_splits(m: int, n: int, k: int) -> int:
    """Into how many ranges of the reduction ``gemm_bf16_split`` cuts a float32 product of ``m`` rows.

    The library takes one workgroup per tile of the result: a long reduction into a narrow result (a
    feed-forward's down projection) leaves most compute units idle. Measured on MI355X (m = 2048, n = 3584,
    k = 18944): 348 us whole, 205 us in two parts. Parts are powers of two up to 8; where the result's tiles do not
    fill their last round over the compute units to 90 % and the reduction has 16384 terms or more, four parts
    still gain (m = 4096 and 8192 at the sizes above)."""
    tiles = -(-m // LIBRARY_TILE) * -(-n // LIBRARY_TILE)
    best = 1
    for parts in (2, 4, 8):
        if k % (32 * parts) == 0 and k // parts >= LIBRARY_SPLIT_LENGTH and tiles * parts <= LIBRARY_WORKGROUPS:
            best = parts
    if best == 1 and k >= 16384 and k % 128 == 0:
        rounds = -(-tiles // 256)
        if tiles > LIBRARY_WORKGROUPS // 2 and tiles < 0.9 * 256 * rounds:
            best = 4
    return best


def gemm_bf16_split(x: torch.Tensor, weight: torch.Tensor, parts: int) -> torch.Tensor:
    """``x @ weight.T`` as ``[parts, m, n]`` float32 sums over ``parts`` equal ranges of the reduction, for the
    caller to add in order: one batched library product over strided views of both operands (no copies)."""
    _device_tensor(x, "gemm input", torch.bfloat16)
    _device_tensor(weight, "gemm weight", torch.bfloat16)
    _need(x.dim() == 2 and weight.dim() == 2 and x.shape[1] == weight.shape[1], "gemm takes [m, k] and [n, k]")
    m, k = x.shape
    _need(parts >= 1 and k % parts == 0, f"{parts} parts do not divide a reduction of {k}")
    if parts == 1:
        return torch.mm(x, weight.t(), out_dtype=torch.float32).unsqueeze(0)
    length = k // parts
    a = x.view(m, parts, length).transpose(0, 1)                          # [parts, m, length]
    b = weight.view(weight.shape[0], parts, length).permute(1, 2, 0)      # [parts, length, n]
    return torch.bmm(a, b, out_dtype=torch.float32)


def decode_splits(n_tokens: int, kv_heads: int, longest: int) -> int:
    """How many splits of the keys: about one workgroup per compute unit, at least 512 keys each, and 1024 where
    that alone fills the GPU (measured on MI355X: a wave keeps two pairs of key tiles on their way, so few long
    splits do as well as many short ones, and joining costs more the more there are)."""
    rows = max(1, n_tokens * kv_heads)
    splits = max(1, min(-(-256 // rows), longest // 512, 256))
    if splits > 1 and rows * splits >= 256 and longest // splits < 1024:
        splits //= 2
    return splits


def paged_attention_decode(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
                           seq_of_token: torch.Tensor, positions: torch.Tensor, scale: float, window: int,
                           heads: int, kv_heads: int, head_dim: int, n_splits: int,
                           out: Optional[torch.Tensor] = None, token_ids: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The MFMA kernel for bfloat16 queries that each attend alone (one token per request).

    ``token_ids`` restricts the work to those rows of ``q`` (the other rows of ``out`` are left alone)."""
    lib = library.load()
    page_size = _check_paged(q, k_cache, v_cache, block_table, heads, kv_heads, head_dim)
    _need(q.dtype == torch.bfloat16, "the decode kernel takes bfloat16")
    _need(head_dim % 16 == 0 and 16 <= head_dim <= 256, "the decode kernel takes head sizes in steps of 16 up to 256")
    _need(page_size % 16 == 0, "the decode kernel takes page sizes in steps of 16")
    n_rows = q.shape[0]
    _device_tensor(seq_of_token, "request of token", torch.int32)
    _device_tensor(positions, "positions", torch.int32)
    _need(seq_of_token.shape[0] == n_rows and positions.shape[0] == n_rows,
          "request-of-token and positions must hold one entry per token")
    n_tokens = n_rows
    if token_ids is not None:
        _device_tensor(token_ids, "token ids", torch.int32)
        _need(token_ids.dim() == 1 and token_ids.shape[0] <= n_rows, "token ids must list rows of q")
        n_tokens = token_ids.shape[0]
    if out is None:
        out = torch.empty_like(q)
    _device_tensor(out, "attention output", q.dtype)
    _need(out.shape == q.shape, "attention output must have the queries' shape")
    part_o = part_ml = None
    if n_splits > 1:
        part_o = torch.empty((n_tokens, heads, n_splits, head_dim), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((n_tokens, heads, n_splits, 2), dtype=torch.float32, device=q.device)
    _check(lib.mll_paged_attention_decode(_ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(block_table), block_table.shape[1],
                                          _ptr(seq_of_token), _ptr(positions), _ptr(token_ids), _ptr(out), _ptr(part_o),
                                          _ptr(part_ml), ctypes.c_float(scale), int(window), n_tokens, heads, kv_heads,
                                          head_dim, page_size, n_splits, _stream()), lib)
    return out


QUERY_TILE = 128   # tokens of one request in one tile of the prefill attention kernel; a workgroup takes two tiles


def pair_query_tiles(tiles: Sequence[Tuple[int, int, int, int]], adjacent: bool = False) -> List[Tuple[int, int, int, int, int]]:
    """The prefill attention's workgroups from its tiles. ``tiles``: (request, first token in the flat list,
    tokens, position of the first token). Returns (request, first token, tokens, first token, tokens) rows, the
    workgroups with the most keys to walk first, so that the longest start first.

    A tile's work grows with its position (it sees every earlier key), so of one request's tiles the last goes
    with the first, the last but one with the second and so on: every workgroup of a request then walks about as
    many keys. With ``adjacent`` neighbours go together instead: under a window every tile sees about as many keys,
    and neighbours see nearly the same ones. A request's odd tile goes alone."""
    by_request: dict = {}
    for tile in tiles:
        by_request.setdefault(tile[0], []).append(tile)
    pairs = []
    for request, own in by_request.items():
        own.sort(key=lambda tile: tile[3])
        count = len(own)
        if adjacent:
            couples = [(own[i], own[i + 1] if i + 1 < count else None) for i in range(0, count, 2)]
        else:
            couples = [(own[count - 1 - i], own[i] if i != count - 1 - i else None) for i in range((count + 1) // 2)]
        for first, second in couples:
            weight = first[3] + first[2] + (second[3] + second[2] if second else 0)
            pairs.append((weight, (request, first[1], first[2], second[1] if second else 0, second[2] if second else 0)))
    pairs.sort(key=lambda pair: -pair[0])
    return [pair[1] for pair in pairs]


def paged_attention_prefill(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
                            query_tiles: torch.Tensor, positions: torch.Tensor, scale: float, window: int,
                            heads: int, kv_heads: int, head_dim: int, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The MFMA kernel for bfloat16 portions of prompts; ``query_tiles`` rows are (request, first token, tokens,
    first token, tokens): two tiles of up to ``QUERY_TILE`` tokens of the request (``pair_query_tiles``)."""
    lib = library.load()
    page_size = _check_paged(q, k_cache, v_cache, block_table, heads, kv_heads, head_dim)
    _need(q.dtype == torch.bfloat16, "the prefill kernel takes bfloat16")
    _need(head_dim % 16 == 0 and 16 <= head_dim <= 256, "the prefill kernel takes head sizes in steps of 16 up to 256")
    _device_tensor(query_tiles, "query tiles", torch.int32)
    _need(query_tiles.dim() == 2 and query_tiles.shape[1] == 5, "query tiles must be [workgroups, 5]")
    _device_tensor(positions, "positions", torch.int32)
    _need(positions.shape[0] == q.shape[0], "positions must hold one entry per token")
    if out is None:
        out = torch.empty_like(q)
    _device_tensor(out, "attention output", q.dtype)
    _need(out.shape == q.shape, "attention output must have the queries' shape")
    _check(lib.mll_paged_attention_prefill(_ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(block_table), block_table.shape[1],
                                           _ptr(query_tiles), query_tiles.shape[0], _ptr(positions), _ptr(out),
                                           ctypes.c_float(scale), int(window), heads, kv_heads, head_dim, page_size,
                                           _stream()), lib)
    return out


def paged_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, view, ctx,
                    scale: float, window: int, heads: int, kv_heads: int, head_dim: int, planner=None) -> torch.Tensor:
    """Attention of the step's queries over their requests' pages; chooses the kernel for the batch's shape.

    bfloat16 with a head size in steps of 16: the MFMA kernels, split over the keys when every request brings
    one token, tiled over the queries otherwise (``planner``: the attention part's, whose plan for the step
    holds the tiles). Everything else (float32, other head sizes): the plain kernel.
    """
    mfma_fits = q.dtype == torch.bfloat16 and head_dim % 16 == 0 and head_dim <= 256
    if mfma_fits and ctx.max_count == 1:
        longest = max(ctx.planned_total, ctx.max_total)
        visible = min(longest, window) if window > 0 else longest
        splits = decode_splits(ctx.n_tokens, kv_heads, visible)
        return paged_attention_decode(q, k_cache, v_cache, view.block_table, ctx.seq_of_token, ctx.positions,
                                      scale, window, heads, kv_heads, head_dim, splits)
    if mfma_fits:
        # Portions go to the tiled kernel; requests that bring one token, if any, to the split kernel.
        _need(planner is not None, "portions of prompts need the attention part's planner for their tiles")
        plan = ctx.plan_of(planner)
        out = torch.empty_like(q)
        if plan.tiles.shape[0] > 0:
            paged_attention_prefill(q, k_cache, v_cache, view.block_table, plan.tiles, ctx.positions,
                                    scale, window, heads, kv_heads, head_dim, out=out)
        if plan.single_tokens.shape[0] > 0:
            longest = max(plan.max_single_total, ctx.planned_total) if ctx.fixed else plan.max_single_total
            visible = min(longest, window) if window > 0 else longest
            splits = decode_splits(plan.single_tokens.shape[0], kv_heads, visible)
            paged_attention_decode(q, k_cache, v_cache, view.block_table, ctx.seq_of_token, ctx.positions,
                                   scale, window, heads, kv_heads, head_dim, splits, out=out, token_ids=plan.single_tokens)
        return out
    return paged_attention_rowwise(q, k_cache, v_cache, view.block_table, ctx.seq_of_token, ctx.positions,
                                   scale, window, heads, kv_heads, head_dim, longest=max(ctx.planned_total, ctx.max_total),
                                   usual=ctx.max_total)


def pack_weight(weight: torch.Tensor, interleave_halves: bool = False,
                row_order: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The weight ``[n, k]`` in the order ``gemm_skinny`` streams it: ``[n/16, k/32, 4, 16, 8]``, zero padded.

    With ``interleave_halves`` rows ``i`` and ``n/2 + i`` become neighbours first (gate and up of a gated
    feed-forward), which is what the gated epilogue expects. With ``row_order`` new row ``i`` is old row
    ``row_order[i]``.
    """
    _need(weight.dim() == 2 and weight.dtype == torch.bfloat16, "pack_weight takes a bfloat16 matrix")
    n, k = weight.shape
    if row_order is not None:
        _need(not interleave_halves and tuple(row_order.shape) == (n,), "row_order must name every row once")
        weight = weight[row_order.to(weight.device)]
    if interleave_halves:
        _need(n % 2 == 0, "interleaving needs an even number of rows")
        weight = torch.stack([weight[: n // 2], weight[n // 2:]], dim=1).reshape(n, k)
    n_padded, k_padded = -(-n // 16) * 16, -(-k // 32) * 32
    if (n_padded, k_padded) != (n, k):
        padded = torch.zeros((n_padded, k_padded), dtype=weight.dtype, device=weight.device)
        padded[:n, :k] = weight
        weight = padded
    packed = weight.view(n_padded // 16, 16, k_padded // 32, 4, 8).permute(0, 2, 3, 1, 4).contiguous()
    return packed


SKINNY_MAX_ROWS = 64


def gemm_skinny(x: torch.Tensor, packed: torch.Tensor, n: int, epilogue: str = "f32",
                scale: Optional[RowScale] = None) -> torch.Tensor:
    """``x @ W.T`` for at most 64 bfloat16 rows and a packed weight.

    ``f32``: float32 ``[m, n]``; ``bf16``: bfloat16 ``[m, n]``; ``gated``: bfloat16 ``[m, n / 2]`` of
    silu(gate) * up for interleaved rows. With ``scale`` (at most 16 rows) the rows of the product are
    multiplied by its factors first.
    """
    lib = library.load()
    _device_tensor(x, "gemm input", torch.bfloat16)
    _device_tensor(packed, "packed weight", torch.bfloat16)
    _need(packed.dim() == 5 and tuple(packed.shape[2:]) == (4, 16, 8), "gemm_skinny takes a packed weight")
    _need(x.dim() == 2, "gemm_skinny takes [m, k] activations")
    m, k = x.shape
    _need(m <= SKINNY_MAX_ROWS, "gemm_skinny takes at most 64 rows")
    _need(k % 8 == 0, "gemm_skinny needs k to be a multiple of 8")
    _need(packed.shape[0] == -(-n // 16) and packed.shape[1] == -(-k // 32), "the packed weight does not fit n and k")
    if epilogue == "f32":
        code, out = 0, torch.empty((m, n), dtype=torch.float32, device=x.device)
    elif epilogue == "bf16":
        code, out = 1, torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
    elif epilogue == "gated":
        code, out = 2, torch.empty((m, n // 2), dtype=torch.bfloat16, device=x.device)
    else:
        raise KernelLibraryError(f"unknown epilogue {epilogue!r}")
    _check(lib.mll_gemm_skinny(_ptr(x), _ptr(packed), _ptr(out), code, m, n, k, _scale_argument(scale, m), _stream()), lib)
    return out


MEDIUM_WORKGROUPS = 224     # workgroups of 8 waves that gemm_medium wants at least (MI355X has 256 compute units)
MEDIUM_WHOLE_WORKGROUPS = 128     # where the reduction cannot be split, two tiles a wave from this many workgroups on


def medium_plan(n: int, k: int, may_split: bool = True) -> Tuple[int, int, int]:
    """(tiles of W a wave takes, waves a workgroup, splits of k) for ``gemm_medium``.

    A function of the weight's shape alone, so that a row's sum does not depend on the other rows. Two tiles a
    wave halve the reads of the activations; they are taken where splitting k (at most 16 times, a stage of 256
    at least per split) still gives enough workgroups.
    """
    n_tiles = -(-n // 16)
    stages = -(-k // 256)
    most = 1
    while may_split and most * 2 <= min(16, stages):
        most *= 2
    tiles_per_wave = 2 if -(-n_tiles // 16) * most >= (MEDIUM_WORKGROUPS if may_split else MEDIUM_WHOLE_WORKGROUPS) else 1
    groups = -(-n_tiles // (8 * tiles_per_wave))
    splits = 1
    while splits < most and groups * splits < MEDIUM_WORKGROUPS:
        splits *= 2
    return tiles_per_wave, 8, splits


def gemm_medium(x: torch.Tensor, packed: torch.Tensor, n: int, epilogue: str = "f32",
                plan: Optional[Tuple[int, int, int]] = None) -> torch.Tensor:
    """``x @ W.T`` for at most 64 bfloat16 rows ``[m, k]`` and a packed weight, activations shared through LDS.

    ``plan`` is ``medium_plan``'s by default; pass ``medium_plan(n, k, may_split=False)`` for a plain ``[m, n]``.

    ``f32``: float32 ``[m, n]``, or ``[splits, m, n]`` partial sums to be added in order when the plan splits k;
    ``bf16`` and ``gated`` as in ``gemm_skinny`` (they never split).
    """
    lib = library.load()
    _device_tensor(x, "gemm input", torch.bfloat16)
    _device_tensor(packed, "packed weight", torch.bfloat16)
    _need(packed.dim() == 5 and tuple(packed.shape[2:]) == (4, 16, 8), "gemm_medium takes a packed weight")
    _need(x.dim() == 2, "gemm_medium takes [m, k] activations")
    m, k = x.shape
    _need(m <= SKINNY_MAX_ROWS, "gemm_medium takes at most 64 rows")
    _need(k % 8 == 0, "gemm_medium needs k to be a multiple of 8")
    _need(packed.shape[0] == -(-n // 16) and packed.shape[1] == -(-k // 32), "the packed weight does not fit n and k")
    tiles_per_wave, waves, splits = plan if plan is not None else medium_plan(n, k, may_split=epilogue == "f32")
    _need(epilogue == "f32" or splits == 1, "only float32 partial sums can be split over k")
    if epilogue == "f32":
        code = 0
        out = torch.empty((splits, m, n) if splits > 1 else (m, n), dtype=torch.float32, device=x.device)
    elif epilogue == "bf16":
        code, out = 1, torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
    elif epilogue == "gated":
        code, out = 2, torch.empty((m, n // 2), dtype=torch.bfloat16, device=x.device)
    else:
        raise KernelLibraryError(f"unknown epilogue {epilogue!r}")
    _check(lib.mll_gemm_medium(_ptr(x), _ptr(packed), _ptr(out), code, m, n, k, tiles_per_wave, waves, splits, _stream()), lib)
    return out


TILED_TILE = 256            # gemm_tiled works in tiles of up to 256 x 256, stages of 64 of the reduction
COMPUTE_UNITS = 256         # of an MI355X: a workgroup of gemm_tiled has one to itself
TILED_SPLIT_STAGES = 8      # a part of the reduction keeps at least this many stages


def tiled_splits(m: int, n: int, k: int) -> int:
    """Into how many parts ``gemm_tiled`` cuts the reduction of a float32 product: while the result's tiles leave
    compute units idle (a workgroup a tile: 28 workgroups for 512 rows by 3584 columns), up to 8."""
    tiles = -(-m // TILED_TILE) * -(-n // TILED_TILE)
    stages = -(-k // 64)
    splits = 1
    while splits < 8 and tiles * splits * 2 <= LIBRARY_WORKGROUPS and stages // (splits * 2) >= TILED_SPLIT_STAGES:
        splits *= 2
    return splits


def tiled_tile_rows(m: int, n: int, splits: int = 1) -> int:
    """The rows of a workgroup's tile that ``gemm_tiled`` chooses for this product: 256, or fewer where that fills
    the compute units better. The result's bits do not depend on it."""
    return int(library.load().mll_tiled_tile_rows(m, n, splits))


def tiled_fill(m: int, n: int, splits: int = 1) -> float:
    """How much of the compute units' time ``gemm_tiled``'s workgroups fill for this product: workgroups over the
    places of the rounds of ``COMPUTE_UNITS`` they take (0.91 for 2048 x 4608 in tiles of 160 rows, 0.56 in tiles
    of 256)."""
    blocks = -(-m // tiled_tile_rows(m, n, splits)) * -(-n // TILED_TILE) * splits
    return blocks / (-(-blocks // COMPUTE_UNITS) * COMPUTE_UNITS)


def gemm_tiled(x: torch.Tensor, packed: torch.Tensor, n: int, epilogue: str = "f32", splits: int = 1,
               tile_rows: int = 0) -> torch.Tensor:
    """``x @ W.T`` for many bfloat16 rows and a packed weight, on this package's tiled MFMA kernel (0.9 to 1.1 of
    the library's untuned rate at 2048 rows and more, 1.1 to 1.4 PFLOP/s: for weights that are kept in the packed
    order alone). ``k`` must be
    a multiple of 32. With ``splits`` > 1 (float32 only) the result is ``[splits, m, n]`` sums over parts of the
    reduction for the caller to add in order."""
    lib = library.load()
    _device_tensor(x, "gemm input", torch.bfloat16)
    _device_tensor(packed, "packed weight", torch.bfloat16)
    _need(x.dim() == 2 and packed.dim() == 5 and tuple(packed.shape[2:]) == (4, 16, 8), "gemm_tiled takes [m, k] and a packed weight")
    m, k = x.shape
    _need(k % 32 == 0, "gemm_tiled needs k to be a multiple of 32")
    _need(packed.shape[0] == -(-n // 16) and packed.shape[1] == k // 32, "the packed weight does not fit n and k")
    _need(splits >= 1 and (splits == 1 or epilogue == "f32"), "only the float32 epilogue takes the reduction in parts")
    if epilogue == "f32":
        code, out = 0, torch.empty((m, n) if splits == 1 else (splits, m, n), dtype=torch.float32, device=x.device)
    elif epilogue == "bf16":
        code, out = 1, torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
    elif epilogue == "gated":
        _need(n % 2 == 0, "the gated epilogue needs an even number of weight rows")
        code, out = 2, torch.empty((m, n // 2), dtype=torch.bfloat16, device=x.device)
    else:
        raise KernelLibraryError(f"unknown epilogue {epilogue!r}")
    _check(lib.mll_gemm_tiled(_ptr(x), _ptr(packed), _ptr(out), code, m, n, k, splits, tile_rows, _stream()), lib)
    return out


def gemm_tiled_qkv(x: torch.Tensor, packed: torch.Tensor, bias: Optional[torch.Tensor],
                   slot_mapping: Optional[torch.Tensor], cos_sin: Optional[torch.Tensor],
                   k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor],
                   heads: int, kv_heads: int, head_dim: int, page_size: int, tile_rows: int = 0) -> torch.Tensor:
    """Queries, keys and values of many bfloat16 rows in one kernel: ``gemm_tiled`` finished by the work of
    ``qkv_rope_store`` (arguments as ``gemm_skinny_qkv``'s; ``k`` a multiple of 32 and an even number of rotary
    pairs). The reduction is not taken in parts, so this pays where ``tiled_splits`` is 1. Returns the queries."""
    lib = library.load()
    _device_tensor(x, "gemm input", torch.bfloat16)
    _device_tensor(packed, "packed weight", torch.bfloat16)
    _need(x.dim() == 2, "gemm_tiled_qkv takes [m, k] activations")
    m, k = x.shape
    total = (heads + 2 * kv_heads) * head_dim
    _need(k % 32 == 0 and head_dim % 16 == 0, "gemm_tiled_qkv needs k % 32 == 0 and head_dim % 16 == 0")
    _need(packed.dim() == 5 and tuple(packed.shape[2:]) == (4, 16, 8) and packed.shape[0] == total // 16
          and packed.shape[1] == k // 32, "the packed weight does not fit the heads and k")
    if bias is not None:
        _device_tensor(bias, "qkv bias", torch.float32)
        _need(tuple(bias.shape) == (total,), "qkv bias has the wrong size")
    n_freq = 0
    if cos_sin is not None:
        _device_tensor(cos_sin, "cos/sin table", torch.float32)
        _need(cos_sin.dim() == 3 and cos_sin.shape[0] == m and cos_sin.shape[2] == 2, "the cos/sin table must be [rows, n_freq, 2]")
        n_freq = cos_sin.shape[1]
        _need(2 * n_freq <= head_dim and n_freq % 2 == 0, "gemm_tiled_qkv takes an even number of rotary pairs, at most head_dim / 2")
    if slot_mapping is not None:
        _device_tensor(slot_mapping, "slot mapping", torch.int32)
        _need(tuple(slot_mapping.shape) == (m,), "slot mapping must hold one entry per token")
        _need(k_cache is not None and v_cache is not None, "slot mapping needs both caches")
        _check_pages(k_cache, v_cache, torch.bfloat16, kv_heads, head_dim, page_size)
    q_out = torch.empty((m, heads * head_dim), dtype=torch.bfloat16, device=x.device)
    store = _QkvStore(_ptr(bias), _ptr(slot_mapping), _ptr(cos_sin), n_freq, _ptr(q_out),
                      _ptr(k_cache), _ptr(v_cache), heads, kv_heads, head_dim, page_size)
    _check(lib.mll_gemm_tiled_qkv(_ptr(x), _ptr(packed), m, k, ctypes.byref(store), tile_rows, _stream()), lib)
    return q_out


def measured_peaks(device: Optional[torch.device] = None, read_bytes: int = 4 << 30) -> dict:
    """What this GPU reaches on a kernel that only reads memory once and on one that only issues bfloat16 MFMAs:
    ``{"hbm_read_GBps": ..., "mfma_bf16_TFLOPs": ...}`` (the best of a few launches each; well under a second)."""
    lib = library.load()
    device = device or torch.device("cuda", torch.cuda.current_device())
    sink = torch.zeros(1, dtype=torch.int32, device=device)
    data = torch.empty(read_bytes // 4, dtype=torch.int32, device=device).random_()
    units = torch.cuda.get_device_properties(device).multi_processor_count

    def best(launch, repeats: int = 5) -> float:
        launch()
        torch.cuda.synchronize(device)
        times = []
        for _ in range(repeats):
            start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            launch()
            stop.record()
            stop.synchronize()
            times.append(start.elapsed_time(stop) * 1e-3)
        return min(times)

    # The rate depends on how many workgroups share the reading (measured on MI355X, 256 units: 6.9 TB/s with two
    # workgroups a unit, 5.5 with eight): the best of a few counts is what the GPU reaches.
    read_time = min(best(lambda: _check(lib.mll_measure_read(_ptr(data), ctypes.c_int64(data.numel() * 4), _ptr(sink),
                                                             units * per_unit, _stream()), lib), repeats=3)
                    for per_unit in (1, 2, 4, 8))
    iterations, blocks = 4096, units * 4       # four waves a SIMD: one wave alone issues at two thirds of this rate
    mfma_time = best(lambda: _check(lib.mll_measure_mfma(iterations, _ptr(sink), blocks, _stream()), lib))
    flops = blocks * 4 * iterations * 16 * 16384.0
    del data
    return {"hbm_read_GBps": round(read_bytes / read_time / 1e9, 1), "mfma_bf16_TFLOPs": round(flops / mfma_time / 1e12, 1)}
