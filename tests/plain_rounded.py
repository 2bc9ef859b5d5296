"""The plain implementation with the roundings that a bfloat16 engine cannot avoid, at the places it makes them.

Everything is still computed in float64 over whole sequences with the part functions of ``plain_qwen2``; what
is added is ``to_bfloat16`` at the points where a bfloat16 engine hands a value to a matrix product or to the
cache: a norm's result, the queries, keys and values after bias and rotation, the attention's probabilities
(the values' weights; their sum is taken before rounding) and its result, SiLU(gate) * up. The residual
stream, the scores, the softmax's sum and the logits stay unrounded, as they are float32 in the engine.

Two of these places depend on how many rows a step has, and so on how the work was cut, which is why every
position carries its own flags (``Rows``):
* ``split_norm``: with few rows the engine takes a norm apart. The product before it adds its result to the
  stream and rounds ``stream * norm weight``; the product after it multiplies its own rows by
  ``1 / sqrt(mean(stream^2) + eps)``. The first norm of the first layer and the final norm have no product
  before them and are never split.
* ``round_gate_up``: with many rows gate and up come out of a library product as bfloat16 and are rounded before
  SiLU; with few rows SiLU(gate) * up is formed from the unrounded sums.

Against this run an engine's error is what its own arithmetic adds (float32 sums in another order, the
probabilities rounded against a running maximum instead of the final one, hardware exponentials), not what the
format costs, so the comparison can be an order of magnitude tighter than against the exact run.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Dict, Optional, Sequence

import numpy as np

import plain_qwen2 as plain


class Twin:
    """An equally valid way to make the same roundings. An engine's float32 arithmetic differs from float64 by a
    few 1e-6 of a value before it is rounded (sums of hundreds to thousands of float32 products, hardware
    exponentials), and its attention rounds a probability against the maximum of the keys walked so far, not the
    final one, which moves every probability on the rounding grid. ``before_rounding`` and ``grid_shift`` do the
    like to the plain run: how far its logits move is how far two faithful bfloat16 implementations of this model
    may lie apart, and an engine is held to a small multiple of that."""
    NOISE = 4e-6        # float32's 1.2e-7 times the root of a thousand terms
    grid_shift = 1.37   # no power of two

    def __init__(self, seed: int):
        self.rng = np.random.default_rng(seed)

    def before_rounding(self, x: np.ndarray) -> np.ndarray:
        return x * (1.0 + self.NOISE * self.rng.standard_normal(x.shape))


def to_bfloat16(x: np.ndarray, twin: Optional[Twin] = None) -> np.ndarray:
    """Round to the nearest value with 8 bits of mantissa, ties to even; returned as float64."""
    if twin is not None:
        x = twin.before_rounding(x)
    bits = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    rounded = (bits + (np.uint32(0x7FFF) + ((bits >> np.uint32(16)) & np.uint32(1)))) & np.uint32(0xFFFF0000)
    return rounded.view(np.float32).astype(np.float64)


@dataclass
class Rows:
    """Per position: how the step that ran it rounds (see the module's text)."""
    split_norm: np.ndarray      # bool [T]
    round_gate_up: np.ndarray   # bool [T]

    @classmethod
    def all(cls, count: int, split_norm: bool, round_gate_up: bool) -> "Rows":
        return cls(np.full(count, split_norm), np.full(count, round_gate_up))


def normed(h: np.ndarray, weight: np.ndarray, eps: float, split: np.ndarray, twin: Optional[Twin] = None):
    """A norm's result as the next product takes it: (rounded values, factor of every row to apply after the
    product). Not split: the norm, rounded, and a factor of 1."""
    whole = to_bfloat16(plain.rms_norm(h, weight, eps), twin)
    factor = 1.0 / np.sqrt(np.mean(h * h, axis=-1) + eps)
    values = np.where(split[:, None], to_bfloat16(h * weight, twin), whole)
    return values, np.where(split, factor, 1.0)


def attention_with_rounded_weights(q: np.ndarray, k: np.ndarray, v: np.ndarray, scale: float,
                                   window: Optional[int], block: int = 256, twin: Optional[Twin] = None) -> np.ndarray:
    """``plain.causal_gqa_attention`` with the probabilities rounded where they weigh the values: weights
    ``exp(s - max)``, their sum taken unrounded, ``sum_j bfloat16(w_j) v_j / sum``."""
    tokens, heads, _ = q.shape
    repeats = heads // k.shape[1]
    out = np.zeros_like(q)
    for head in range(heads):
        kv_head = head // repeats
        for first in range(0, tokens, block):
            last = min(tokens, first + block)
            low = 0 if window is None else max(0, first - window + 1)
            scores = (q[first:last, head, :] @ k[low:last, kv_head, :].T) * scale
            p = np.arange(first, last)[:, None]
            j = np.arange(low, last)[None, :]
            visible = j <= p if window is None else (j <= p) & (p - j < window)
            scores = np.where(visible, scores, -np.inf)
            weights = np.exp(scores - scores.max(axis=1, keepdims=True))
            total = weights.sum(axis=1, keepdims=True)
            if twin is None:
                rounded = to_bfloat16(weights)
            else:
                rounded = to_bfloat16(weights * twin.grid_shift, twin) / twin.grid_shift
            out[first:last, head, :] = (rounded @ v[low:last, kv_head, :]) / total
    return out


def attention_layer(values: np.ndarray, factor: np.ndarray, weights: Dict[str, np.ndarray], prefix: str, config: dict,
                    window: Optional[int], twin: Optional[Twin] = None) -> np.ndarray:
    heads, kv_heads, head_dim = config["num_attention_heads"], config["num_key_value_heads"], plain.head_dim_of(config)
    tokens = values.shape[0]
    positions = np.arange(tokens)

    def project(role: str, count: int):
        y = plain.linear(values, weights[f"{prefix}.self_attn.{role}_proj.weight"]) * factor[:, None]
        bias = weights.get(f"{prefix}.self_attn.{role}_proj.bias")
        return (y if bias is None else y + bias).reshape(tokens, count, head_dim)

    q = to_bfloat16(plain.rope_split_half(project("q", heads), positions, config["rope_theta"]), twin)
    k = to_bfloat16(plain.rope_split_half(project("k", kv_heads), positions, config["rope_theta"]), twin)
    v = to_bfloat16(project("v", kv_heads), twin)
    o = to_bfloat16(attention_with_rounded_weights(q, k, v, 1.0 / math.sqrt(head_dim), window, twin=twin), twin)
    return plain.linear(o.reshape(tokens, heads * head_dim), weights[f"{prefix}.self_attn.o_proj.weight"])


def feed_forward(values: np.ndarray, factor: np.ndarray, weights: Dict[str, np.ndarray], prefix: str,
                 round_gate_up: np.ndarray, twin: Optional[Twin] = None) -> np.ndarray:
    gate = plain.linear(values, weights[f"{prefix}.mlp.gate_proj.weight"]) * factor[:, None]
    up = plain.linear(values, weights[f"{prefix}.mlp.up_proj.weight"]) * factor[:, None]
    gate = np.where(round_gate_up[:, None], to_bfloat16(gate, twin), gate)
    up = np.where(round_gate_up[:, None], to_bfloat16(up, twin), up)
    return plain.linear(to_bfloat16(plain.silu(gate) * up, twin), weights[f"{prefix}.mlp.down_proj.weight"])


def forward(config: dict, weights: Dict[str, np.ndarray], tokens: Sequence[int], rows: Rows,
            twin: Optional[Twin] = None) -> np.ndarray:
    """Logits [T, vocab] as ``plain.forward`` gives them, with a bfloat16 engine's roundings; with ``twin`` made
    in another, equally valid way."""
    windows = plain.layer_windows(config)
    eps = config["rms_norm_eps"]
    never = np.zeros(len(tokens), dtype=bool)
    h = plain.embedding(weights["model.embed_tokens.weight"], tokens)
    for index in range(config["num_hidden_layers"]):
        prefix = f"model.layers.{index}"
        values, factor = normed(h, weights[f"{prefix}.input_layernorm.weight"], eps, never if index == 0 else rows.split_norm, twin)
        h = h + attention_layer(values, factor, weights, prefix, config, windows[index], twin)
        values, factor = normed(h, weights[f"{prefix}.post_attention_layernorm.weight"], eps, rows.split_norm, twin)
        h = h + feed_forward(values, factor, weights, prefix, rows.round_gate_up, twin)
    x, _ = normed(h, weights["model.norm.weight"], eps, never, twin)
    head = weights["model.embed_tokens.weight"] if config["tie_word_embeddings"] else weights["lm_head.weight"]
    return plain.linear(x, head)
