"""A plain, slow implementation of the Qwen2 dense decoder: whole sequences, no cache, float64.

Written from the reference's formulas, one function for each part, and sharing
no code with the package. Paths are relative to the reference's root. Where the
package goes beyond the reference (head_dim as a key, the sliding window) the
rule is stated in the function that implements it.
"""
from __future__ import annotations

import json
import math
import os
import struct
from typing import Dict, List, Optional, Sequence

import numpy as np


# ------------------------------------------------------------------------------------------------
# reading a model folder (independent of the package's reader)
def read_safetensors(path: str) -> Dict[str, np.ndarray]:
    """Header length, JSON header, payload (src/io/safetensors.cpp:492-526); values widened to float64."""
    with open(path, "rb") as handle:
        (header_size,) = struct.unpack("<Q", handle.read(8))
        header = json.loads(handle.read(header_size).decode("utf-8"))
        payload = handle.read()
    out = {}
    for name, member in header.items():
        if name == "__metadata__":
            continue
        begin, end = member["data_offsets"]
        raw = payload[begin:end]
        if member["dtype"] == "F32":
            values = np.frombuffer(raw, dtype="<f4").astype(np.float64)
        elif member["dtype"] == "BF16":
            bits = np.frombuffer(raw, dtype="<u2").astype(np.uint32) << 16
            values = bits.view(np.float32).astype(np.float64)
        elif member["dtype"] == "F16":
            values = np.frombuffer(raw, dtype="<f2").astype(np.float64)
        else:
            raise ValueError(f"plain reader does not know dtype {member['dtype']}")
        out[name] = values.reshape(member["shape"])
    return out


def read_config(folder: str) -> dict:
    with open(os.path.join(folder, "config.json"), "r", encoding="utf-8") as handle:
        return json.load(handle)


# ------------------------------------------------------------------------------------------------
# parts
def embedding(table: np.ndarray, ids: Sequence[int]) -> np.ndarray:
    """h0[t] = E[id_t] (src/ops/ops.cpp:608-617)."""
    return table[np.asarray(ids, dtype=np.int64)]


def rms_norm(x: np.ndarray, weight: np.ndarray, eps: float) -> np.ndarray:
    """y = x / sqrt(mean(x^2) + eps) * w: eps inside the root, weight last (src/ops/ops.cpp:687-698)."""
    mean_square = np.mean(x * x, axis=-1, keepdims=True)
    return x * (1.0 / np.sqrt(mean_square + eps)) * weight


def linear(x: np.ndarray, weight: np.ndarray, bias: Optional[np.ndarray] = None) -> np.ndarray:
    """y = x W^T + b with W as the checkpoint stores it, [out, in]; the reference multiplies by the
    transposed copy it makes at load (src/model/model.cpp:285, 1939-1947)."""
    y = x @ weight.T
    return y if bias is None else y + bias


def rope_split_half(x: np.ndarray, positions: np.ndarray, theta: float) -> np.ndarray:
    """x: [tokens, heads, hd]. Pair i is (i, i + hd/2); angle = p * theta^(-2i/hd);
    x'[i] = x[i] cos - x[i+hd/2] sin; x'[i+hd/2] = x[i] sin + x[i+hd/2] cos (src/ops/ops.cpp:863-878)."""
    head_dim = x.shape[-1]
    half = head_dim // 2
    pair = np.arange(half, dtype=np.float64)
    inv_freq = theta ** (-2.0 * pair / head_dim)
    angle = np.asarray(positions, dtype=np.float64)[:, None] * inv_freq[None, :]   # [tokens, half]
    cos, sin = np.cos(angle)[:, None, :], np.sin(angle)[:, None, :]
    first, second = x[..., :half], x[..., half:]
    return np.concatenate([first * cos - second * sin, first * sin + second * cos], axis=-1)


def causal_gqa_attention(q: np.ndarray, k: np.ndarray, v: np.ndarray, scale: float,
                         window: Optional[int] = None) -> np.ndarray:
    """q: [T, H, hd]; k, v: [T, KVH, hd] of one request, positions 0..T-1.

    Query head h uses kv head h // (H / KVH); scores (q . k_j) * scale over j <= p only; subtract the
    maximum, exponentiate, divide each probability by the sum, then weigh the values
    (src/ops/ops.cpp:2348-2383). Window (not in the reference, which refuses the option,
    src/model/huggingface.cpp:159-161): key j is visible to the query at p iff j <= p and p - j < window.
    """
    tokens, heads, head_dim = q.shape
    kv_heads = k.shape[1]
    repeats = heads // kv_heads
    if tokens > ROW_BY_ROW_LIMIT:
        return causal_gqa_attention_in_blocks(q, k, v, scale, window)
    out = np.zeros_like(q)
    for head in range(heads):
        kv_head = head // repeats
        for p in range(tokens):
            low = 0 if window is None else max(0, p - window + 1)
            scores = (k[low:p + 1, kv_head, :] @ q[p, head, :]) * scale
            weights = np.exp(scores - scores.max())
            weights = weights / weights.sum()
            out[p, head, :] = weights @ v[low:p + 1, kv_head, :]
    return out


ROW_BY_ROW_LIMIT = 256   # longer sequences take the same formula a block of queries at a time


def causal_gqa_attention_in_blocks(q: np.ndarray, k: np.ndarray, v: np.ndarray, scale: float,
                                   window: Optional[int] = None, block: int = 256) -> np.ndarray:
    """The formula of ``causal_gqa_attention`` for long sequences: the scores of a block of queries against every
    key up to the block's last position as one matrix, invisible keys set to -inf before the maximum is taken
    (their weights are then exactly 0), the same subtraction, exponential, division and weighted sum. A test
    holds it to the row-by-row function."""
    tokens, heads, head_dim = q.shape
    repeats = heads // k.shape[1]
    out = np.zeros_like(q)
    for head in range(heads):
        kv_head = head // repeats
        for first in range(0, tokens, block):
            last = min(tokens, first + block)
            low = 0 if window is None else max(0, first - window + 1)
            scores = (q[first:last, head, :] @ k[low:last, kv_head, :].T) * scale        # [queries, keys low..last)
            p = np.arange(first, last)[:, None]
            j = np.arange(low, last)[None, :]
            visible = j <= p if window is None else (j <= p) & (p - j < window)
            scores = np.where(visible, scores, -np.inf)
            weights = np.exp(scores - scores.max(axis=1, keepdims=True))
            weights = weights / weights.sum(axis=1, keepdims=True)
            out[first:last, head, :] = weights @ v[low:last, kv_head, :]
    return out


def silu(x: np.ndarray) -> np.ndarray:
    """x * sigmoid(x) with the sigmoid evaluated in the branch that cannot overflow (src/ops/ops.cpp:72-76)."""
    positive = x >= 0
    safe = np.where(positive, -x, x)          # always <= 0
    e = np.exp(safe)
    sigmoid = np.where(positive, 1.0 / (1.0 + e), e / (1.0 + e))
    return x * sigmoid


def swiglu_ffn(x: np.ndarray, gate_w: np.ndarray, up_w: np.ndarray, down_w: np.ndarray) -> np.ndarray:
    """down(silu(gate(x)) * up(x)), no biases (src/model/model.cpp:787-789; src/ops/ops.cpp:779-783)."""
    return linear(silu(linear(x, gate_w)) * linear(x, up_w), down_w)


def attention_layer(x: np.ndarray, weights: Dict[str, np.ndarray], prefix: str, config: dict,
                    window: Optional[int], kv_override=None, return_kv: bool = False):
    """Projections with bias, head split, rotation of q and k, attention, output projection without bias
    (src/model/model.cpp:472-520). ``kv_override`` = (k, v) of another layer replaces this layer's own."""
    heads, kv_heads, head_dim = config["num_attention_heads"], config["num_key_value_heads"], head_dim_of(config)
    tokens = x.shape[0]
    positions = np.arange(tokens)

    def project(role: str, count: int):
        bias = weights.get(f"{prefix}.self_attn.{role}_proj.bias")
        return linear(x, weights[f"{prefix}.self_attn.{role}_proj.weight"], bias).reshape(tokens, count, head_dim)

    q = rope_split_half(project("q", heads), positions, config["rope_theta"])
    if kv_override is None:
        k = rope_split_half(project("k", kv_heads), positions, config["rope_theta"])
        v = project("v", kv_heads)
    else:
        k, v = kv_override
    o = causal_gqa_attention(q, k, v, 1.0 / math.sqrt(head_dim), window)
    out = linear(o.reshape(tokens, heads * head_dim), weights[f"{prefix}.self_attn.o_proj.weight"])
    return (out, (k, v)) if return_kv else out


def head_dim_of(config: dict) -> int:
    """hidden / heads as in the reference (src/model/config.cpp:46-51) unless config.json gives head_dim."""
    return config.get("head_dim") or config["hidden_size"] // config["num_attention_heads"]


def layer_windows(config: dict) -> List[Optional[int]]:
    """Layers with index >= max_window_layers use the window when use_sliding_window is true."""
    layers = config["num_hidden_layers"]
    if not config.get("use_sliding_window", False):
        if "sliding_attention" in (config.get("layer_types") or []):
            raise ValueError("layer_types names sliding_attention layers but use_sliding_window is false")
        return [None] * layers
    if config.get("layer_types"):
        return [config["sliding_window"] if kind == "sliding_attention" else None for kind in config["layer_types"]]
    return [config["sliding_window"] if index >= config["max_window_layers"] else None for index in range(layers)]


def block(h: np.ndarray, weights: Dict[str, np.ndarray], index: int, config: dict, window: Optional[int]) -> np.ndarray:
    """Pre-norm: h' = h + Attn(Norm1(h)); h'' = h' + FFN(Norm2(h')) (src/model/model.cpp:851-860)."""
    prefix = f"model.layers.{index}"
    eps = config["rms_norm_eps"]
    h = h + attention_layer(rms_norm(h, weights[f"{prefix}.input_layernorm.weight"], eps), weights, prefix, config, window)
    x = rms_norm(h, weights[f"{prefix}.post_attention_layernorm.weight"], eps)
    return h + swiglu_ffn(x, weights[f"{prefix}.mlp.gate_proj.weight"], weights[f"{prefix}.mlp.up_proj.weight"],
                          weights[f"{prefix}.mlp.down_proj.weight"])


def forward(config: dict, weights: Dict[str, np.ndarray], tokens: Sequence[int],
            order: Optional[Sequence[int]] = None) -> np.ndarray:
    """Logits [T, vocab] at every position of one request (src/model/model.cpp:1031-1089): embedding, the
    layers (in ``order`` when given: a layer may run twice), final norm, head (tied: x E^T,
    src/model/model.cpp:1121-1128)."""
    windows = layer_windows(config)
    h = embedding(weights["model.embed_tokens.weight"], tokens)
    for index in (order if order is not None else range(config["num_hidden_layers"])):
        h = block(h, weights, index, config, windows[index])
    x = rms_norm(h, weights["model.norm.weight"], config["rms_norm_eps"])
    head = weights["model.embed_tokens.weight"] if config["tie_word_embeddings"] else weights["lm_head.weight"]
    return linear(x, head)


def layer_streams(config: dict, weights: Dict[str, np.ndarray], tokens: Sequence[int]) -> np.ndarray:
    """The residual stream after every layer, [layers, T, hidden]: what the reference's tensor trace shows layer
    by layer (include/microllm/profiling/trace.h:63, src/model/model.cpp:851-860)."""
    windows = layer_windows(config)
    h = embedding(weights["model.embed_tokens.weight"], tokens)
    after = []
    for index in range(config["num_hidden_layers"]):
        h = block(h, weights, index, config, windows[index])
        after.append(h)
    return np.stack(after)


# ------------------------------------------------------------------------------------------------
# token selection
def greedy(logits: np.ndarray) -> int:
    """First maximum (std::max_element, src/inference/generator.cpp:49-52)."""
    return int(np.argmax(logits))


def uniform_for(seed: int, draw: int) -> float:
    """The uniform in [0, 1) of a request's ``draw``-th sampled token: splitmix64 of seed and draw, top 24 bits.
    The reference draws from mt19937_64 through discrete_distribution (src/inference/generator.cpp:67-68),
    whose algorithm the library defines; a counter-based rule is used here so that any implementation can
    reproduce the stream."""
    mask = (1 << 64) - 1
    z = (seed * 0x9E3779B97F4A7C15 + (draw + 1) * 0xBF58476D1CE4E5B9) & mask
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & mask
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & mask
    z = z ^ (z >> 31)
    return (z >> 40) / float(1 << 24)


def sampling_weights(logits: np.ndarray, temperature: float, top_k: int) -> np.ndarray:
    """Weights exp(l/T - max/T) of the top_k largest logits (all when top_k == 0), zero elsewhere
    (src/inference/generator.cpp:54-66). Ties at the k-th value go to the lower token ids."""
    vocab = logits.shape[0]
    keep = np.ones(vocab, dtype=bool)
    if 0 < top_k < vocab:
        order = np.lexsort((np.arange(vocab), -logits))  # by logit descending, then id ascending
        keep[:] = False
        keep[order[:top_k]] = True
    scaled = logits / temperature
    return np.where(keep, np.exp(scaled - scaled.max()), 0.0)


def sample(logits: np.ndarray, temperature: float, top_k: int, uniform: float) -> int:
    """temperature 0 or top_k 1: the first maximum (src/inference/generator.cpp:49-52). Otherwise the token whose
    interval of the cumulative weights, taken in token order, holds uniform * total."""
    if temperature == 0.0 or top_k == 1:
        return greedy(logits)
    weights = sampling_weights(logits, temperature, top_k)
    cumulative = np.cumsum(weights)
    return int(np.searchsorted(cumulative, uniform * cumulative[-1], side="right"))


def generate_greedy(config: dict, weights: Dict[str, np.ndarray], prompt: Sequence[int], new_tokens: int) -> List[int]:
    """Append the argmax of the last position's logits, re-running the whole sequence each time
    (src/inference/generator.cpp:127-148 without its cache)."""
    sequence = list(prompt)
    for _ in range(new_tokens):
        sequence.append(greedy(forward(config, weights, sequence)[-1]))
    return sequence[len(prompt):]
