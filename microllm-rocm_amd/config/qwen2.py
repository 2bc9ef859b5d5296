"""Typed configuration of the Qwen2 dense decoder, read from its config.json keys.

Keys and checks follow the reference's loader (src/model/huggingface.cpp:152-179)
and validation (src/model/config.cpp:27-44). Added to what the reference reads:
``head_dim`` (the reference derives hidden/heads, src/model/config.cpp:46-51),
and the sliding-window keys ``use_sliding_window``, ``sliding_window``,
``max_window_layers`` and ``layer_types``, which the reference refuses
(src/model/huggingface.cpp:159-161).
"""
from __future__ import annotations

import dataclasses
import json
import math
import os
from dataclasses import dataclass
from typing import Any, Dict, Mapping, Optional, Tuple

from . import fields
from .fields import ConfigError

FULL_ATTENTION = "full_attention"
SLIDING_ATTENTION = "sliding_attention"


@dataclass(frozen=True)
class Qwen2Config:
    vocab_size: int
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    max_position_embeddings: int
    rope_theta: float
    rms_norm_eps: float
    tie_word_embeddings: bool
    use_sliding_window: bool = False
    sliding_window: Optional[int] = None
    max_window_layers: Optional[int] = None
    layer_types: Optional[Tuple[str, ...]] = None
    hidden_act: str = "silu"
    attention_bias: bool = True  # fixed for this architecture, src/model/huggingface.cpp:175
    torch_dtype: Optional[str] = None
    bos_token_id: Optional[int] = None
    eos_token_id: Optional[int] = None
    architecture: str = "Qwen2ForCausalLM"
    model_type: str = "qwen2"

    # ---- reading -------------------------------------------------------------------
    @classmethod
    def from_dict(cls, source: Mapping[str, Any]) -> "Qwen2Config":
        model_type = fields.string(source, "model_type", "qwen2")
        if model_type != "qwen2":
            raise ConfigError(f"Qwen2Config needs model_type qwen2, got {model_type!r}")
        hidden_act = fields.string(source, "hidden_act", "silu")
        if hidden_act != "silu":
            raise ConfigError(f"Qwen2 hidden_act must be silu, got {hidden_act!r}")
        if fields.boolean(source, "use_mrope", False):
            raise ConfigError("MRoPE variants of Qwen2 are not supported")
        if source.get("rope_scaling") is not None:
            raise ConfigError("rope_scaling is not supported by this engine")
        architectures = fields.string_list(source, "architectures", ["Qwen2ForCausalLM"])
        hidden = fields.integer(source, "hidden_size")
        heads = fields.integer(source, "num_attention_heads")
        head_dim = fields.integer(source, "head_dim", None)
        if head_dim is None:
            if heads <= 0 or hidden % heads != 0:
                raise ConfigError("hidden_size must divide into num_attention_heads when head_dim is absent")
            head_dim = hidden // heads
        layer_types = fields.string_list(source, "layer_types", None)
        config = cls(
            vocab_size=fields.integer(source, "vocab_size"),
            hidden_size=hidden,
            num_hidden_layers=fields.integer(source, "num_hidden_layers"),
            num_attention_heads=heads,
            num_key_value_heads=fields.integer(source, "num_key_value_heads", heads),
            head_dim=head_dim,
            intermediate_size=fields.integer(source, "intermediate_size"),
            max_position_embeddings=fields.integer(source, "max_position_embeddings"),
            rope_theta=fields.number(source, "rope_theta"),
            rms_norm_eps=fields.number(source, "rms_norm_eps"),
            tie_word_embeddings=fields.boolean(source, "tie_word_embeddings"),
            use_sliding_window=fields.boolean(source, "use_sliding_window", False),
            sliding_window=fields.integer(source, "sliding_window", None),
            max_window_layers=fields.integer(source, "max_window_layers", None),
            layer_types=tuple(layer_types) if layer_types is not None else None,
            hidden_act=hidden_act,
            torch_dtype=fields.string(source, "torch_dtype", None),
            bos_token_id=fields.integer(source, "bos_token_id", None),
            eos_token_id=fields.integer(source, "eos_token_id", None),
            architecture=architectures[0] if architectures else "Qwen2ForCausalLM",
            model_type=model_type,
        )
        config.validate()
        return config

    @classmethod
    def from_json_file(cls, path: str) -> "Qwen2Config":
        return cls.from_dict(fields.read_json_object(path))

    # ---- checks --------------------------------------------------------------------
    def validate(self) -> None:
        positives = {
            "vocab_size": self.vocab_size, "hidden_size": self.hidden_size,
            "num_hidden_layers": self.num_hidden_layers, "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads, "head_dim": self.head_dim,
            "intermediate_size": self.intermediate_size,
            "max_position_embeddings": self.max_position_embeddings,
        }
        for key, value in positives.items():
            if value <= 0:
                raise ConfigError(f"{key} must be positive, got {value}")
        if self.num_attention_heads % self.num_key_value_heads != 0:
            raise ConfigError("num_attention_heads must divide into num_key_value_heads groups")
        if self.head_dim % 2 != 0:
            raise ConfigError("RoPE head_dim must be even")
        if not self.rope_theta > 0.0:
            raise ConfigError("rope_theta must be positive")
        if not (math.isfinite(self.rms_norm_eps) and self.rms_norm_eps > 0.0):
            raise ConfigError("rms_norm_eps must be finite and positive")
        if self.layer_types is not None:
            if len(self.layer_types) != self.num_hidden_layers:
                raise ConfigError("layer_types must name every layer")
            for kind in self.layer_types:
                if kind not in (FULL_ATTENTION, SLIDING_ATTENTION):
                    raise ConfigError(f"unknown layer type {kind!r}")
            if SLIDING_ATTENTION in self.layer_types and not self.use_sliding_window:
                # The two keys contradict each other, and implementations differ in which one wins (one that
                # drops sliding_window when use_sliding_window is false attends to every key in every layer):
                # refused rather than guessed.
                raise ConfigError("layer_types names sliding_attention layers but use_sliding_window is false; "
                                  "set use_sliding_window to true or make every layer full_attention")
        windowed = any(window is not None for window in self.layer_windows())
        if windowed or self.use_sliding_window:
            if self.sliding_window is None or self.sliding_window <= 0:
                raise ConfigError("sliding_window must be positive when a layer uses the window")
        if self.use_sliding_window and self.layer_types is None:
            if self.max_window_layers is None or not 0 <= self.max_window_layers <= self.num_hidden_layers:
                raise ConfigError("max_window_layers must lie in [0, num_hidden_layers] when use_sliding_window is true")

    # ---- derived -------------------------------------------------------------------
    def layer_windows(self) -> Tuple[Optional[int], ...]:
        """The window of every layer, ``None`` for a layer that sees all keys.

        Without ``use_sliding_window`` no layer has one. With it, ``layer_types`` decides where it is given if
        present; otherwise layers with index ``>= max_window_layers`` use it.
        """
        if not self.use_sliding_window:
            return tuple(None for _ in range(self.num_hidden_layers))
        if self.layer_types is not None:
            return tuple(self.sliding_window if kind == SLIDING_ATTENTION else None
                         for kind in self.layer_types)
        first = self.max_window_layers if self.max_window_layers is not None else self.num_hidden_layers
        return tuple(self.sliding_window if index >= first else None
                     for index in range(self.num_hidden_layers))

    @property
    def q_size(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_key_value_heads * self.head_dim

    def parameter_count(self) -> int:
        """Closed form of src/model/config.cpp:58-78 with an explicit head_dim."""
        attention = 2 * self.hidden_size * self.q_size + 2 * self.hidden_size * self.kv_size
        biases = self.q_size + 2 * self.kv_size if self.attention_bias else 0
        ffn = 3 * self.hidden_size * self.intermediate_size
        norms = 2 * self.hidden_size
        total = self.vocab_size * self.hidden_size
        total += self.num_hidden_layers * (attention + biases + ffn + norms)
        total += self.hidden_size
        if not self.tie_word_embeddings:
            total += self.hidden_size * self.vocab_size
        return total

    # ---- writing -------------------------------------------------------------------
    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {
            "architectures": [self.architecture],
            "model_type": self.model_type,
            "hidden_act": self.hidden_act,
            "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "intermediate_size": self.intermediate_size,
            "max_position_embeddings": self.max_position_embeddings,
            "rope_theta": self.rope_theta,
            "rms_norm_eps": self.rms_norm_eps,
            "tie_word_embeddings": self.tie_word_embeddings,
            "use_sliding_window": self.use_sliding_window,
        }
        for key in ("sliding_window", "max_window_layers", "torch_dtype", "bos_token_id", "eos_token_id"):
            value = getattr(self, key)
            if value is not None:
                out[key] = value
        if self.layer_types is not None:
            out["layer_types"] = list(self.layer_types)
        return out

    def save(self, folder: str) -> str:
        os.makedirs(folder, exist_ok=True)
        path = os.path.join(folder, "config.json")
        with open(path, "w", encoding="utf-8") as handle:
            json.dump(self.to_dict(), handle, indent=2)
            handle.write("\n")
        return path

    def replace(self, **changes) -> "Qwen2Config":
        config = dataclasses.replace(self, **changes)
        config.validate()
        return config
