"""The Qwen2 dense decoder as a ``ModelSpec`` (``Qwen2ForCausalLM``).

Tensor names are the checkpoint's own; the reference's renaming table gives them
(src/model/model.cpp:1931-1980). Per layer: RMSNorm, attention with q/k/v biases
and split-half rotation, RMSNorm, SwiGLU, in the pre-norm arrangement
(src/model/model.cpp:851-860); a final RMSNorm and a head that is tied to the
embedding when ``tie_word_embeddings`` says so (src/model/model.cpp:1121-1128).
"""
from __future__ import annotations

from ..config.qwen2 import Qwen2Config
from ..config.registry import Architecture, register_architecture
from ..parts.spec import LayerSpec, ModelSpec, PartSpec, in_order
from ..weights.random_init import InitRule


def build_spec(config: Qwen2Config) -> ModelSpec:
    windows = config.layer_windows()
    position = PartSpec("rope_split_half", {"theta": config.rope_theta, "head_dim": config.head_dim})
    layers = []
    for index in range(config.num_hidden_layers):
        prefix = f"model.layers.{index}"
        attention_names = {"o_proj.weight": f"{prefix}.self_attn.o_proj.weight"}
        for role in ("q", "k", "v"):
            attention_names[f"{role}_proj.weight"] = f"{prefix}.self_attn.{role}_proj.weight"
            if config.attention_bias:
                attention_names[f"{role}_proj.bias"] = f"{prefix}.self_attn.{role}_proj.bias"
        layers.append(LayerSpec(
            arrangement="pre_norm",
            mixer_norm=PartSpec("rms_norm", {"size": config.hidden_size, "eps": config.rms_norm_eps},
                                {"weight": f"{prefix}.input_layernorm.weight"}),
            mixer=PartSpec("paged_attention", {
                "hidden_size": config.hidden_size, "num_heads": config.num_attention_heads,
                "num_kv_heads": config.num_key_value_heads, "head_dim": config.head_dim,
                "qkv_bias": config.attention_bias, "window": windows[index],
                "scale": config.head_dim ** -0.5, "position": position}, attention_names),
            ffn_norm=PartSpec("rms_norm", {"size": config.hidden_size, "eps": config.rms_norm_eps},
                              {"weight": f"{prefix}.post_attention_layernorm.weight"}),
            ffn=PartSpec("swiglu", {"hidden_size": config.hidden_size,
                                    "intermediate_size": config.intermediate_size},
                         {f"{role}_proj.weight": f"{prefix}.mlp.{role}_proj.weight"
                          for role in ("gate", "up", "down")}),
        ))
    sizes = {"vocab_size": config.vocab_size, "hidden_size": config.hidden_size}
    head_weight = "model.embed_tokens.weight" if config.tie_word_embeddings else "lm_head.weight"
    return ModelSpec(
        architecture=config.architecture,
        vocab_size=config.vocab_size,
        hidden_size=config.hidden_size,
        max_positions=config.max_position_embeddings,
        embedding=PartSpec("token_embedding", sizes, {"weight": "model.embed_tokens.weight"}),
        layers=tuple(layers),
        order=in_order(config.num_hidden_layers),
        final_norm=PartSpec("rms_norm", {"size": config.hidden_size, "eps": config.rms_norm_eps},
                            {"weight": "model.norm.weight"}),
        head=PartSpec("lm_head", sizes, {"weight": head_weight}),
    )


def init_rules(config: Qwen2Config):
    """Random weights: matrices, tables and biases ~ N(0, 0.02); norm weights 1 (+ N(0, norm_std) on request).

    The reference draws linears with std 1/sqrt(in) and zero biases
    (src/model/model.cpp:232-237, 285-295); biases are drawn here so that a test with
    random weights exercises them.
    """
    return [
        InitRule(suffix="layernorm.weight", mean=1.0, std_key="norm_std"),
        InitRule(suffix="norm.weight", mean=1.0, std_key="norm_std"),
        InitRule(suffix="", mean=0.0, std_key="std"),
    ]


register_architecture(Architecture(
    name="Qwen2ForCausalLM",
    config_from_dict=Qwen2Config.from_dict,
    build_spec=build_spec,
    init_rules=init_rules,
))
