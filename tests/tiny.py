"""The tiny configurations the tests run, and helpers to make model folders and compare logits."""
from __future__ import annotations

import os

import numpy as np
import torch

from microllm_rocm_amd.config import Qwen2Config
from microllm_rocm_amd.weights import write_model_folder

# Two configurations that differ in every size and option.
TINY_A = Qwen2Config(
    vocab_size=256, hidden_size=64, num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2,
    head_dim=16, intermediate_size=176, max_position_embeddings=128, rope_theta=10000.0, rms_norm_eps=1e-6,
    tie_word_embeddings=True, use_sliding_window=False)
TINY_B = Qwen2Config(
    vocab_size=384, hidden_size=96, num_hidden_layers=3, num_attention_heads=3, num_key_value_heads=1,
    head_dim=32, intermediate_size=256, max_position_embeddings=256, rope_theta=1e6, rms_norm_eps=1e-5,
    tie_word_embeddings=False, use_sliding_window=True, sliding_window=24, max_window_layers=1)
# A third one for long sequences: head_dim 48 (a multiple of 16 that is no power of two), a vocabulary and a
# width that are no powers of two, a window that spans several pages, more positions.
TINY_C = Qwen2Config(
    vocab_size=331, hidden_size=120, num_hidden_layers=2, num_attention_heads=5, num_key_value_heads=5,
    head_dim=48, intermediate_size=200, max_position_embeddings=1024, rope_theta=50000.0, rms_norm_eps=3e-6,
    tie_word_embeddings=False, use_sliding_window=True, sliding_window=100, max_window_layers=1)

SEEDS = {"A": 0, "B": 2, "C": 5}
STDS = {"A": {"std": 0.02, "norm_std": 0.0}, "B": {"std": 0.02, "norm_std": 0.1},
        "C": {"std": 0.05, "norm_std": 0.1}}
CONFIGS = {"A": TINY_A, "B": TINY_B, "C": TINY_C}


def make_folder(tmp_path, which: str, stds=None) -> str:
    folder = os.path.join(str(tmp_path), f"tiny_{which}")
    write_model_folder(folder, CONFIGS[which], SEEDS[which], dtype=torch.bfloat16, stds=stds or STDS[which])
    return folder


def random_tokens(seed: int, count: int, vocab: int):
    return np.random.default_rng(seed).integers(0, vocab, size=count).tolist()
