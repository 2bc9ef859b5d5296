"""Choosing the next token: greedy, temperature and top-k, on the device.

Rules follow the reference's ``sample_token`` (src/inference/generator.cpp:36-69):
temperature 0 or top_k 1 gives the first maximum; otherwise the top_k largest
logits (all when top_k is 0) are weighed by ``exp(l/T - max/T)`` and one is drawn;
non-finite logits are an error. The reference draws with ``mt19937_64`` and
``std::discrete_distribution``, whose algorithm the C++ library defines; here the
draw is by inverse CDF in token order with one uniform per token from a
counter-based rule keyed by (seed, index of the draw), so that the device kernel,
a plain implementation and a preempted request that is run again all see the
same stream. Defaults are the reference's (include/microllm/inference/generator.h:11-23).
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import List, Sequence, Tuple

import numpy as np
import torch

from ..ops import kernels
from ..ops.transfers import count_copy_to_host, on_device, on_host

_MASK = (1 << 64) - 1


@dataclass(frozen=True)
class SamplingParams:
    max_new_tokens: int = 32
    temperature: float = 1.0
    top_k: int = 0
    seed: int = 1
    stop_tokens: Tuple[int, ...] = ()

    @property
    def greedy(self) -> bool:
        return self.temperature == 0.0 or self.top_k == 1

    def validate(self, vocab_size: int) -> None:
        """The checks of src/inference/scheduler.cpp:32-63."""
        if self.max_new_tokens < 0:
            raise ValueError("max_new_tokens must be non-negative")
        if not math.isfinite(self.temperature) or self.temperature < 0.0:
            raise ValueError("sampling temperature must be finite and non-negative")
        if not 0 <= self.top_k <= vocab_size:
            raise ValueError("top_k is outside the vocabulary")
        if len(set(self.stop_tokens)) != len(self.stop_tokens):
            raise ValueError("stop tokens must be unique")
        for token in self.stop_tokens:
            if not 0 <= token < vocab_size:
                raise ValueError(f"stop token {token} is outside the vocabulary")


def uniform_for(seed: int, draw: int) -> float:
    """The uniform in [0, 1) for a request's ``draw``-th sampled token (splitmix64 finaliser, top 24 bits)."""
    z = (seed * 0x9E3779B97F4A7C15 + (draw + 1) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    z ^= z >> 31
    return (z >> 40) / float(1 << 24)


class NonFiniteLogits(RuntimeError):
    """A row of logits held NaN or infinity (the reference throws too, src/inference/scheduler.cpp:918-920)."""


class Selection:
    """Tokens that have been chosen on the device and are on their way to the host. ``device`` is the int32 tensor
    of chosen ids (a row per row of logits), which a following step may take its tokens from without waiting;
    ``tokens()`` waits for the copy and returns them, raising ``NonFiniteLogits`` for a row that held none."""

    def __init__(self, device: torch.Tensor, host: torch.Tensor, copied: "torch.cuda.Event"):
        self.device, self._host, self._copied = device, host, copied
        self._tokens = None

    def tokens(self) -> List[int]:
        if self._tokens is None:
            self._copied.synchronize()
            self._tokens = self._host.tolist()
            for row, token in enumerate(self._tokens):
                if token < 0:
                    raise NonFiniteLogits(f"row {row} of the logits is not finite")
        return self._tokens


class Sampler:
    """Selects one token per row of logits on the device; one transfer of the chosen ids back."""

    def _choose(self, logits: torch.Tensor, params: Sequence[SamplingParams], draws: Sequence[int]) -> torch.Tensor:
        if logits.shape[0] != len(params) or len(params) != len(draws):
            raise ValueError("one SamplingParams and one draw index per row of logits")
        if all(p.greedy for p in params):
            return kernels.argmax(logits)
        # one transfer for the three per-row values: temperatures, top-k counts (as int32 bits) and uniforms
        packed = np.empty((3, len(params)), dtype=np.float32)
        packed[0] = [0.0 if p.greedy else p.temperature for p in params]
        packed[1].view(np.int32)[:] = [p.top_k for p in params]
        packed[2] = [uniform_for(p.seed, d) for p, d in zip(params, draws)]
        values = on_device(packed, logits.device)
        temperature, top_k, uniform = values[0], values[1].view(torch.int32), values[2]
        if all(p.top_k == 0 for p in params):
            top_k = None      # no row is restricted: the kernel leaves its search for the k-th value out
        return kernels.sample(logits, temperature, top_k, uniform)

    def select(self, logits: torch.Tensor, params: Sequence[SamplingParams], draws: Sequence[int]) -> List[int]:
        tokens = on_host(self._choose(logits, params, draws)).tolist()
        for row, token in enumerate(tokens):
            if token < 0:
                raise NonFiniteLogits(f"row {row} of the logits is not finite")
        return tokens

    def select_later(self, logits: torch.Tensor, params: Sequence[SamplingParams], draws: Sequence[int]) -> Selection:
        """The same choice without waiting for it: the ids stay on the device for whoever steps next, and their
        copy to pinned host memory is under way when this returns."""
        chosen = self._choose(logits, params, draws)
        host = torch.empty(chosen.shape, dtype=chosen.dtype, pin_memory=True)
        host.copy_(chosen, non_blocking=True)
        count_copy_to_host(chosen)
        copied = torch.cuda.Event()
        copied.record()
        return Selection(chosen, host, copied)
