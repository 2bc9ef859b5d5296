"""Builders of replay traces (the JSON lines bin/trace_run reads) and the comparison with the plain implementation."""
from __future__ import annotations

import io
import json
import os
from typing import Dict, List, Sequence, Tuple

import numpy as np

import plain_qwen2 as plain


def round_up(value: int, multiple: int) -> int:
    return -(-value // multiple) * multiple


def whole(requests: Dict[str, List[int]]) -> List[dict]:
    """Each request alone and whole: one step each, every position wanted."""
    return [{"step": index, "entries": [{"id": rid, "tokens": tokens, "want": list(range(len(tokens)))}], "end": [rid]}
            for index, (rid, tokens) in enumerate(requests.items())]


def prefill_then_decode(rid: str, tokens: List[int], tail: int = 32) -> List[dict]:
    """Most of it in one step, the last ``tail`` tokens one by one."""
    head = len(tokens) - tail
    steps = [{"step": 0, "entries": [{"id": rid, "tokens": tokens[:head], "want": list(range(head))}], "end": []}]
    for index in range(tail):
        steps.append({"step": index + 1, "entries": [{"id": rid, "tokens": [tokens[head + index]], "want": [0]}],
                      "end": [rid] if index == tail - 1 else []})
    return steps


def portions(rid: str, tokens: List[int], sizes: Sequence[int]) -> List[dict]:
    """Portions of changing size; ``sizes`` is cycled until the tokens are used up."""
    steps, position, index = [], 0, 0
    while position < len(tokens):
        count = min(sizes[index % len(sizes)], len(tokens) - position)
        steps.append({"step": index, "entries": [{"id": rid, "tokens": tokens[position:position + count],
                                                  "want": list(range(count))}], "end": []})
        position += count
        index += 1
    steps[-1]["end"] = [rid]
    return steps


def mixed(requests: Dict[str, List[int]], seed: int, max_live: int = 4, decode_tail: int = 12,
          max_portion: int = 17) -> Tuple[List[dict], int]:
    """Up to ``max_live`` live requests: portions of some beside decoded tokens of others, some left out of a
    step now and then; a request that ends makes room for the next. Returns the steps and the most tokens
    live requests hold at any time (each rounded up to 64): a pool of that size makes pages be used again."""
    rng = np.random.default_rng(seed)
    waiting = list(requests.items())
    live: Dict[str, int] = {}       # id -> tokens fed
    steps: List[dict] = []
    peak = 0
    while waiting or live:
        while waiting and len(live) < max_live and (not live or rng.integers(0, 3) > 0):
            rid, _ = waiting.pop(0)
            live[rid] = 0
        entries, ended = [], []
        for rid in list(live):
            tokens = requests[rid]
            fed = live[rid]
            if len(live) > 1 and rng.integers(0, 5) == 0:
                continue                                  # left out of this step, goes on later
            remaining = len(tokens) - fed
            if remaining <= decode_tail:
                count = 1                                 # a decoded token, given not sampled
            else:
                count = int(min(rng.integers(2, max_portion + 1), remaining - decode_tail))
                if count < 2:
                    count = min(2, remaining)
            entries.append({"id": rid, "tokens": tokens[fed:fed + count], "want": list(range(count))})
            live[rid] = fed + count
            if live[rid] == len(tokens):
                ended.append(rid)
        if not entries:
            continue
        peak = max(peak, sum(round_up(count, 64) for count in live.values()))
        for rid in ended:
            del live[rid]
        steps.append({"step": len(steps), "entries": entries, "end": ended})
    return steps, peak


def to_lines(steps: List[dict]) -> str:
    return "".join(json.dumps(step) + "\n" for step in steps)


def collect(steps: List[dict], out_dir: str, vocab: int) -> Dict[Tuple[str, int], np.ndarray]:
    """Read the <step>.f32 files back: logits by (request, position)."""
    fed: Dict[str, int] = {}
    out: Dict[Tuple[str, int], np.ndarray] = {}
    for step in steps:
        wanted = [(entry["id"], fed.get(entry["id"], 0) + place) for entry in step["entries"] for place in entry["want"]]
        for entry in step["entries"]:
            fed[entry["id"]] = fed.get(entry["id"], 0) + len(entry["tokens"])
        for rid in step["end"]:
            fed.pop(rid, None)
        path = os.path.join(out_dir, f"{step['step']}.f32")
        if not wanted:
            assert not os.path.exists(path)
            continue
        rows = np.fromfile(path, dtype="<f4").reshape(len(wanted), vocab)
        for key, row in zip(wanted, rows):
            assert key not in out
            out[key] = row
    return out


class PlainModel:
    """The plain implementation on a model folder; logits of whole sequences, cached by token tuple."""

    def __init__(self, folder: str):
        self.config = plain.read_config(folder)
        self.weights = plain.read_safetensors(os.path.join(folder, "model.safetensors"))
        self._cache: Dict[tuple, np.ndarray] = {}

    def logits(self, tokens: Sequence[int]) -> np.ndarray:
        key = tuple(tokens)
        if key not in self._cache:
            for known, rows in self._cache.items():     # causal: a prefix's logits are the first rows of the longer run
                if len(known) > len(key) and known[:len(key)] == key:
                    return rows[:len(key)]
            self._cache[key] = plain.forward(self.config, self.weights, list(tokens))
        return self._cache[key]


# Tolerances, relative to the scale of a request's logits (largest magnitude for "max", root mean square for
# "rms", the error of one row of logits). float32: the engine sums in float32 where the plain implementation sums
# in float64; a few 1e-6 are seen, the bound leaves one order of magnitude. bfloat16: what the engine must round
# to 8 bits of mantissa (the inputs of every matrix product, keys, values, attention outputs) was rounded at the
# same places in the float64 plain implementation; on these models that alone gives a worst row of 1.4e-2 to
# 2.1e-2 rms and 1.1e-2 to 1.6e-2 max. The bounds are twice that: an engine within them adds no error of its own
# that is larger than the format's.
TOLERANCE = {"float32": {"max": 2e-5, "rms": 2e-5}, "bfloat16": {"max": 3.5e-2, "rms": 4.5e-2}}


def compare(got: Dict[Tuple[str, int], np.ndarray], requests: Dict[str, List[int]], model: PlainModel, dtype: str,
            expect_all: bool = True) -> Tuple[float, float]:
    """Every row against the plain implementation; returns (worst max error, worst rms error), both relative
    to the request's logit scale. Names the first wrong (request, position) when a bound is passed."""
    bound = TOLERANCE[dtype]
    worst_max = worst_rms = 0.0
    if expect_all:
        assert set(got) == {(rid, p) for rid, tokens in requests.items() for p in range(len(tokens))}
    for rid, tokens in requests.items():
        reference = model.logits(tokens)
        scale = np.abs(reference).max()
        rms_scale = np.sqrt(np.mean(reference ** 2))
        for position in range(len(tokens)):
            if (rid, position) not in got:
                continue
            row = got[(rid, position)].astype(np.float64)
            assert np.all(np.isfinite(row)), f"request {rid} position {position}: logits are not finite"
            error_max = np.abs(row - reference[position]).max() / scale
            error_rms = np.sqrt(np.mean((row - reference[position]) ** 2)) / rms_scale
            assert error_max <= bound["max"] and error_rms <= bound["rms"], (
                f"{dtype}: first wrong row is request {rid} position {position} of {len(tokens)}: "
                f"max error {error_max:.3e} (bound {bound['max']:.1e}), rms error {error_rms:.3e} (bound {bound['rms']:.1e})")
            worst_max, worst_rms = max(worst_max, error_max), max(worst_rms, error_rms)
    return worst_max, worst_rms
