"""Builders of replay traces (the JSON lines bin/trace_run reads) and the comparison with the plain implementation."""
from __future__ import annotations

import io
import json
import os
from typing import Dict, List, Sequence, Tuple

import numpy as np

import plain_qwen2 as plain
import plain_rounded


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
        self._rounded: Dict[tuple, np.ndarray] = {}

    def logits(self, tokens: Sequence[int]) -> np.ndarray:
        key = tuple(tokens)
        if key not in self._cache:
            for known, rows in self._cache.items():     # causal: a prefix's logits are the first rows of the longer run
                if len(known) > len(key) and known[:len(key)] == key:
                    return rows[:len(key)]
            self._cache[key] = plain.forward(self.config, self.weights, list(tokens))
        return self._cache[key]


    def rounded_logits(self, tokens: Sequence[int], rows: "plain_rounded.Rows", twin: bool = False) -> np.ndarray:
        """The plain run with a bfloat16 engine's roundings (``plain_rounded``), every position flagged by ``rows``;
        with ``twin`` the same made in another, equally valid way."""
        key = (tuple(tokens), rows.split_norm.tobytes(), rows.round_gate_up.tobytes(), twin)
        if key not in self._rounded:
            self._rounded[key] = plain_rounded.forward(self.config, self.weights, list(tokens), rows,
                                                       plain_rounded.Twin(seed=1) if twin else None)
        return self._rounded[key]


def rows_of_positions(steps: List[dict]) -> Dict[str, List[int]]:
    """For every request of a trace, the number of rows (tokens of all its requests) of the step that ran each of
    its positions."""
    out: Dict[str, List[int]] = {}
    for step in steps:
        rows = sum(len(entry["tokens"]) for entry in step["entries"])
        for entry in step["entries"]:
            out.setdefault(entry["id"], []).extend([rows] * len(entry["tokens"]))
    return out


def roundings(step_rows: Sequence[int], one_weight_copy: bool = False) -> "plain_rounded.Rows":
    """How the engine rounds a position that ran in a step of so many rows: up to ``SKINNY_ROWS`` rows its
    products take the norms between them apart; gate and up are rounded before SiLU where the library multiplies
    (more than ``MEDIUM_GATED_ROWS`` rows, and a copy of the weights as stored to multiply with)."""
    from microllm_rocm_amd.parts.linear import MEDIUM_GATED_ROWS, SKINNY_ROWS
    rows = np.asarray(step_rows)
    return plain_rounded.Rows(split_norm=rows <= SKINNY_ROWS,
                              round_gate_up=(rows > MEDIUM_GATED_ROWS) & (not one_weight_copy))


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


# Against the plain run that rounds where a bfloat16 engine must (``plain_rounded``) an engine's error is no longer
# the format's but its own arithmetic's. How small that can be is a property of the model, not of the engine: the
# attention's probabilities are rounded against whatever maximum a kernel has seen so far, which no whole-sequence
# run can follow, and after the first layer any difference of that size moves most later roundings to other
# steps of the grid. ``plain_rounded.Twin`` makes the same roundings in another, equally valid way; how far its
# logits lie from the rounded run's is how far two faithful bfloat16 implementations of this model lie apart
# (weights N(0, 0.02): 2e-3 to 5e-3 of the logits' scale; the sharp models: 1e-2 to 1.5e-2, which is the distance to
# the exact run too). An engine is held to that: no row further than ``ROW_FACTOR`` times the twin's worst row, and
# the error over all rows of a request no more than ``ALL_ROWS_FACTOR`` times the twin's.
ROW_FACTOR = 1.5
ALL_ROWS_FACTOR = 1.0


def compare_rounded(got: Dict[Tuple[str, int], np.ndarray], requests: Dict[str, List[int]], steps: List[dict],
                    model: PlainModel, one_weight_copy: bool = False) -> Tuple[float, float]:
    """Every row of a bfloat16 engine against the plain run with the same roundings, in units of the distance
    between that run and its twin; returns (worst row's max error, worst request's error over all rows) in those
    units."""
    step_rows = rows_of_positions(steps)
    worst_row = worst_request = 0.0
    for rid, tokens in requests.items():
        if rid not in step_rows:
            continue
        assert len(step_rows[rid]) == len(tokens)
        flags = roundings(step_rows[rid], one_weight_copy)
        reference = model.rounded_logits(tokens, flags)
        twin = model.rounded_logits(tokens, flags, twin=True) - reference
        places = [position for position in range(len(tokens)) if (rid, position) in got]
        if not places:
            continue
        difference = np.stack([got[(rid, position)] for position in places]).astype(np.float64) - reference[places]
        twin_max = np.abs(twin).max()                              # worst element of the twin's worst row
        twin_rms = np.sqrt(np.mean(twin ** 2, axis=1)).max()       # worst row of the twin
        twin_all = np.sqrt(np.mean(twin[places] ** 2))
        row_max = np.abs(difference).max(axis=1)
        row_rms = np.sqrt(np.mean(difference ** 2, axis=1))
        for index, position in enumerate(places):
            assert row_max[index] <= ROW_FACTOR * twin_max and row_rms[index] <= ROW_FACTOR * twin_rms, (
                f"bfloat16 against the rounded plain run: first wrong row is request {rid} position {position} of "
                f"{len(tokens)}: max error {row_max[index] / twin_max:.2f}, rms error {row_rms[index] / twin_rms:.2f} "
                f"times the twin's worst (bound {ROW_FACTOR})")
        overall = np.sqrt(np.mean(difference ** 2)) / twin_all
        assert overall <= ALL_ROWS_FACTOR, (f"bfloat16 against the rounded plain run: request {rid}: the error over all "
                                            f"rows is {overall:.2f} times the twin's (bound {ALL_ROWS_FACTOR})")
        worst_row = max(worst_row, float((row_max / twin_max).max()), float((row_rms / twin_rms).max()))
        worst_request = max(worst_request, float(overall))
    return worst_row, worst_request
