"""Timed workloads shared by ``bench.py`` and the command line: steady decoding and one prefill.

Decoding is measured the way the reference's "steady" mode is (apps/hf_infer.cpp:352-361): every
timed token runs one forward. Caches are filled with random keys and values instead of by a
prefill of the context, which changes no byte that a decode step reads or writes.
"""
from __future__ import annotations

import time
from typing import Dict

import numpy as np
import torch

from ..parts.linear import Weight
from ..sampling import Sampler, SamplingParams
from .batch import StepEntry
from .engine import Engine


def _fill_random(engine: Engine) -> None:
    for binding in engine.cache.bindings():
        if binding is not None and binding.need.paged and binding.owned:
            for tensor in binding.tensors():
                tensor.normal_(0.0, 1.0)


def decode_throughput(engine: Engine, batch: int, context: int, steps: int, warmup: int, seed: int = 0,
                      lookahead: bool = True) -> Dict[str, float]:
    """``batch`` requests that each hold ``context`` positions decode ``warmup + steps`` tokens, greedily.

    With ``lookahead`` the loop is generation's (``Scheduler(lookahead=True)``): a step takes its tokens from the
    ids that the step before chose on the device, and the host reads a step's ids while the next one runs. Without
    it the host waits for every step's ids before it builds the next step."""
    rng = np.random.default_rng(seed)
    sampler = Sampler()
    params = [SamplingParams(temperature=0.0)] * batch
    draws = [0] * batch
    ids = [("bench", batch, index) for index in range(batch)]
    for request_id in ids:
        request = engine.open(request_id)
        engine.cache.reserve(request, context)
        engine.cache.commit(request, context)
    _fill_random(engine)
    first = rng.integers(0, engine.spec.vocab_size, size=batch).tolist()

    def one_step(current):
        logits = engine.step([StepEntry(request_id, [token], [0]) for request_id, token in zip(ids, current)], borrow_logits=True)
        return sampler.select(logits, params, draws)

    def one_step_ahead(before):
        """Launches the step after ``before`` (a Selection; None: the first step), then learns ``before``'s ids."""
        if before is None:
            logits = engine.step([StepEntry(request_id, [token], [0]) for request_id, token in zip(ids, first)], borrow_logits=True)
        else:
            entries = [StepEntry(request_id, [0], [0], token_from=row) for row, request_id in enumerate(ids)]
            logits = engine.step(entries, borrow_logits=True, device_tokens=before.device)
        selection = sampler.select_later(logits, params, draws)
        if before is not None:
            before.tokens()
        return selection

    def run(count, state):
        for _ in range(count):
            state = one_step_ahead(state) if lookahead else one_step(state)
        return state

    try:
        state = run(warmup, None if lookahead else first)
        torch.cuda.synchronize()
        started = time.perf_counter()
        state = run(steps, state)
        last = state.tokens() if lookahead else state
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - started
    finally:
        for request_id in ids:
            engine.close(request_id)
    return {"tokens_per_second": batch * steps / elapsed, "ms_per_step": elapsed / steps * 1e3, "last_tokens": list(last)}


def prefill_throughput(engine: Engine, tokens: int, repeats: int = 3, seed: int = 0) -> Dict[str, float]:
    """One request's prompt of ``tokens`` ids in one step, logits at its last position, ``repeats`` times after
    two runs that warm up (the library, where it is tuned, settles its choice of algorithm over the first calls of
    a shape): the best run (``ms``, ``tokens_per_second``) and the mean of the runs (``mean_ms``)."""
    rng = np.random.default_rng(seed)
    prompt = rng.integers(0, engine.spec.vocab_size, size=tokens).tolist()
    times = []
    warmup = 2
    for repeat in range(repeats + warmup):
        request_id = ("prefill", repeat)
        engine.open(request_id)
        torch.cuda.synchronize()
        started = time.perf_counter()
        logits = engine.step([StepEntry(request_id, prompt, [tokens - 1])])
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - started
        engine.close(request_id)
        assert torch.isfinite(logits).all()
        if repeat >= warmup:
            times.append(elapsed)
    best, mean = min(times), sum(times) / len(times)
    return {"tokens_per_second": tokens / best, "ms": best * 1e3, "mean_ms": mean * 1e3, "mean_tokens_per_second": tokens / mean,
            "all_ms": [round(elapsed * 1e3, 3) for elapsed in times]}


def weight_bytes(engine: Engine) -> int:
    """Bytes of every weight a decode step reads once: all layers, the final norm and the head (an embedding
    table that is not the head's is read one row per token, which is counted apart). A matrix counts once,
    at its own size, whichever of its copies (as stored, packed) the step reads."""
    model = engine.model
    total = 0
    seen = set()

    def count(value) -> int:
        if isinstance(value, Weight):
            kept = value.tensor if value.tensor is not None else value.packed
            if kept.data_ptr() in seen:
                return 0
            seen.add(kept.data_ptr())
            return value.out_features * value.in_features * kept.element_size()
        if isinstance(value, torch.Tensor):
            if value.data_ptr() in seen:
                return 0
            seen.add(value.data_ptr())
            return value.numel() * value.element_size()
        return 0

    total += count(model.final_norm.weight) + count(model.head.weight)
    for block in model.blocks:
        for part in block.parts():
            for piece in (part, *part.sub_parts()):
                total += sum(count(value) for value in vars(piece).values())
    return total


def step_bytes(engine: Engine, batch: int, context: int) -> int:
    """What a decode step has to read: every weight once, the cache of the live requests, one embedding row each."""
    cache = 0
    for group in engine.cache.groups:
        visible = context if group.need.window is None else min(context, group.need.window)
        cache += len(group.entries) * visible * group.need.bytes_per_position(engine.dtype)
    cache += engine.cache.state_bytes() // engine.cache.max_requests
    return weight_bytes(engine) + batch * cache + engine.model.embedding.bytes_read(batch, context)


def step_flops(engine: Engine, tokens: int) -> float:
    """Floating-point operations of one prompt of ``tokens`` ids: 2 per multiply-add of every matrix product over
    all tokens (the head for one row) and of causal attention (scores and values)."""
    flops = sum(part.flops(tokens) for block in engine.model.blocks for part in block.parts())
    return flops + engine.model.head.flops(tokens, wanted=1)


def percentile(values, quantile: float) -> float:
    """Linear interpolation between the two nearest of the sorted values (apps/hf_infer.cpp:570-580)."""
    ordered = sorted(values)
    position = quantile * (len(ordered) - 1)
    lower = int(position)
    upper = min(lower + 1, len(ordered) - 1)
    fraction = position - lower
    return ordered[lower] * (1.0 - fraction) + ordered[upper] * fraction


def serving_throughput(engine: Engine, requests: int = 64, prompt_range=(128, 2048), new_tokens: int = 256,
                       prefill_chunk: int = 512, max_batched_tokens: int = 2048, runs: int = 3, warmup: int = 1,
                       seed: int = 0) -> Dict[str, float]:
    """The reference's continuous-batching workload (apps/hf_infer.cpp:862-900): ``requests`` prompts of
    uniform-random lengths, all there at step 0, ``new_tokens`` greedy tokens each, through the scheduler.
    The whole workload runs ``warmup`` times untimed and ``runs`` times timed; every run must give the same tokens.
    Returns generated tokens a second and the latencies of the last run."""
    from .generate import generate
    rng = np.random.default_rng(seed)
    lengths = rng.integers(prompt_range[0], prompt_range[1] + 1, size=requests)
    prompts = [rng.integers(0, engine.spec.vocab_size, size=int(length)).tolist() for length in lengths]
    params = SamplingParams(max_new_tokens=new_tokens, temperature=0.0)

    def run_once():
        return generate(engine, prompts, params, max_batched_tokens=max_batched_tokens, prefill_chunk=prefill_chunk,
                        return_scheduler=True)

    for _ in range(warmup):
        run_once()
    torch.cuda.synchronize()
    elapsed, outputs, scheduler = 0.0, None, None
    for _ in range(runs):
        started = time.perf_counter()
        current, scheduler = run_once()
        torch.cuda.synchronize()
        elapsed += time.perf_counter() - started
        if outputs is not None and current != outputs:
            raise RuntimeError("continuous generation changed across measured runs")
        outputs = current
    generated = sum(len(output) - len(prompt) for output, prompt in zip(outputs, prompts))
    served = [scheduler.request(index) for index in range(requests)]
    ttft = [(r.first_token_time - r.submit_time) * 1e3 for r in served]
    completion = [(r.completion_time - r.submit_time) * 1e3 for r in served]
    metrics = scheduler.metrics
    return {"tokens_per_second": generated * runs / elapsed, "ms_per_run": elapsed / runs * 1e3,
            "generated_tokens": generated, "prompt_tokens": int(lengths.sum()),
            "model_tokens_per_second": (generated + int(lengths.sum())) * runs / elapsed,
            "scheduler_steps": metrics.scheduler_steps, "preemptions": metrics.preemptions,
            "ttft_p50_ms": percentile(ttft, 0.5), "ttft_p95_ms": percentile(ttft, 0.95),
            "completion_p50_ms": percentile(completion, 0.5), "completion_p95_ms": percentile(completion, 0.95),
            "graph_replays": engine.graph_replays, "mixed_graph_replays": engine.mixed_graph_replays,
            "graphs_captured": engine.graphs_captured}
