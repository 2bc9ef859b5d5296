"""The command line, in the manner of the reference's ``microllm_hf_infer`` (apps/hf_infer.cpp:32-73, 75-286):
``--name value`` pairs, booleans as ``true|false``, an unknown option is an error, one JSON object on
standard output. Options the reference has keep their names and meanings; what this engine adds
(``--model``, ``--dtype``, sampling, pages, the token budget) follows the same style.

    microllm_hf_infer --config DIR/config.json --weights DIR/model.safetensors --tokens 1,2,3 \\
                      --device hip --new-tokens 16

``--use-cache false`` generates by running every sequence whole for each new token (the reference's oracle for
its cached path), ``--cache-prefill-mode token`` feeds the prompt one token a step, ``--prefill-logits full`` computes
the logits of every prompt position, ``--batch-argmax-mode host`` picks tokens from logits copied to the host,
``--cache-logits-output`` writes the last decode step's logits, ``--bf16-ffn`` with ``--bf16-attention``
choose the precision as ``--dtype`` does (apps/hf_infer.cpp:52-57, 1121-1123, 1238-1305), and ``--trace-output``
writes a value trace of one prefill, a JSON line per layer and one for the logits (apps/hf_infer.cpp:1132-1160).

Workloads (``--workload``): ``prefill`` times the prompt alone, ``decode`` times steady decoding after it,
``both`` (default) generates ``--new-tokens`` tokens after the prompt, ``continuous`` serves several requests
whose prompts are cyclic slices of the given token ids (apps/hf_infer.cpp:845-861), arriving at given steps.
"""
from __future__ import annotations

import json
import math
import os
import sys
import time
from typing import Dict, List, Optional

OPTIONS: Dict[str, object] = {
    # the reference's options
    "config": None, "weights": None, "tokens": "", "device": "hip", "top-k": 10, "logits-output": None,
    "new-tokens": 0, "warmup": 0, "steps": 1, "prefill-warmup": 0, "prefill-steps": 1, "workload": "both",
    "batch": 1, "decode-mode": "generation", "kv-cache-dtype": None, "cache-capacity": 0,
    "continuous-slots": 0, "continuous-prompt-lengths": "", "continuous-new-token-lengths": "",
    "continuous-prompt-offsets": "", "continuous-arrival-steps": "",
    "use-cache": "true", "cache-prefill-mode": "full", "prefill-logits": "last", "batch-argmax-mode": "device",
    "cache-logits-output": None, "bf16-ffn": None, "bf16-attention": None,
    "trace-output": None, "trace-max-elements": 4096,
    # this engine's own
    "model": None, "dtype": "bfloat16", "temperature": 0.0, "sample-top-k": 0, "seed": 1, "stop-tokens": "",
    "block-size": 16, "num-blocks": 0, "max-batched-tokens": 2048, "prefill-chunk": 512, "max-requests": 64,
    "random-config": None, "prompt-lengths": "", "prompt-seed": 0, "use-graphs": "true", "weight-copies": "auto",
    "tune-library": "false",
}


class UsageError(Exception):
    pass


def parse(argv: List[str]) -> Dict[str, object]:
    options = dict(OPTIONS)
    index = 0
    while index < len(argv):
        name = argv[index]
        if not name.startswith("--") or name[2:] not in OPTIONS:
            raise UsageError(f"unknown option {name}")
        if index + 1 >= len(argv):
            raise UsageError(f"option {name} needs a value")
        key, text = name[2:], argv[index + 1]
        default = OPTIONS[key]
        try:
            if isinstance(default, bool) or isinstance(default, str) or default is None:
                options[key] = text
            elif isinstance(default, int):
                options[key] = int(text)
            elif isinstance(default, float):
                options[key] = float(text)
        except ValueError:
            raise UsageError(f"option {name} needs a number, got {text!r}") from None
        index += 2
    return options


def percentile(values, quantile: float) -> float:
    """Linear interpolation between the two nearest of the sorted values (apps/hf_infer.cpp:570-580)."""
    if not values or not 0.0 <= quantile <= 1.0:
        raise ValueError("percentile input is invalid")
    ordered = sorted(values)
    position = quantile * (len(ordered) - 1)
    lower, upper = int(math.floor(position)), int(math.ceil(position))
    fraction = position - lower
    return ordered[lower] * (1.0 - fraction) + ordered[upper] * fraction


def trace_record(sequence: int, kind: str, name: str, tensor, max_elements: int) -> dict:
    """One record of the value trace: what the tensor is, its statistics and its first values, with the reference's
    field names (src/profiling/trace.cpp:156-196; include/microllm/profiling/trace.h:25-47)."""
    import torch
    values = tensor.detach().to(torch.float64).flatten()
    finite = values[torch.isfinite(values)]
    some = finite.numel() > 0
    first = values[:max_elements].cpu().tolist()
    return {"schema_version": 1, "framework": "microllm_rocm_amd", "run_id": "hf-prefill", "phase": "inference-values",
            "sequence": sequence, "iteration": 0, "kind": kind, "name": name, "shape": list(tensor.shape),
            "dtype": str(tensor.dtype).replace("torch.", ""), "device": str(tensor.device), "wall_ms": 0.0,
            "statistics": {"numel": values.numel(), "finite_count": finite.numel(),
                           "minimum": float(finite.min()) if some else 0.0, "maximum": float(finite.max()) if some else 0.0,
                           "mean": float(finite.mean()) if some else 0.0, "l2_norm": float(finite.square().sum().sqrt())},
            "values_truncated": values.numel() > max_elements,
            "values": [value if math.isfinite(value) else ("nan" if math.isnan(value) else ("inf" if value > 0 else "-inf"))
                       for value in first]}


def write_trace(path: str, records: List[dict]) -> None:
    folder = os.path.dirname(path)
    if folder:
        os.makedirs(folder, exist_ok=True)
    with open(path, "w", encoding="utf-8") as handle:
        for record in records:
            handle.write(json.dumps(record) + "\n")


def integers(text: str, what: str) -> List[int]:
    if not text:
        return []
    try:
        values = [int(piece) for piece in text.split(",")]
    except ValueError:
        raise UsageError(f"{what} must be comma-separated integers") from None
    if any(value < 0 for value in values):
        raise UsageError(f"{what} must be non-negative")
    return values


def boolean(text: str, what: str) -> bool:
    if text not in ("true", "false"):
        raise UsageError(f"{what} must be true or false")
    return text == "true"


def main(argv: Optional[List[str]] = None) -> int:
    argv = list(sys.argv[1:] if argv is None else argv)
    if argv and argv[0] in ("-h", "--help"):
        print(__doc__)
        print("options: " + " ".join(f"--{name}" for name in OPTIONS))
        return 0
    try:
        options = parse(argv)
        return run(options)
    except UsageError as error:
        print(f"microllm_hf_infer: {error}", file=sys.stderr)
        return 2


def run(options: Dict[str, object]) -> int:
    if options["device"] != "hip":
        raise UsageError("this engine runs on --device hip only")
    if options["workload"] not in ("both", "prefill", "decode", "continuous"):
        raise UsageError("--workload must be both, prefill, decode or continuous")
    model_dir = options["model"]
    if model_dir is None and options["config"] is not None:
        model_dir = os.path.dirname(os.path.abspath(str(options["config"])))
        if options["weights"] is not None and os.path.dirname(os.path.abspath(str(options["weights"]))) != model_dir:
            raise UsageError("--config and --weights must lie in one model folder")
    if model_dir is None and options["random-config"] is None:
        raise UsageError("give --model DIR, --config and --weights, or --random-config FILE")
    dtype = str(options["dtype"])
    # The reference keeps its weights in 32-bit unless --bf16-ffn and --bf16-attention say otherwise
    # (apps/hf_infer.cpp:52-53); this engine has one precision for all: both switches together choose it.
    switches = {name: boolean(str(options[name]), f"--{name}") for name in ("bf16-ffn", "bf16-attention") if options[name] is not None}
    if switches:
        if len(switches) != 2 or len(set(switches.values())) != 1:
            raise UsageError("this engine has one precision: give --bf16-ffn and --bf16-attention the same value, or use --dtype")
        dtype = "bfloat16" if switches["bf16-ffn"] else "float32"
    use_cache = boolean(str(options["use-cache"]), "--use-cache")
    for name, allowed in (("cache-prefill-mode", ("full", "token")), ("prefill-logits", ("last", "full")),
                          ("batch-argmax-mode", ("device", "host"))):
        if options[name] not in allowed:
            raise UsageError(f"--{name} must be {' or '.join(allowed)}")      # apps/hf_infer.cpp:194-202
    if int(options["trace-max-elements"]) <= 0:
        raise UsageError("--trace-max-elements must be positive")      # apps/hf_infer.cpp:265-266
    if options["trace-output"] and (options["workload"] != "prefill" or int(options["prefill-warmup"]) != 0
                                    or int(options["prefill-steps"]) != 1):
        raise UsageError("--trace-output requires prefill workload, zero prefill warmup, and one prefill step")   # :268-272
    if options["workload"] == "continuous" and not use_cache:
        raise UsageError("the continuous workload needs --use-cache true")      # apps/hf_infer.cpp:241
    if options["cache-logits-output"] and (not use_cache or options["workload"] == "prefill" or int(options["new-tokens"]) < 2):
        raise UsageError("--cache-logits-output needs --use-cache true, a workload with decoding and "
                         "--new-tokens of at least 2")                          # apps/hf_infer.cpp:280-284
    if options["kv-cache-dtype"] is not None and options["kv-cache-dtype"] not in ("fp32", "bf16"):
        raise UsageError("--kv-cache-dtype must be fp32 or bf16")
    if dtype in ("fp32",):
        dtype = "float32"
    if dtype in ("bf16",):
        dtype = "bfloat16"
    if options["kv-cache-dtype"] is not None and {"fp32": "float32", "bf16": "bfloat16"}[str(options["kv-cache-dtype"])] != dtype:
        raise UsageError("the cache has the engine's dtype: --kv-cache-dtype must agree with --dtype")

    import numpy as np
    import torch
    from .. import Engine, GenerationConfig, Scheduler, generate
    from ..config import load_config
    from ..engine.benchmark import decode_throughput, prefill_throughput
    from ..engine.batch import StepEntry
    from ..ops.transfers import on_host, reset_transfer_stats, transfer_stats

    tokens = integers(str(options["tokens"]), "--tokens")
    prompt_lengths = integers(str(options["prompt-lengths"]), "--prompt-lengths")
    batch = int(options["batch"])
    new_tokens = int(options["new-tokens"])
    block_size = int(options["block-size"])
    started = time.perf_counter()

    continuous = options["workload"] == "continuous"
    if continuous:
        lengths = integers(str(options["continuous-prompt-lengths"]), "--continuous-prompt-lengths")
        new_lengths = integers(str(options["continuous-new-token-lengths"]), "--continuous-new-token-lengths")
        arrivals = integers(str(options["continuous-arrival-steps"]), "--continuous-arrival-steps") or [0] * len(lengths)
        offsets = integers(str(options["continuous-prompt-offsets"]), "--continuous-prompt-offsets") or [0] * len(lengths)
        if not lengths or not (len(lengths) == len(new_lengths) == len(arrivals) == len(offsets)):
            raise UsageError("continuous lengths, new-token lengths, arrival steps and offsets must match in count")
        needed = sum(-(-(a + b) // block_size) * block_size for a, b in zip(lengths, new_lengths))
    else:
        needed = batch * (-(-(max(len(tokens), max(prompt_lengths, default=0)) + new_tokens + int(options["steps"])
                               + int(options["warmup"])) // block_size) + 1) * block_size
    capacity = int(options["cache-capacity"])
    num_blocks = int(options["num-blocks"]) or None
    max_tokens = None if num_blocks else max(needed, capacity * batch, block_size)
    engine_options = dict(dtype=dtype, device="cuda:0", page_size=block_size, max_tokens=max_tokens, num_pages=num_blocks,
                          max_requests=max(int(options["max-requests"]), batch),
                          use_graphs=boolean(str(options["use-graphs"]), "--use-graphs"),
                          weight_copies=str(options["weight-copies"]),
                          tune_library=boolean(str(options["tune-library"]), "--tune-library"),
                          max_portion=int(options["prefill-chunk"]) if continuous else None)
    if model_dir is not None:
        engine = Engine.from_folder(str(model_dir), **engine_options)
    else:
        architecture, config = load_config(str(options["random-config"]))
        engine = Engine.from_random(config, seed=int(options["seed"]), on_device=True, **engine_options)
    load_ms = (time.perf_counter() - started) * 1e3
    vocab = engine.spec.vocab_size
    if not tokens and prompt_lengths:
        rng = np.random.default_rng(int(options["prompt-seed"]))
        tokens = rng.integers(0, vocab, size=prompt_lengths[0]).tolist()
    if not tokens:
        raise UsageError("give --tokens a,b,c or --prompt-lengths N with --prompt-seed")

    report = {"schema_version": 1, "device": "hip", "device_name": torch.cuda.get_device_name(0),
              "architecture": engine.spec.architecture, "compute_dtype": dtype, "workload": options["workload"],
              "load_ms": round(load_ms, 3), "token_count": len(tokens), "batch": batch,
              "kv_block_size": block_size, "kv_blocks": engine.cache.groups[0].pool.num_pages if engine.cache.groups else 0,
              "allocated_cache_bytes": engine.cache.allocated_bytes(), "weight_copies": engine.weight_copies}
    stop_tokens = tuple(integers(str(options["stop-tokens"]), "--stop-tokens"))

    def measured_transfers() -> dict:
        """Copies between host and device since the engine was loaded, warm-up runs included, under the reference's
        keys (apps/hf_infer.cpp:1001-1012, 1407-1418)."""
        moved = transfer_stats()
        return {"measured_h2d_calls": moved.host_to_device_calls, "measured_h2d_bytes": moved.host_to_device_bytes,
                "measured_d2h_calls": moved.device_to_host_calls, "measured_d2h_bytes": moved.device_to_host_bytes,
                "measured_d2d_calls": moved.device_to_device_calls, "measured_d2d_bytes": moved.device_to_device_bytes}

    reset_transfer_stats()
    params = GenerationConfig(max_new_tokens=new_tokens, temperature=float(options["temperature"]),
                              top_k=int(options["sample-top-k"]), seed=int(options["seed"]), stop_tokens=stop_tokens)

    if continuous:
        prompts = [[tokens[(index + offset) % len(tokens)] for index in range(length)]
                   for length, offset in zip(lengths, offsets)]
        per_request = [GenerationConfig(max_new_tokens=new, temperature=params.temperature, top_k=params.top_k,
                                        seed=params.seed + index, stop_tokens=stop_tokens)
                       for index, new in enumerate(new_lengths)]
        slots = int(options["continuous-slots"]) or None

        def run_once():
            return generate(engine, prompts, per_request, max_batched_tokens=int(options["max-batched-tokens"]),
                            prefill_chunk=int(options["prefill-chunk"]), max_requests=slots,
                            arrival_steps=arrivals, return_scheduler=True)

        # The whole workload runs --warmup times untimed and --steps times timed; every timed run must generate the
        # same tokens (apps/hf_infer.cpp:862-900).
        torch.cuda.synchronize()
        begun = time.perf_counter()
        for _ in range(int(options["warmup"])):
            run_once()
        torch.cuda.synchronize()
        warmup_ms = (time.perf_counter() - begun) * 1e3
        elapsed, outputs, scheduler = 0.0, None, None
        for _ in range(max(1, int(options["steps"]))):
            begun = time.perf_counter()
            current, scheduler = run_once()
            torch.cuda.synchronize()
            elapsed += time.perf_counter() - begun
            if outputs is not None and current != outputs:
                raise RuntimeError("continuous generation changed across measured runs")
            outputs = current
        generated = [output[len(prompt):] for output, prompt in zip(outputs, prompts)]
        metrics = scheduler.metrics
        requests = [scheduler.request(index) for index in range(len(prompts))]
        report.update({
            "request_count": len(prompts), "continuous_slots": slots or engine.cache.max_requests,
            "prompt_lengths": lengths, "new_token_lengths": new_lengths, "arrival_steps": arrivals, "prompt_offsets": offsets,
            "warmup": int(options["warmup"]), "steps": max(1, int(options["steps"])), "warmup_ms": round(warmup_ms, 3),
            "measured_ms": round(elapsed * 1e3, 3), "measured_tokens": sum(len(g) for g in generated) * max(1, int(options["steps"])),
            "tokens_per_second": round(sum(len(g) for g in generated) * max(1, int(options["steps"])) / elapsed, 3),
            "scheduler_steps": metrics.scheduler_steps, "slot_admissions": metrics.admissions,
            "preemptions": metrics.preemptions, "prefill_tokens": metrics.prefill_tokens, "decode_tokens": metrics.decode_tokens,
            "completed_requests": metrics.completed_requests, "peak_active_requests": metrics.peak_active_requests,
            "peak_active_cache_bytes": metrics.peak_held_pages * (engine.cache.allocated_bytes() // max(1, report["kv_blocks"])),
            "request_ttft_ms": [round((r.first_token_time - r.submit_time) * 1e3, 3) for r in requests],
            "request_completion_ms": [round((r.completion_time - r.submit_time) * 1e3, 3) for r in requests],
            "request_ttft_p50_ms": round(percentile([(r.first_token_time - r.submit_time) * 1e3 for r in requests], 0.50), 3),
            "request_ttft_p95_ms": round(percentile([(r.first_token_time - r.submit_time) * 1e3 for r in requests], 0.95), 3),
            "request_completion_p50_ms": round(percentile([(r.completion_time - r.submit_time) * 1e3 for r in requests], 0.50), 3),
            "request_completion_p95_ms": round(percentile([(r.completion_time - r.submit_time) * 1e3 for r in requests], 0.95), 3),
            "kv_cache_byte_utilization": round(metrics.peak_held_pages / max(1, report["kv_blocks"]), 4),
            "generated": generated, "token_checksum": int(sum((i + 1) * t for g in generated for i, t in enumerate(g)) % (1 << 31)),
        })
        report.update(measured_transfers())
        print(json.dumps(report), flush=True)
        return 0

    prompts = [list(tokens) for _ in range(batch)]
    if options["workload"] in ("prefill", "both"):
        timings = []
        logits = None
        for iteration in range(int(options["prefill-warmup"]) + int(options["prefill-steps"])):
            ids = [("prefill", iteration, row) for row in range(batch)]
            for request_id in ids:
                engine.open(request_id)
            torch.cuda.synchronize()
            begun = time.perf_counter()
            # --prefill-logits full: the logits of every position are computed, last: of the last alone; the
            # report and --logits-output take the last row either way (apps/hf_infer.cpp:1121-1123, 1166-1181)
            every = options["prefill-logits"] == "full"
            records = []
            if options["trace-output"]:
                engine.observe_layers(lambda index, stream: records.append(trace_record(
                    len(records), "layer", f"run_entry.{index}", stream.view(batch, len(tokens), -1), int(options["trace-max-elements"]))))
            logits = engine.step([StepEntry(request_id, prompt, list(range(len(prompt))) if every else [len(prompt) - 1])
                                  for request_id, prompt in zip(ids, prompts)])
            if every:
                logits = logits.view(batch, len(tokens), -1)[:, -1]
            torch.cuda.synchronize()
            if options["trace-output"]:
                engine.observe_layers(None)
                records.append(trace_record(len(records), "model", "logits", logits, int(options["trace-max-elements"])))
                write_trace(str(options["trace-output"]), records)
                report["trace_records"] = len(records)
            if iteration >= int(options["prefill-warmup"]):
                timings.append(time.perf_counter() - begun)
            for request_id in ids:
                engine.close(request_id)
        report["prefill_ms"] = round(min(timings) * 1e3, 3)
        report["prefill_tokens_per_second"] = round(batch * len(tokens) / min(timings), 3)
        last = on_host(logits[0]).numpy()
        top = np.argsort(-last, kind="stable")[:int(options["top-k"])]
        report["top_logits"] = [[int(index), float(last[index])] for index in top]
        if options["logits-output"]:
            last.astype("<f4").tofile(str(options["logits-output"]))       # apps/hf_infer.cpp:1175-1181
    if options["workload"] == "decode" or (options["workload"] == "both" and options["decode-mode"] == "steady"):
        steady = decode_throughput(engine, batch, max(len(tokens), capacity and capacity - int(options["steps"]) - int(options["warmup"]) or len(tokens)),
                                   max(1, int(options["steps"])), int(options["warmup"]))
        report["decode_tokens_per_second"] = round(steady["tokens_per_second"], 3)
        report["decode_ms_per_step"] = round(steady["ms_per_step"], 4)
    if options["workload"] == "both" and new_tokens > 0:
        from ..ops import kernels
        argmax_on_host = options["batch-argmax-mode"] == "host"

        def engine_argmax(logits):
            chosen = on_host(kernels.argmax(logits)).tolist()
            if min(chosen) < 0:
                raise RuntimeError("a row of the logits is not finite")
            return chosen

        def first_maximum(logits):
            """Greedy choice per row, on the device or (--batch-argmax-mode host) from the rows copied out."""
            if not argmax_on_host:
                return engine_argmax(logits)
            rows = on_host(logits).numpy()
            if not np.isfinite(rows).all():
                raise RuntimeError("a row of the logits is not finite")
            return [int(np.argmax(row)) for row in rows]

        def without_cache():
            """Every new token runs its whole sequence again through an empty cache: the reference's
            generate_uncached (apps/hf_infer.cpp:1262-1283), an oracle for the cached path."""
            sequences = [list(prompt) for prompt in prompts]
            for produced in range(new_tokens):
                ids = [("uncached", produced, row) for row in range(batch)]
                for request_id in ids:
                    engine.open(request_id)
                logits = engine.step([StepEntry(request_id, sequence, [len(sequence) - 1]) for request_id, sequence in zip(ids, sequences)])
                for request_id in ids:
                    engine.close(request_id)
                for sequence, token in zip(sequences, first_maximum(logits)):
                    sequence.append(token)
            return sequences, None

        def with_cache_step_by_step():
            """The prompt whole or token by token (--cache-prefill-mode), then one token a step for all rows; keeps
            the last step's logits for --cache-logits-output (apps/hf_infer.cpp:1238-1260)."""
            ids = [("cached", row) for row in range(batch)]
            for request_id in ids:
                engine.open(request_id)
            sequences = [list(prompt) for prompt in prompts]
            portion = len(tokens) if options["cache-prefill-mode"] == "full" else 1
            logits = None
            for start in range(0, len(tokens), portion):
                last = start + portion >= len(tokens)
                logits = engine.step([StepEntry(request_id, prompt[start:start + portion], [min(portion, len(prompt) - start) - 1] if last else [])
                                      for request_id, prompt in zip(ids, prompts)])
            for produced in range(new_tokens):
                chosen = first_maximum(logits)
                for sequence, token in zip(sequences, chosen):
                    sequence.append(token)
                if produced + 1 < new_tokens:
                    logits = engine.step([StepEntry(request_id, [token], [0]) for request_id, token in zip(ids, chosen)], borrow_logits=produced + 2 < new_tokens)
            for request_id in ids:
                engine.close(request_id)
            return sequences, logits

        greedy = params.temperature == 0.0 or params.top_k == 1
        explicit = not use_cache or options["cache-prefill-mode"] == "token" or options["cache-logits-output"] or argmax_on_host
        if explicit and not greedy:
            raise UsageError("--use-cache false, --cache-prefill-mode token, --batch-argmax-mode host and "
                             "--cache-logits-output are for greedy generation (--temperature 0)")
        outputs, elapsed = None, 0.0
        for _ in range(max(1, int(options["steps"])) if options["decode-mode"] == "generation" else 1):
            torch.cuda.synchronize()
            begun = time.perf_counter()
            if not use_cache:
                current, last_logits = without_cache()
            elif explicit:
                current, last_logits = with_cache_step_by_step()
            else:
                current, last_logits = generate(engine, prompts, params, max_batched_tokens=int(options["max-batched-tokens"]),
                                                prefill_chunk=int(options["prefill-chunk"])), None
            torch.cuda.synchronize()
            elapsed += time.perf_counter() - begun
            if outputs is not None and current != outputs:
                raise RuntimeError("deterministic generation changed across steps")      # apps/hf_infer.cpp:1285-1287
            outputs = current
            if options["cache-logits-output"] and last_logits is not None:
                on_host(last_logits).numpy().astype("<f4").tofile(str(options["cache-logits-output"]))   # apps/hf_infer.cpp:1297-1305
        runs = max(1, int(options["steps"])) if options["decode-mode"] == "generation" else 1
        report["generated_tokens"] = outputs[0][len(tokens):]
        report["generation_ms"] = round(elapsed * 1e3, 3)
        report["generation_tokens_per_second"] = round(runs * sum(len(o) - len(tokens) for o in outputs) / elapsed, 3)
        report.update({"use_cache": use_cache, "cache_prefill_mode": options["cache-prefill-mode"],
                       "batch_argmax_mode": options["batch-argmax-mode"]})
    report["prefill_logits_mode"] = options["prefill-logits"]
    report["prompt_tokens"] = len(tokens)
    report.update(measured_transfers())
    print(json.dumps(report), flush=True)
    return 0
