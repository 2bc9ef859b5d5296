"""Decode and prefill throughput of the engine at Qwen2-7B size (or, with --size, 72B or 0.5B) with random weights on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W

A step is one decode step of the engine's own loop: one token of every request through `Engine.step`,
greedy selection on the device, the chosen ids back to the host. Prints one JSON line.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

SIZES = {
    "7b": dict(vocab_size=152064, hidden_size=3584, num_hidden_layers=28, num_attention_heads=28, num_key_value_heads=4,
               head_dim=128, intermediate_size=18944, tie_word_embeddings=False),
    "72b": dict(vocab_size=152064, hidden_size=8192, num_hidden_layers=80, num_attention_heads=64, num_key_value_heads=8,
                head_dim=128, intermediate_size=29568, tie_word_embeddings=False),
    "0.5b": dict(vocab_size=151936, hidden_size=896, num_hidden_layers=24, num_attention_heads=14, num_key_value_heads=2,
                 head_dim=64, intermediate_size=4864, tie_word_embeddings=True),
}
HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
BF16_PEAK_FLOPS = 2.5e15       # MI355X dense bf16 MFMA, published
FP32_PEAK_FLOPS = 157.3e12


def serve(args, config, full_layers: int, page_size: int) -> int:
    """The reference's continuous-batching workload through the scheduler; prints one JSON line."""
    from microllm_rocm_amd import Engine
    from microllm_rocm_amd.engine.benchmark import serving_throughput
    requests, longest, new_tokens, chunk, budget = args.serve_requests, 2048, 256, 512, 2048
    max_tokens = requests * (-(-(longest + new_tokens) // page_size) + 1) * page_size
    engine = Engine.from_random(config, seed=0, dtype=args.dtype, device="cuda:0", on_device=True, page_size=page_size,
                                max_tokens=max_tokens, max_requests=requests, weight_copies=args.weight_copies,
                                max_portion=chunk, graph_mixed_steps=not args.no_mixed_graphs)
    runs = max(1, min(args.steps, 5))
    warmup = max(1, min(args.warmup, 2))
    result = serving_throughput(engine, requests=requests, prompt_range=(128, longest), new_tokens=new_tokens,
                                prefill_chunk=chunk, max_batched_tokens=budget, runs=runs, warmup=warmup)
    line = {
        "metric": f"continuous batching, generated tok/s, Qwen2-{args.size.upper()} {'bf16' if args.dtype == 'bfloat16' else 'fp32'}",
        "value": round(result["tokens_per_second"], 1), "unit": "tok/s", "n_gpus": 1, "steps": runs, "warmup": warmup,
        "ms_per_step": round(result["ms_per_run"], 2), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic: random N(0,0.02) weights, uniform-random token ids and prompt lengths; a step is one whole run of the workload",
        "config": {"model": f"Qwen2-{args.size.upper()} size", "layers": args.layers, "layers_of_full_model": full_layers,
                   "requests": requests, "prompt_lengths": "uniform 128..2048", "new_tokens": new_tokens,
                   "prefill_chunk": chunk, "max_batched_tokens": budget, "kv_block_size": page_size,
                   "weight_copies": engine.weight_copies, "mixed_step_graphs": not args.no_mixed_graphs,
                   "parallelism": "single GPU"},
        "serve": {key: (round(value, 2) if isinstance(value, float) else value) for key, value in result.items()},
    }
    print(json.dumps(line), flush=True)
    return 0


def main() -> int:
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=64)
    parser.add_argument("--warmup", type=int, default=8)
    parser.add_argument("--batch", type=int, default=8)
    parser.add_argument("--context", type=int, default=4096)
    parser.add_argument("--size", default="7b", choices=sorted(SIZES), help="layer sizes: Qwen2-7B's (the default), 72B's or 0.5B's")
    parser.add_argument("--layers", type=int, default=None, help="fewer than the model has only where memory or time needs it")
    parser.add_argument("--prefill-tokens", type=int, default=2048)
    parser.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    parser.add_argument("--points", default="1,64", help="other decode batch sizes to report")
    parser.add_argument("--no-prefill", action="store_true")
    parser.add_argument("--weight-copies", default="auto", choices=["auto", "both", "packed"],
                        help="packed: one copy of every weight, and this package's own matrix kernels for every product")
    parser.add_argument("--no-library-tuning", action="store_true",
                        help="leave the choice of the library's algorithm for the prompt's large products to its heuristic")
    parser.add_argument("--no-calibration", action="store_true", help="skip measuring what a read-only and an MFMA-only kernel reach")
    parser.add_argument("--serve", action="store_true",
                        help="the continuous-batching workload instead: 64 requests, prompts of 128 to 2048 tokens, 256 new tokens each, "
                             "portions of 512 (--steps whole runs timed after --warmup untimed ones); meant for --size 0.5b")
    parser.add_argument("--serve-requests", type=int, default=64)
    parser.add_argument("--no-mixed-graphs", action="store_true", help="run steps that mix portions and single tokens eagerly")
    parser.add_argument("--no-extras", action="store_true",
                        help="leave out what the default run adds to its line after the main figures: decoding on the 32-bit path "
                             "at batch 8 and the continuous-batching workload at Qwen2-0.5B sizes")
    args = parser.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported (this engine runs on a single MI355X)")
        return 2

    import torch
    from microllm_rocm_amd import Engine, Qwen2Config
    from microllm_rocm_amd.engine.benchmark import decode_throughput, prefill_throughput, step_bytes, step_flops

    sizes = dict(SIZES[args.size])
    full_layers = sizes.pop("num_hidden_layers")
    if args.layers is None:
        args.layers = full_layers
    config = Qwen2Config(num_hidden_layers=args.layers, max_position_embeddings=32768, rope_theta=1e6, rms_norm_eps=1e-6, **sizes)
    page_size = 16
    if args.serve:
        return serve(args, config, full_layers, page_size)
    points = sorted({int(b) for b in args.points.split(",") if b} | {args.batch})
    largest = max(points)
    per_request = args.context + args.steps + args.warmup + 2 * page_size
    max_tokens = max(largest * per_request, args.prefill_tokens + page_size)
    engine = Engine.from_random(config, seed=0, dtype=args.dtype, device="cuda:0", on_device=True,
                                page_size=page_size, max_tokens=max_tokens, max_requests=max(largest, 4),
                                weight_copies=args.weight_copies,
                                tune_library=not args.no_library_tuning and not args.no_prefill)
    peak_flops = BF16_PEAK_FLOPS if args.dtype == "bfloat16" else FP32_PEAK_FLOPS

    results = {}
    for batch in points:
        results[batch] = decode_throughput(engine, batch, args.context, args.steps, args.warmup, seed=batch)
    main_result = results[args.batch]
    bytes_step = step_bytes(engine, args.batch, args.context + args.warmup + args.steps // 2)
    achieved = bytes_step / (main_result["ms_per_step"] * 1e-3) / 1e9

    line = {
        "metric": f"decode tok/s (ctx {args.context}) Qwen2-{args.size.upper()} {'bf16' if args.dtype == 'bfloat16' else 'fp32'}",
        "value": round(main_result["tokens_per_second"], 2),
        "unit": "tok/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(main_result["ms_per_step"], 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic: random N(0,0.02) weights, uniform-random token ids, caches filled with random keys and values",
        "config": {
            "model": f"Qwen2-{args.size.upper()} size", "layers": args.layers, "layers_of_full_model": full_layers,
            "hidden_size": config.hidden_size, "heads": config.num_attention_heads,
            "kv_heads": config.num_key_value_heads, "head_dim": config.head_dim,
            "intermediate_size": config.intermediate_size, "vocab_size": config.vocab_size,
            "tie_word_embeddings": config.tie_word_embeddings, "weight_copies": engine.weight_copies,
            "library_tuning": not args.no_library_tuning and not args.no_prefill, "global_batch": args.batch, "seq_len": args.context,
            "kv_block_size": page_size, "prefill_tokens": args.prefill_tokens, "parallelism": "single GPU",
        },
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
        "points": {f"decode_b{batch}": round(results[batch]["tokens_per_second"], 2) for batch in points if batch != args.batch},
    }
    if not args.no_prefill:
        prefill = prefill_throughput(engine, args.prefill_tokens, repeats=3)
        flops = step_flops(engine, args.prefill_tokens)
        line["prefill"] = {"value": round(prefill["tokens_per_second"], 1), "tokens": args.prefill_tokens,
                           "ms": round(prefill["ms"], 3),
                           "frac": round(flops / (prefill["ms"] * 1e-3) / peak_flops, 4),
                           "runs": "best of 3 (value, ms, frac); their mean beside it",
                           "mean_ms": round(prefill["mean_ms"], 3), "mean_value": round(prefill["mean_tokens_per_second"], 1),
                           "mean_frac": round(flops / (prefill["mean_ms"] * 1e-3) / peak_flops, 4), "all_ms": prefill["all_ms"]}
    if not args.no_calibration and args.dtype == "bfloat16":
        # What kernels that do nothing but read memory, or nothing but bfloat16 MFMAs, reach on this GPU: the
        # fractions of these stand beside the fractions of the published peaks.
        from microllm_rocm_amd.ops.kernels import measured_peaks
        measured = measured_peaks()
        line["measured_peaks"] = measured
        line["roofline"]["frac_of_measured"] = round(achieved / measured["hbm_read_GBps"], 4)
        if "prefill" in line:
            line["prefill"]["frac_of_measured"] = round(flops / (prefill["ms"] * 1e-3) / (measured["mfma_bf16_TFLOPs"] * 1e12), 4)
    extras = not args.no_extras and args.size == "7b" and args.dtype == "bfloat16" and args.layers == full_layers
    if extras:
        # Two more figures of the same program on the same GPU, each on an engine of its own after the main one is
        # gone: decoding on the true 32-bit path, and the continuous-batching workload at the smallest model's sizes.
        del engine
        torch.cuda.empty_cache()
        exact = Engine.from_random(config, seed=0, dtype="float32", device="cuda:0", on_device=True, page_size=page_size,
                                   max_tokens=8 * (args.context + 8 + 2 * page_size), max_requests=8)
        fp32 = decode_throughput(exact, 8, args.context, steps=5, warmup=1, seed=8)
        fp32_bytes = step_bytes(exact, 8, args.context + 3)
        line["points"]["fp32_decode_b8"] = round(fp32["tokens_per_second"], 2)
        line["fp32"] = {"config": "the same model and context on the true 32-bit path, batch 8, 5 steps after 1", "dtype": "fp32",
                        "value": round(fp32["tokens_per_second"], 2), "ms_per_step": round(fp32["ms_per_step"], 3),
                        "roofline_frac": round(fp32_bytes / (fp32["ms_per_step"] * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
        del exact
        torch.cuda.empty_cache()
        from microllm_rocm_amd.engine.benchmark import serving_throughput
        small_sizes = dict(SIZES["0.5b"])
        small = Qwen2Config(max_position_embeddings=32768, rope_theta=1e6, rms_norm_eps=1e-6, **small_sizes)
        requests, longest, new_tokens, chunk, budget = 64, 2048, 256, 512, 2048
        server = Engine.from_random(small, seed=0, dtype="bfloat16", device="cuda:0", on_device=True, page_size=page_size,
                                    max_tokens=requests * (-(-(longest + new_tokens) // page_size) + 1) * page_size,
                                    max_requests=requests, max_portion=chunk)
        served = serving_throughput(server, requests=requests, prompt_range=(128, longest), new_tokens=new_tokens,
                                    prefill_chunk=chunk, max_batched_tokens=budget, runs=3, warmup=1)
        line["serve"] = {"config": "Qwen2-0.5B size, bf16, 64 requests, prompts uniform 128..2048, 256 new tokens each, "
                                   "portions of 512, 2048 tokens a step, 3 runs after 1",
                         "value": round(served["tokens_per_second"], 1), "unit": "generated tok/s",
                         "ttft_p50_ms": round(served["ttft_p50_ms"], 1), "ttft_p95_ms": round(served["ttft_p95_ms"], 1),
                         "completion_p95_ms": round(served["completion_p95_ms"], 1), "preemptions": served["preemptions"],
                         "scheduler_steps": served["scheduler_steps"]}
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
