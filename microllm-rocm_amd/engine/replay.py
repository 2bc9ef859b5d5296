"""Trace replay: feed given token ids through the engine step by step and write the logits.

Nothing is sampled. Steps come as JSON lines; each step is one call of
``Engine.step`` on the engine that generation uses, so the logits written are
what a scheduler would have seen for the same cut. The reference has only
fragments of this: token-by-token prefill (apps/hf_infer.cpp:331-338) and raw
float32 logit dumps (apps/hf_infer.cpp:1175-1181, 1297-1305).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
from typing import IO, Optional

import numpy as np
import torch

from ..ops.transfers import on_host
from .batch import StepEntry
from .engine import Engine


def replay(engine: Engine, lines: IO[str], out_dir: str, report: Optional[IO[str]] = None,
           dump_layers: bool = False) -> int:
    """Run every step read from ``lines``; returns the number of steps run.

    With ``dump_layers`` a step that wants logits also writes ``<step>.layers.f32``: the float32 residual stream
    at the wanted places after every run entry, ``[entries, wanted, hidden]`` (the reference traces tensors by
    name instead, include/microllm/profiling/trace.h:63). Steps then run without graphs."""
    os.makedirs(out_dir, exist_ok=True)
    report = report or sys.stdout
    steps = 0
    streams = []
    if dump_layers:
        engine.observe_layers(lambda index, stream: streams.append(stream))
    for line in lines:
        line = line.strip()
        if not line:
            continue
        record = json.loads(line)
        step = record["step"]
        entries = []
        for item in record.get("entries", []):
            request_id = item["id"]
            if not engine.is_open(request_id):
                engine.open(request_id)
            entries.append(StepEntry(request_id, list(item["tokens"]), list(item.get("want", []))))
        streams.clear()
        logits = engine.step(entries) if entries else None
        if logits is not None:
            array = on_host(logits).numpy().astype("<f4", copy=False)
            array.tofile(os.path.join(out_dir, f"{step}.f32"))
            if dump_layers:
                rows, first = [], 0
                for entry in entries:
                    rows += [first + place for place in entry.want]
                    first += len(entry.tokens)
                wanted = on_host(torch.stack(streams)[:, rows]).numpy().astype("<f4", copy=False)
                wanted.tofile(os.path.join(out_dir, f"{step}.layers.f32"))
        for request_id in record.get("end", []):
            if engine.is_open(request_id):
                engine.close(request_id)
        print(f"done {step}", file=report, flush=True)
        steps += 1
    return steps


def main(argv=None) -> int:
    parser = argparse.ArgumentParser(
        prog="trace_run", description="Feed token ids through a model step by step and write logits.")
    parser.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    parser.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    parser.add_argument("--out", required=True, help="folder for <step>.f32 files")
    parser.add_argument("--max-tokens", type=int, required=True,
                        help="most tokens live requests hold at any time; the cache pool is made for this many")
    parser.add_argument("--page-size", type=int, default=16)
    parser.add_argument("--max-requests", type=int, default=16)
    parser.add_argument("--device", default="cuda:0")
    parser.add_argument("--dump-layers", action="store_true",
                        help="also write <step>.layers.f32: the residual stream at the wanted places after every layer")
    args = parser.parse_args(argv)
    if args.max_tokens <= 0:
        parser.error("--max-tokens must be positive")
    engine = Engine.from_folder(args.model, dtype=args.dtype, device=args.device, page_size=args.page_size,
                                max_tokens=args.max_tokens, max_requests=args.max_requests)
    replay(engine, sys.stdin, args.out, dump_layers=args.dump_layers)
    return 0
