"""Trace replay on the GPU against the plain implementation: whole, prefill then decode, changing portions and
mixed batches with reused pages, in float32 and in bfloat16, on tiny configurations that differ in every size."""
import io
import json
import os
import subprocess
import sys

import numpy as np
import pytest

from replay_tools import (PlainModel, collect, compare, compare_rounded, mixed, portions, prefill_then_decode, round_up, to_lines,
                          whole)
from tiny import CONFIGS, make_folder, random_tokens

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SHARP = {"std": 0.12, "norm_std": 0.1}   # sharper attention and larger biases than N(0, 0.02) gives
DTYPES = ["float32", "bfloat16"]
CASES = [("A", None), ("B", None), ("A", SHARP), ("B", SHARP), ("C", SHARP)]
_models = {}


def model_for(tmp_path_factory, which, stds):
    key = (which, bool(stds))
    if key not in _models:
        folder = make_folder(tmp_path_factory.mktemp(f"model_{which}_{'sharp' if stds else 'std'}"), which, stds)
        _models[key] = (folder, PlainModel(folder))
    return _models[key]


def run_trace(folder, dtype, steps, out_dir, max_tokens, **options):
    """In-process replay: the same ``replay`` that bin/trace_run calls, on a fresh engine."""
    from microllm_rocm_amd.engine import Engine
    from microllm_rocm_amd.engine.replay import replay
    engine = Engine.from_folder(folder, dtype=dtype, max_tokens=max_tokens, max_requests=8, **options)
    report = io.StringIO()
    replay(engine, io.StringIO(to_lines(steps)), str(out_dir), report)
    assert report.getvalue().split() == [word for step in steps for word in ("done", str(step["step"]))]
    engine.cache.check()
    assert not engine.cache.requests, "every request of a trace is ended"
    assert all(free == group.pool.num_pages for free, group in zip(engine.cache.free_pages(), engine.cache.groups))
    return engine


def requests_for(config, lengths, seed):
    return {f"r{index}": random_tokens(seed + index, length, config.vocab_size) for index, length in enumerate(lengths)}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("which,stds", CASES)
def test_every_cut_matches_the_plain_implementation(tmp_path_factory, tmp_path, which, stds, dtype):
    config = CONFIGS[which]
    folder, plain_model = model_for(tmp_path_factory, which, stds)
    lengths = [100, 64, 37] if which != "C" else [300, 129, 64]
    requests = requests_for(config, lengths, seed=10)
    vocab = config.vocab_size
    results = {}

    steps = whole(requests)
    run_trace(folder, dtype, steps, tmp_path / "whole", max_tokens=round_up(max(lengths), 64))
    results["whole"] = collect(steps, tmp_path / "whole", vocab)
    compare(results["whole"], requests, plain_model, dtype)
    if dtype == "bfloat16":
        compare_rounded(results["whole"], requests, steps, plain_model)

    for rid, tokens in requests.items():
        steps = prefill_then_decode(rid, tokens, tail=32)
        run_trace(folder, dtype, steps, tmp_path / f"decode_{rid}", max_tokens=round_up(len(tokens), 64))
        results[f"decode_{rid}"] = collect(steps, tmp_path / f"decode_{rid}", vocab)
        compare(results[f"decode_{rid}"], {rid: tokens}, plain_model, dtype)
        if dtype == "bfloat16":
            compare_rounded(results[f"decode_{rid}"], {rid: tokens}, steps, plain_model)

        steps = portions(rid, tokens, sizes=[7, 2, 5, 16, 3, 2, 33, 2, 17])
        run_trace(folder, dtype, steps, tmp_path / f"portions_{rid}", max_tokens=round_up(len(tokens), 64))
        results[f"portions_{rid}"] = collect(steps, tmp_path / f"portions_{rid}", vocab)
        compare(results[f"portions_{rid}"], {rid: tokens}, plain_model, dtype)
        if dtype == "bfloat16":
            compare_rounded(results[f"portions_{rid}"], {rid: tokens}, steps, plain_model)

    if dtype == "float32":
        # In 32-bit every kernel sums in an order that depends on the row alone: the cuts agree bit for bit.
        for name, rows in results.items():
            if name == "whole":
                continue
            for key, row in rows.items():
                assert np.array_equal(row, results["whole"][key]), f"{name}: {key} differs from the whole run"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("which,stds", [("A", SHARP), ("B", SHARP), ("C", SHARP)])
def test_mixed_batches_with_reused_pages(tmp_path_factory, tmp_path, which, stds, dtype):
    config = CONFIGS[which]
    folder, plain_model = model_for(tmp_path_factory, which, stds)
    lengths = [70, 45, 90, 33, 64, 50, 81] if which != "C" else [200, 70, 150, 64, 260, 90]
    requests = requests_for(config, lengths, seed=20)
    steps, peak = mixed(requests, seed=3)
    assert max(len(step["entries"]) for step in steps) == 4
    assert any(len(e["tokens"]) == 1 for s in steps for e in s["entries"]) and any(len(e["tokens"]) == 2 for s in steps for e in s["entries"])
    engine = run_trace(folder, dtype, steps, tmp_path / "mixed", max_tokens=peak)
    pool = engine.cache.groups[0].pool
    assert pool.total_taken > pool.num_pages, "the pool is small enough for pages to be used again"
    got = collect(steps, tmp_path / "mixed", config.vocab_size)
    compare(got, requests, plain_model, dtype)
    if dtype == "bfloat16":
        compare_rounded(got, requests, steps, plain_model)
    if dtype == "float32":
        alone = whole(requests)
        run_trace(folder, dtype, alone, tmp_path / "alone", max_tokens=round_up(max(lengths), 64))
        reference = collect(alone, tmp_path / "alone", config.vocab_size)
        for key, row in got.items():
            assert np.array_equal(row, reference[key]), f"mixed: {key} differs from the request run alone"


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_first_tokens_and_long_decoding(tmp_path_factory, tmp_path, dtype):
    config = CONFIGS["C"]
    folder, plain_model = model_for(tmp_path_factory, "C", SHARP)
    tokens = random_tokens(77, 400, config.vocab_size)
    # the first tokens of a sequence, one by one from an empty cache, then a long run of decoding past the window
    steps = prefill_then_decode("long", tokens, tail=399)
    run_trace(folder, dtype, steps, tmp_path / "long", max_tokens=round_up(len(tokens), 64))
    got = collect(steps, tmp_path / "long", config.vocab_size)
    compare(got, {"long": tokens}, plain_model, dtype)
    if dtype == "bfloat16":
        compare_rounded(got, {"long": tokens}, steps, plain_model)
    for count in (1, 2, 3):
        steps = whole({"first": tokens[:count]})
        run_trace(folder, dtype, steps, tmp_path / f"first{count}", max_tokens=64)
        compare(collect(steps, tmp_path / f"first{count}", config.vocab_size), {"first": tokens[:count]}, plain_model, dtype)


@pytest.mark.parametrize("which", ["B", "C"])
def test_one_copy_of_the_weights(tmp_path_factory, tmp_path, which):
    """With the packed copy alone, steps with many rows go through the streaming products 64 rows at a time."""
    config = CONFIGS[which]
    folder, plain_model = model_for(tmp_path_factory, which, SHARP)
    requests = requests_for(config, [150, 64, 37, 70, 90], seed=30)
    steps = whole(requests)
    engine = run_trace(folder, "bfloat16", steps, tmp_path / "whole", max_tokens=512, weight_copies="packed")
    assert engine.weight_copies == "packed"
    block = engine.model.blocks[0]
    assert block.ffn.down_weight.tensor is None and block.ffn.down_weight.packed is not None
    assert block.mixer.qkv_weight.tensor is None and engine.model.head.weight.packed is not None
    compare(collect(steps, tmp_path / "whole", config.vocab_size), requests, plain_model, "bfloat16")
    compare_rounded(collect(steps, tmp_path / "whole", config.vocab_size), requests, steps, plain_model, one_weight_copy=True)
    steps, peak = mixed(requests, seed=9)
    run_trace(folder, "bfloat16", steps, tmp_path / "mixed", max_tokens=peak, weight_copies="packed")
    compare(collect(steps, tmp_path / "mixed", config.vocab_size), requests, plain_model, "bfloat16")
    compare_rounded(collect(steps, tmp_path / "mixed", config.vocab_size), requests, steps, plain_model, one_weight_copy=True)
    both = run_trace(folder, "bfloat16", whole({"r0": requests["r0"]}), tmp_path / "both", max_tokens=256)
    assert both.weight_copies == "both" and both.model.blocks[0].ffn.down_weight.tensor is not None


def test_logits_only_where_wanted_and_requests_left_out(tmp_path_factory, tmp_path):
    config = CONFIGS["B"]
    folder, plain_model = model_for(tmp_path_factory, "B", SHARP)
    a, b = random_tokens(1, 40, config.vocab_size), random_tokens(2, 30, config.vocab_size)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:20], "want": []}], "end": []},
        {"step": 1, "entries": [{"id": "b", "tokens": b[:30], "want": [29, 0]}], "end": ["b"]},
        {"step": 2, "entries": [{"id": "a", "tokens": a[20:40], "want": [19]}], "end": ["a"]},
    ]
    run_trace(folder, "float32", steps, tmp_path / "out", max_tokens=128)
    assert not os.path.exists(tmp_path / "out" / "0.f32")
    rows = np.fromfile(tmp_path / "out" / "1.f32", dtype="<f4").reshape(2, config.vocab_size)
    reference = plain_model.logits(b)
    scale = np.abs(reference).max()
    assert np.abs(rows[0] - reference[29]).max() <= 2e-5 * scale and np.abs(rows[1] - reference[0]).max() <= 2e-5 * scale
    last = np.fromfile(tmp_path / "out" / "2.f32", dtype="<f4")
    assert np.abs(last - plain_model.logits(a)[39]).max() <= 2e-5 * np.abs(plain_model.logits(a)).max()


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_program_itself(tmp_path_factory, tmp_path, dtype):
    """bin/trace_run as a user calls it: a process, steps on standard input, files in --out."""
    config = CONFIGS["B"]
    folder, plain_model = model_for(tmp_path_factory, "B", SHARP)
    requests = requests_for(config, [50, 64, 33, 40, 70], seed=40)
    steps, peak = mixed(requests, seed=5)
    out_dir = tmp_path / "program"
    result = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
                             "--out", str(out_dir), "--max-tokens", str(peak)],
                            input=to_lines(steps), capture_output=True, text=True, timeout=300)
    assert result.returncode == 0, result.stderr
    assert result.stdout.split() == [word for step in steps for word in ("done", str(step["step"]))]
    compare(collect(steps, out_dir, config.vocab_size), requests, plain_model, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("page_size", [32, 64])
def test_larger_pages(tmp_path_factory, tmp_path, dtype, page_size):
    """Pages of 32 and 64 positions hold two and four 16-position tiles; the window's edge falls inside a page."""
    from microllm_rocm_amd.engine import Engine
    from microllm_rocm_amd.engine.replay import replay
    config = CONFIGS["C"]
    folder, plain_model = model_for(tmp_path_factory, "C", SHARP)
    requests = requests_for(config, [150, 70, 129, 64, 200], seed=60)
    steps, peak = mixed(requests, seed=9)
    engine = Engine.from_folder(folder, dtype=dtype, page_size=page_size, max_tokens=round_up(peak, page_size) + 2 * page_size,
                                max_requests=8)
    replay(engine, io.StringIO(to_lines(steps)), str(tmp_path / "out"), io.StringIO())
    engine.cache.check()
    compare(collect(steps, tmp_path / "out", config.vocab_size), requests, plain_model, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_weights_stored_in_32_bit_stay_32_bit(tmp_path, dtype):
    """A file of float32 tensors whose values bfloat16 cannot hold: they are not rounded, in either engine."""
    import torch
    from microllm_rocm_amd.engine import Engine
    from microllm_rocm_amd.weights import write_model_folder
    config = CONFIGS["B"]
    folder = write_model_folder(str(tmp_path / "f32"), config, seed=11, dtype=torch.float32, stds=SHARP)
    plain_model = PlainModel(folder)
    assert np.abs(plain_model.weights["lm_head.weight"] - plain_model.weights["lm_head.weight"].astype(np.float32)
                  .view(np.uint32).__and__(0xFFFF0000).view(np.float32)).max() > 0    # not bfloat16 values
    requests = requests_for(config, [90, 40], seed=70)
    steps = portions("r0", requests["r0"], [40, 2, 17, 1, 1, 1]) + [dict(step, step=step["step"] + 100) for step in whole({"r1": requests["r1"]})]
    engine = run_trace(folder, dtype, steps, tmp_path / "out", max_tokens=192)
    assert engine.model.head.weight.tensor.dtype == torch.float32
    assert engine.model.blocks[0].mixer.qkv_weight.tensor.dtype == torch.float32
    got = collect(steps, tmp_path / "out", config.vocab_size)
    worst_max, _ = compare(got, requests, plain_model, dtype)
    if dtype == "bfloat16":
        assert worst_max > 1e-4      # activations are still bfloat16: this is not the 32-bit engine in disguise


@pytest.mark.parametrize("dtype", DTYPES)
def test_stale_pages_hold_anything(tmp_path_factory, tmp_path, dtype):
    """Every page is filled with NaN before the trace: what a request has not written itself must never reach a
    result, whether it lies beyond the request's length, before its window, or on a page used again."""
    import torch
    from microllm_rocm_amd.cache.manager import PagedBinding
    from microllm_rocm_amd.engine import Engine
    from microllm_rocm_amd.engine.replay import replay
    config = CONFIGS["C"]
    folder, plain_model = model_for(tmp_path_factory, "C", SHARP)
    requests = requests_for(config, [170, 70, 129, 66, 210], seed=80)
    steps, peak = mixed(requests, seed=11)
    engine = Engine.from_folder(folder, dtype=dtype, max_tokens=peak, max_requests=8)
    for binding in engine.cache.bindings():
        if isinstance(binding, PagedBinding):
            binding.k.fill_(float("nan"))
            binding.v.fill_(float("nan"))
    replay(engine, io.StringIO(to_lines(steps)), str(tmp_path / "out"), io.StringIO())
    pool = engine.cache.groups[0].pool
    assert pool.total_taken > pool.num_pages
    compare(collect(steps, tmp_path / "out", config.vocab_size), requests, plain_model, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_stream_layer_by_layer(tmp_path_factory, tmp_path, dtype):
    """--dump-layers: the residual stream at the wanted places after every layer, against the plain
    implementation's, in portions of changing size (few rows: the norms are taken by the products; many: not)."""
    import plain_qwen2 as plain
    from replay_tools import TOLERANCE
    config = CONFIGS["B"]
    folder, plain_model = model_for(tmp_path_factory, "B", SHARP)
    tokens = random_tokens(77, 90, config.vocab_size)
    steps = portions("a", tokens, [40, 2, 17, 1, 1, 29])
    out_dir = tmp_path / "layers"
    result = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
                             "--out", str(out_dir), "--max-tokens", "128", "--dump-layers"],
                            input=to_lines(steps), capture_output=True, text=True, timeout=300)
    assert result.returncode == 0, result.stderr
    compare(collect(steps, out_dir, config.vocab_size), {"a": tokens}, plain_model, dtype)
    expected = plain.layer_streams(plain_model.config, plain_model.weights, tokens)
    layers, width = config.num_hidden_layers, config.hidden_size
    first = 0
    for step in steps:
        entry = step["entries"][0]
        got = np.fromfile(out_dir / f"{step['step']}.layers.f32", dtype="<f4").reshape(layers, len(entry["want"]), width)
        for layer in range(layers):
            want = expected[layer][[first + place for place in entry["want"]]]
            error = np.abs(got[layer] - want).max() / np.abs(expected[layer]).max()
            assert error <= TOLERANCE[dtype]["max"], f"{dtype}: step {step['step']} layer {layer}: {error:.3e}"
        first += len(entry["tokens"])
