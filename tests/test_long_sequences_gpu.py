"""Requests of thousands of positions through the engine against the plain implementation, at the attention
geometries of the real models (28 query heads on 4 kv heads of 128; 14 on 2 of 64) over narrow layers: a 2048-token
prompt whole (sixteen tiles of queries), a request of 4564 positions in portions of 512 and then 64 single tokens
(portions over thousands of cached keys, block tables of hundreds of pages, several splits of the keys), and the
same request beside shorter ones on a pool so small that pages are used again; one model with a window of 1000 in
its later layer. Both dtypes; in 32-bit every cut gives the bits of the request run whole.
The reference walks contexts and batch sizes the same way (tests/inference/shape_matrix_test.cpp:61-116)."""
import io
import os

import numpy as np
import pytest
import torch

from microllm_rocm_amd.config import Qwen2Config
from microllm_rocm_amd.weights import write_model_folder
from replay_tools import PlainModel, collect, compare, compare_rounded, mixed, portions, round_up, to_lines, whole
from tiny import random_tokens

pytestmark = pytest.mark.gpu

LONG = {
    "hd128": Qwen2Config(vocab_size=1009, hidden_size=256, num_hidden_layers=2, num_attention_heads=28, num_key_value_heads=4,
                         head_dim=128, intermediate_size=704, max_position_embeddings=8192, rope_theta=1e6, rms_norm_eps=1e-6,
                         tie_word_embeddings=False),
    "hd64_window": Qwen2Config(vocab_size=787, hidden_size=192, num_hidden_layers=2, num_attention_heads=14, num_key_value_heads=2,
                               head_dim=64, intermediate_size=528, max_position_embeddings=8192, rope_theta=1e6, rms_norm_eps=1e-6,
                               tie_word_embeddings=True, use_sliding_window=True, sliding_window=1000, max_window_layers=1),
}
LENGTH, TAIL, PROMPT = 4564, 64, 2048
_models = {}


def model_for(tmp_path_factory, which):
    if which not in _models:
        folder = os.path.join(str(tmp_path_factory.mktemp(f"long_{which}")), "model")
        # Weights large enough that a query's few strongest keys, anywhere among thousands, carry its result.
        write_model_folder(folder, LONG[which], seed=21, dtype=torch.bfloat16, stds={"std": 0.08, "norm_std": 0.1})
        _models[which] = (folder, PlainModel(folder))
    return _models[which]


def run_trace(folder, dtype, steps, out_dir, max_tokens, **options):
    from microllm_rocm_amd.engine import Engine
    from microllm_rocm_amd.engine.replay import replay
    engine = Engine.from_folder(folder, dtype=dtype, max_tokens=max_tokens, max_requests=8, **options)
    replay(engine, io.StringIO(to_lines(steps)), str(out_dir), io.StringIO())
    engine.cache.check()
    assert not engine.cache.requests
    assert all(free == group.pool.num_pages for free, group in zip(engine.cache.free_pages(), engine.cache.groups))
    return engine


def portions_then_single_tokens(rid, tokens, portion, tail):
    steps = portions(rid, tokens[:len(tokens) - tail], sizes=[portion])
    steps[-1]["end"] = []
    for index in range(tail):
        place = len(tokens) - tail + index
        steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": [tokens[place]], "want": [0]}],
                      "end": [rid] if index == tail - 1 else []})
    return steps


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["hd128", "hd64_window"])
def test_thousands_of_positions_under_every_cut(tmp_path_factory, tmp_path, which, dtype):
    config = LONG[which]
    vocab = config.vocab_size
    folder, plain_model = model_for(tmp_path_factory, which)
    long = random_tokens(300, LENGTH, vocab)
    plain_model.logits(long)        # the prompt below is its prefix: one plain run serves both

    # (a) a prompt of 2048 tokens, whole
    prompt = {"long": long[:PROMPT]}
    steps = whole(prompt)
    run_trace(folder, dtype, steps, tmp_path / "prompt", max_tokens=PROMPT)
    prompt_rows = collect(steps, tmp_path / "prompt", vocab)
    compare(prompt_rows, prompt, plain_model, dtype)
    if dtype == "bfloat16":
        compare_rounded(prompt_rows, prompt, steps, plain_model)

    # (b) 4500 positions in portions of 512, then 64 single tokens
    steps = portions_then_single_tokens("long", long, 512, TAIL)
    assert len(steps) == 9 + TAIL
    engine = run_trace(folder, dtype, steps, tmp_path / "portions", max_tokens=round_up(LENGTH, 64))
    assert engine.graph_replays >= TAIL - 1
    in_portions = collect(steps, tmp_path / "portions", vocab)
    assert max(position for _, position in in_portions) == LENGTH - 1
    compare(in_portions, {"long": long}, plain_model, dtype)
    if dtype == "bfloat16":
        compare_rounded(in_portions, {"long": long}, steps, plain_model)

    # (c) the same request, portions of up to 512 and its last 64 tokens one by one, beside shorter requests that come
    # and go, on a pool so small that their pages are used again
    requests = {"long": long}
    for index, length in enumerate([700, 330, 1200, 150, 520]):
        requests[f"s{index}"] = random_tokens(310 + index, length, vocab)
    steps, peak = mixed(requests, seed=1, decode_tail=TAIL, max_portion=512)
    assert max(len(step["entries"]) for step in steps) == 4
    portions_beside_single_tokens = sum(1 for step in steps if any(e["id"] == "long" and len(e["tokens"]) > 1 for e in step["entries"])
                                        and any(len(e["tokens"]) == 1 for e in step["entries"]))
    single_tokens_beside_others = sum(1 for step in steps if len(step["entries"]) > 1
                                      and any(e["id"] == "long" and len(e["tokens"]) == 1 for e in step["entries"]))
    assert portions_beside_single_tokens >= 10 and single_tokens_beside_others >= 32
    engine = run_trace(folder, dtype, steps, tmp_path / "mixed", max_tokens=peak)
    pool = engine.cache.groups[0].pool
    assert pool.total_taken > pool.num_pages, "the pool is small enough for pages to be used again"
    together = collect(steps, tmp_path / "mixed", vocab)
    compare(together, requests, plain_model, dtype)
    if dtype == "bfloat16":
        compare_rounded(together, requests, steps, plain_model)

    if dtype == "float32":
        steps = whole({"long": long})
        run_trace(folder, dtype, steps, tmp_path / "whole", max_tokens=round_up(LENGTH, 64))
        alone = collect(steps, tmp_path / "whole", vocab)
        for name, rows in (("the prompt", prompt_rows), ("portions", in_portions), ("mixed", together)):
            for key, row in rows.items():
                if key[0] == "long":
                    assert np.array_equal(row, alone[key]), f"{name}: {key} differs from the request run whole"
