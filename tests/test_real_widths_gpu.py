"""Two layers at the widths of real models (the sizes the kernels are tuned and measured at) against the plain
implementation: a head size of 128 with 7 query heads a group, a head size of 64, reductions of 18944, a vocabulary
that is no power of two. Whole prompts, then decoding, and mixed batches on reused pages, in both dtypes."""
import io
import os

import numpy as np
import pytest
import torch

from microllm_rocm_amd.config import Qwen2Config
from microllm_rocm_amd.weights import write_model_folder
from replay_tools import PlainModel, collect, compare, compare_rounded, mixed, prefill_then_decode, round_up, to_lines, whole
from tiny import random_tokens

pytestmark = pytest.mark.gpu

WIDE = {
    "7b": Qwen2Config(vocab_size=20011, hidden_size=3584, num_hidden_layers=2, num_attention_heads=28, num_key_value_heads=4,
                      head_dim=128, intermediate_size=18944, max_position_embeddings=4096, rope_theta=1e6, rms_norm_eps=1e-6,
                      tie_word_embeddings=False),
    "0.5b": Qwen2Config(vocab_size=15013, hidden_size=896, num_hidden_layers=2, num_attention_heads=14, num_key_value_heads=2,
                        head_dim=64, intermediate_size=4864, max_position_embeddings=4096, rope_theta=1e6, rms_norm_eps=1e-6,
                        tie_word_embeddings=True),
    # the full vocabulary of the 7B model over one layer of its widths: ids up to 152 063 through the embedding, the
    # head's product over 152 064 rows of 3584 (tied, so that the file holds the table once)
    "7b_vocab": Qwen2Config(vocab_size=152064, hidden_size=3584, num_hidden_layers=1, num_attention_heads=28, num_key_value_heads=4,
                            head_dim=128, intermediate_size=18944, max_position_embeddings=4096, rope_theta=1e6, rms_norm_eps=1e-6,
                            tie_word_embeddings=True),
    # one layer at the widths of the largest model (kept in the packed order alone on one GPU)
    "72b": Qwen2Config(vocab_size=10007, hidden_size=8192, num_hidden_layers=1, num_attention_heads=64, num_key_value_heads=8,
                       head_dim=128, intermediate_size=29568, max_position_embeddings=4096, rope_theta=1e6, rms_norm_eps=1e-6,
                       tie_word_embeddings=False),
}
_models = {}


def model_for(tmp_path_factory, which):
    if which not in _models:
        folder = os.path.join(str(tmp_path_factory.mktemp(f"wide_{which}")), "model")
        # Larger weights than N(0, 0.02): the logits of two layers would else be all but the embedding's own.
        write_model_folder(folder, WIDE[which], seed=11, dtype=torch.bfloat16, stds={"std": 0.04, "norm_std": 0.1})
        _models[which] = (folder, PlainModel(folder))
    return _models[which]


def run_trace(folder, dtype, steps, out_dir, max_tokens, **options):
    from microllm_rocm_amd.engine import Engine
    from microllm_rocm_amd.engine.replay import replay
    engine = Engine.from_folder(folder, dtype=dtype, max_tokens=max_tokens, max_requests=8, **options)
    replay(engine, io.StringIO(to_lines(steps)), str(out_dir), io.StringIO())
    engine.cache.check()
    assert not engine.cache.requests
    return engine


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["7b", "0.5b"])
def test_real_widths_match_the_plain_implementation(tmp_path_factory, tmp_path, which, dtype):
    config = WIDE[which]
    folder, plain_model = model_for(tmp_path_factory, which)
    requests = {f"r{index}": random_tokens(40 + index, length, config.vocab_size) for index, length in enumerate([150, 70, 40, 33, 64, 50, 81])}
    # every request whole in one step (many rows: the library's products and the prompt kernels in bfloat16)
    steps = whole(requests)
    run_trace(folder, dtype, steps, tmp_path / "whole", max_tokens=round_up(sum(len(t) for t in requests.values()), 64) + 256)
    together = collect(steps, tmp_path / "whole", config.vocab_size)
    compare(together, requests, plain_model, dtype)
    if dtype == "bfloat16":
        compare_rounded(together, requests, steps, plain_model)
    # most of a request in one step, the last 32 tokens one by one (few rows: the streaming products and their epilogues)
    steps = prefill_then_decode("r0", requests["r0"], tail=32)
    run_trace(folder, dtype, steps, tmp_path / "decode", max_tokens=round_up(len(requests["r0"]), 64))
    decoded = collect(steps, tmp_path / "decode", config.vocab_size)
    compare(decoded, {"r0": requests["r0"]}, plain_model, dtype)
    if dtype == "bfloat16":
        compare_rounded(decoded, {"r0": requests["r0"]}, steps, plain_model)
    # portions of some beside decoded tokens of others, on a pool so small that pages are used again
    steps, peak = mixed(requests, seed=5)
    engine = run_trace(folder, dtype, steps, tmp_path / "mixed", max_tokens=peak)
    pool = engine.cache.groups[0].pool
    assert pool.total_taken > pool.num_pages
    got = collect(steps, tmp_path / "mixed", config.vocab_size)
    compare(got, requests, plain_model, dtype)
    if dtype == "bfloat16":
        compare_rounded(got, requests, steps, plain_model)
    if dtype == "float32":
        for key, row in got.items():
            assert np.array_equal(row, together[key]), f"mixed: {key} differs from the request run whole"
        for key, row in decoded.items():
            assert np.array_equal(row, together[key]), f"decoding: {key} differs from the request run whole"


@pytest.mark.parametrize("which", ["7b", "0.5b"])
def test_real_widths_with_the_packed_weights_alone(tmp_path_factory, tmp_path, which):
    """No copy of the weights for the library: prompts go through this package's tiled product (the reduction in
    parts where the result is narrow), mixed steps through the streaming ones."""
    config = WIDE[which]
    folder, plain_model = model_for(tmp_path_factory, which)
    requests = {f"r{index}": random_tokens(60 + index, length, config.vocab_size) for index, length in enumerate([300, 70, 129, 33])}
    steps = whole(requests)
    engine = run_trace(folder, "bfloat16", steps, tmp_path / "whole", weight_copies="packed",
                       max_tokens=round_up(sum(len(t) for t in requests.values()), 64) + 256)
    assert all(block.ffn.down_weight.tensor is None for block in engine.model.blocks)
    compare(collect(steps, tmp_path / "whole", config.vocab_size), requests, plain_model, "bfloat16")
    steps, peak = mixed(requests, seed=9)
    run_trace(folder, "bfloat16", steps, tmp_path / "mixed", max_tokens=peak, weight_copies="packed")
    compare(collect(steps, tmp_path / "mixed", config.vocab_size), requests, plain_model, "bfloat16")


def staggered_then_together(requests, tail, wave):
    """Prompts come in waves of ``wave`` requests a step, each whole but for its last ``tail`` tokens, beside single
    tokens of up to three requests of earlier waves (which therefore run ahead); then every request decodes, all of
    them in every step, until each has fed its tokens: steps of as many rows as there are live requests."""
    ids = list(requests)
    fed = {rid: 0 for rid in ids}
    steps = []
    for first in range(0, len(ids), wave):
        entries = []
        for rid in ids[:first][:3]:
            if len(requests[rid]) - fed[rid] > 2:        # keeps at least two tokens for the steps together
                entries.append({"id": rid, "tokens": [requests[rid][fed[rid]]], "want": [0]})
                fed[rid] += 1
        for rid in ids[first:first + wave]:
            count = len(requests[rid]) - tail
            entries.append({"id": rid, "tokens": requests[rid][:count], "want": list(range(count))})
            fed[rid] = count
        steps.append({"step": len(steps), "entries": entries, "end": []})
    while any(fed[rid] < len(requests[rid]) for rid in ids):
        entries, ended = [], []
        for rid in ids:
            if fed[rid] < len(requests[rid]):
                entries.append({"id": rid, "tokens": [requests[rid][fed[rid]]], "want": [0]})
                fed[rid] += 1
                if fed[rid] == len(requests[rid]):
                    ended.append(rid)
        steps.append({"step": len(steps), "entries": entries, "end": ended})
    return steps


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_many_requests_decode_together_at_real_widths(tmp_path_factory, tmp_path, dtype):
    """Decode steps of 17, 40, 64 and 96 rows at 7B widths: from 17 rows on the products share their activations
    through LDS and the norms, the rotation and SiLU run as kernels of their own; beyond 64 rows the library's
    products run inside the captured graph; block tables have dozens of rows of differing lengths."""
    from microllm_rocm_amd.engine import Engine
    from microllm_rocm_amd.engine.replay import replay
    config = WIDE["7b"]
    folder, plain_model = model_for(tmp_path_factory, "7b")
    lengths = np.random.default_rng(17).integers(9, 30, size=96)
    everyone = {f"m{index}": random_tokens(500 + index, int(length), config.vocab_size) for index, length in enumerate(lengths)}
    engine = Engine.from_folder(folder, dtype=dtype, max_tokens=96 * 64, max_requests=128)
    alone = {}
    for count in (17, 40, 64, 96):
        requests = dict(list(everyone.items())[:count])
        steps = staggered_then_together(requests, tail=5, wave=11)
        assert max(len(step["entries"]) for step in steps) == count
        out = tmp_path / f"together_{count}"
        replays_before = engine.graph_replays
        replay(engine, io.StringIO(to_lines(steps)), str(out), io.StringIO())
        engine.cache.check()
        assert not engine.cache.requests and engine.graph_replays > replays_before
        got = collect(steps, out, config.vocab_size)
        compare(got, requests, plain_model, dtype)
        if dtype == "float32":
            if not alone:
                steps_alone = whole(everyone)
                replay(engine, io.StringIO(to_lines(steps_alone)), str(tmp_path / "alone"), io.StringIO())
                alone = collect(steps_alone, tmp_path / "alone", config.vocab_size)
            for key, row in got.items():
                assert np.array_equal(row, alone[key]), f"{count} together: {key} differs from the request run alone"


def test_one_layer_at_the_largest_widths_with_the_packed_weights_alone(tmp_path_factory, tmp_path):
    """Hidden 8192, 64 query heads in 8 groups, a feed-forward of 29 568: prompts through the tiled product, decoding
    and mixed steps through the streaming products, no copy of the weights for the library."""
    config = WIDE["72b"]
    folder, plain_model = model_for(tmp_path_factory, "72b")
    requests = {f"r{index}": random_tokens(90 + index, length, config.vocab_size) for index, length in enumerate([140, 37, 70])}
    steps = whole(requests)
    engine = run_trace(folder, "bfloat16", steps, tmp_path / "whole", weight_copies="packed",
                       max_tokens=round_up(sum(len(t) for t in requests.values()), 64) + 256)
    assert all(block.ffn.down_weight.tensor is None and block.mixer.qkv_weight.tensor is None for block in engine.model.blocks)
    compare(collect(steps, tmp_path / "whole", config.vocab_size), requests, plain_model, "bfloat16")
    del engine
    steps, peak = mixed(requests, seed=3)
    run_trace(folder, "bfloat16", steps, tmp_path / "mixed", max_tokens=peak, weight_copies="packed")
    compare(collect(steps, tmp_path / "mixed", config.vocab_size), requests, plain_model, "bfloat16")
    steps = prefill_then_decode("r0", requests["r0"], tail=32)
    run_trace(folder, "bfloat16", steps, tmp_path / "decode", max_tokens=round_up(len(requests["r0"]), 64), weight_copies="packed")
    compare(collect(steps, tmp_path / "decode", config.vocab_size), {"r0": requests["r0"]}, plain_model, "bfloat16")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_full_vocabulary_at_7b_widths(tmp_path_factory, tmp_path, dtype):
    """152 064 logits a row against the plain implementation: a prompt whole, then single tokens (the head's
    streaming product), then a mixed step; tokens from both ends of the vocabulary."""
    config = WIDE["7b_vocab"]
    folder, plain_model = model_for(tmp_path_factory, "7b_vocab")
    requests = {"r0": random_tokens(7, 44, config.vocab_size), "r1": [152063, 0, 151999, 1] + random_tokens(8, 17, config.vocab_size)}
    steps = whole(requests)
    run_trace(folder, dtype, steps, tmp_path / "whole", max_tokens=256)
    together = collect(steps, tmp_path / "whole", config.vocab_size)
    compare(together, requests, plain_model, dtype)
    steps = prefill_then_decode("r0", requests["r0"], tail=6)
    steps[0]["entries"].append({"id": "r1", "tokens": requests["r1"][:9], "want": [0, 8]})
    steps[3]["entries"].append({"id": "r1", "tokens": requests["r1"][9:], "want": list(range(12))})
    steps[3]["end"].append("r1")
    run_trace(folder, dtype, steps, tmp_path / "cut", max_tokens=256)
    got = collect(steps, tmp_path / "cut", config.vocab_size)
    compare(got, requests, plain_model, dtype, expect_all=False)
    assert len(got) == 44 + 2 + 12
    if dtype == "float32":
        for key, row in got.items():
            assert np.array_equal(row, together[key]), f"{key} differs from the request run whole"
    # the selection kernels over the whole row agree with the plain rule on these logits
    from microllm_rocm_amd.ops import kernels
    rows = torch.from_numpy(np.stack([together[("r1", p)] for p in range(4)])).to("cuda:0")
    assert kernels.argmax(rows).tolist() == [int(np.argmax(together[("r1", p)])) for p in range(4)]
