"""All 28 layers at Qwen2-7B sizes with random weights: the 32-bit engine gives the same bits however the work is
cut (a prompt whole, in portions of changing size, most of it at once and the last 32 tokens one by one, mixed with
other requests on reused pages), and the bfloat16 engine on the same weights stays as close to it as the format
allows at this depth. Engine against engine: the comparison with the plain implementation is made at two layers of
these widths and at thousands of positions elsewhere; this one covers the chains of partial sums over 56 norms and
the full depth.

What the format allows at 28 layers: rounding errors add up layer by layer (the worst row of the plain run with a
bfloat16 engine's roundings lies 1.1e-2 of the logits' scale from the exact run at 2 layers, 2.1e-2 at 7 and 4.8e-2
at 28, the root of the depth), so the bound of the two- and three-layer models does not apply. The plain
implementation cannot run 7.6e9 weights in float64 in a test's time; it runs a narrow model of the same depth whose
layers have the same gains instead (hidden 256 with N(0, 0.075) where the real one has 3584 with N(0, 0.02): both
multiply a normalised row by 1.2, and both feed-forwards are 5.3 times as wide as the stream), exact and with the
roundings, and the engine's rows may lie half as far again from the 32-bit engine's as that run's worst row from
the exact one."""
import os

import numpy as np
import pytest
import torch

from microllm_rocm_amd.config import Qwen2Config
from replay_tools import PlainModel, mixed, portions, prefill_then_decode, roundings, whole
from tiny import random_tokens

pytestmark = pytest.mark.gpu

FULL_7B = Qwen2Config(vocab_size=152064, hidden_size=3584, num_hidden_layers=28, num_attention_heads=28, num_key_value_heads=4,
                      head_dim=128, intermediate_size=18944, max_position_embeddings=4096, rope_theta=1e6, rms_norm_eps=1e-6,
                      tie_word_embeddings=False)
LENGTHS = {"a": 330, "b": 90, "c": 150, "d": 47, "e": 64, "f": 113, "g": 70}


PROXY = Qwen2Config(vocab_size=1000, hidden_size=256, num_hidden_layers=28, num_attention_heads=4, num_key_value_heads=2,
                    head_dim=64, intermediate_size=1408, max_position_embeddings=4096, rope_theta=1e6, rms_norm_eps=1e-6,
                    tie_word_embeddings=False)


def what_rounding_costs_at_this_depth(folder, tokens):
    """(max, rms) error of the worst row of the narrow model's rounded plain run against its exact run, relative
    to the logits' scale, for a prompt run whole and for one run a token at a time."""
    from microllm_rocm_amd.weights import write_model_folder
    write_model_folder(folder, PROXY, seed=3, dtype=torch.bfloat16, stds={"std": 0.075, "norm_std": 0.0})
    model = PlainModel(folder)
    tokens = [token % PROXY.vocab_size for token in tokens]
    exact = model.logits(tokens)
    worst_max = worst_rms = 0.0
    for step_rows in (len(tokens), 1):
        difference = model.rounded_logits(tokens, roundings([step_rows] * len(tokens))) - exact
        worst_max = max(worst_max, np.abs(difference).max() / np.abs(exact).max())
        worst_rms = max(worst_rms, np.sqrt(np.mean(difference ** 2, axis=1)).max() / np.sqrt(np.mean(exact ** 2)))
    return worst_max, worst_rms


def kept_positions(length):
    """The places whose logits are compared: around page and tile edges, every eleventh, and the last 40."""
    edges = [p for edge in (0, 16, 64, 128, 256) for p in (edge - 1, edge, edge + 1) if 0 <= p < length]
    return set(edges) | set(range(0, length, 11)) | set(range(max(0, length - 40), length))


def run_steps(engine, steps, keep):
    """The trace's steps through ``Engine.step``; logits by (request, position) at the kept places."""
    from microllm_rocm_amd.engine.batch import StepEntry
    fed, rows = {}, {}
    for step in steps:
        entries, wanted = [], []
        for item in step["entries"]:
            rid, first = item["id"], fed.get(item["id"], 0)
            if not engine.is_open(rid):
                engine.open(rid)
            places = [place for place in item["want"] if first + place in keep[rid]]
            entries.append(StepEntry(rid, list(item["tokens"]), places))
            wanted += [(rid, first + place) for place in places]
            fed[rid] = first + len(item["tokens"])
        logits = engine.step(entries)
        if wanted:
            for key, row in zip(wanted, logits.to("cpu").numpy()):
                assert key not in rows
                rows[key] = row
        for rid in step["end"]:
            engine.close(rid)
            fed.pop(rid, None)
    engine.cache.check()
    assert not engine.cache.requests
    return rows


def test_every_cut_gives_the_same_bits_at_full_depth_and_bfloat16_stays_close(tmp_path):
    from microllm_rocm_amd.engine import Engine
    requests = {rid: random_tokens(900 + index, length, FULL_7B.vocab_size) for index, (rid, length) in enumerate(LENGTHS.items())}
    keep = {rid: kept_positions(len(tokens)) for rid, tokens in requests.items()}
    mixed_steps, peak = mixed(requests, seed=6, max_portion=40, decode_tail=12)
    assert max(len(step["entries"]) for step in mixed_steps) == 4
    pool_tokens = max(peak, 384)
    exact = Engine.from_random(FULL_7B, seed=3, dtype="float32", on_device=True, page_size=16, max_tokens=pool_tokens, max_requests=8)
    assert exact.dtype == torch.float32 and len(exact.model.blocks) == 28

    alone = run_steps(exact, whole(requests), keep)
    assert set(alone) == {(rid, p) for rid in requests for p in keep[rid]}
    assert all(np.all(np.isfinite(row)) for row in alone.values())
    cuts = {
        "portions": portions("a", requests["a"], sizes=[7, 2, 5, 16, 3, 2, 33, 2, 17, 64]),
        "prefill then single tokens": prefill_then_decode("a", requests["a"], tail=32),
    }
    for name, steps in cuts.items():
        rows = run_steps(exact, steps, keep)
        assert set(rows) == {("a", p) for p in keep["a"]}
        for key, row in rows.items():
            assert np.array_equal(row, alone[key]), f"{name}: {key} differs from the request run whole"
    pool = exact.cache.groups[0].pool
    taken_before = pool.total_taken
    rows = run_steps(exact, mixed_steps, keep)
    assert pool.total_taken - taken_before > pool.num_pages, "the pool is small enough for pages to be used again"
    assert set(rows) == set(alone)
    for key, row in rows.items():
        assert np.array_equal(row, alone[key]), f"mixed: {key} differs from the request run alone"
    del exact, rows
    torch.cuda.empty_cache()

    # bfloat16 on the same weights (the same seed draws the same bfloat16 tensors), against the 32-bit engine
    served = Engine.from_random(FULL_7B, seed=3, dtype="bfloat16", on_device=True, page_size=16, max_tokens=pool_tokens, max_requests=8)
    format_max, format_rms = what_rounding_costs_at_this_depth(os.path.join(str(tmp_path), "narrow"), requests["a"])
    assert 2e-2 < format_max < 1e-1 and 2e-2 < format_rms < 1.5e-1      # the root of the depth times the two-layer figures
    bound = {"max": 1.5 * format_max, "rms": 1.5 * format_rms}
    worst = {"max": 0.0, "rms": 0.0}
    for name, steps in (("whole", whole(requests)), ("prefill then single tokens", cuts["prefill then single tokens"]),
                        ("mixed", mixed_steps)):
        rows = run_steps(served, steps, keep)
        for rid in requests:
            reference = np.stack([alone[(rid, p)] for p in sorted(keep[rid])]).astype(np.float64)
            scale, rms_scale = np.abs(reference).max(), np.sqrt(np.mean(reference ** 2))
            for p in sorted(keep[rid]):
                if (rid, p) not in rows:
                    continue
                difference = rows[(rid, p)].astype(np.float64) - alone[(rid, p)]
                error_max, error_rms = np.abs(difference).max() / scale, np.sqrt(np.mean(difference ** 2)) / rms_scale
                assert error_max <= bound["max"] and error_rms <= bound["rms"], (
                    f"bfloat16, {name}: request {rid} position {p}: max error {error_max:.3e} (bound {bound['max']:.3e}), "
                    f"rms error {error_rms:.3e} (bound {bound['rms']:.3e})")
                worst = {"max": max(worst["max"], error_max), "rms": max(worst["rms"], error_rms)}
    # and not suspiciously close either: a bfloat16 engine that was nearer the 32-bit one than a third of what the
    # format costs would not be rounding where it says it does
    assert worst["max"] > format_max / 3
