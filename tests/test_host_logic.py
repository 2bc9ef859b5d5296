"""Host-side rules that need no GPU: how the products split their work, the row order of a rotary weight, and how
parts take their tensors from the loader."""
import numpy as np
import pytest
import torch

from microllm_rocm_amd.architectures.qwen2 import build_spec, init_rules
from microllm_rocm_amd.ops import kernels
from microllm_rocm_amd.parts import Model, Runtime
from microllm_rocm_amd.parts.linear import MEDIUM_GATED_ROWS, MEDIUM_ROWS, SKINNY_ROWS, Weight, takes_packed, takes_unscaled
from microllm_rocm_amd.weights.random_init import random_tensors
from tiny import TINY_A, TINY_B


@pytest.mark.parametrize("n,k", [(4608, 3584), (3584, 18944), (37888, 3584), (152064, 3584), (256, 64), (896, 4864), (8192, 29568), (331, 120)])
def test_medium_plan_depends_on_the_weight_alone_and_is_launchable(n, k):
    tiles, waves, splits = kernels.medium_plan(n, k)
    assert tiles in (1, 2) and waves == 8
    assert 1 <= splits <= 16 and splits & (splits - 1) == 0
    assert splits <= max(1, -(-k // 256)), "a split takes at least one stage of 256"
    assert kernels.medium_plan(n, k, may_split=False)[2] == 1
    groups = -(-(-(-n // 16)) // (8 * tiles))
    if splits > 1:
        assert groups * (splits // 2) < kernels.MEDIUM_WORKGROUPS, "no more splits than the GPU needs"


@pytest.mark.parametrize("m,n,k,parts", [
    (2048, 3584, 18944, 2), (1024, 3584, 18944, 4), (512, 3584, 18944, 8), (65, 3584, 18944, 8),     # a long reduction into a narrow result
    (4096, 3584, 18944, 4), (8192, 3584, 18944, 4),                                                   # a last round of tiles that is not full
    (2048, 3584, 3584, 1), (2048, 4608, 3584, 1), (512, 3584, 3584, 1),                               # short reductions stay whole
    (2048, 8192, 29568, 1), (4096, 8192, 29568, 1), (512, 8192, 29568, 2), (256, 8192, 8192, 4),      # wide results fill the GPU by themselves
    (2048, 896, 4864, 2), (8192, 896, 4864, 1), (100, 331, 120, 1), (300, 64, 4160, 2), (300, 64, 4128, 1)])
def test_library_splits(m, n, k, parts):
    assert kernels.library_splits(m, n, k) == parts
    assert k % parts == 0 and (parts == 1 or k // parts >= kernels.LIBRARY_SPLIT_LENGTH)


@pytest.mark.parametrize("m,n,k,splits", [(512, 3584, 3584, 4), (512, 3584, 18944, 8), (2048, 3584, 18944, 2), (2048, 37888, 3584, 1),
                                          (300, 64, 512, 1), (100, 8192, 8192, 4), (4096, 8192, 29568, 1)])
def test_tiled_splits(m, n, k, splits):
    assert kernels.tiled_splits(m, n, k) == splits
    assert -(-k // 64) // splits >= (kernels.TILED_SPLIT_STAGES if splits > 1 else 0)


@pytest.mark.parametrize("tokens,kv_heads,longest,splits", [(1, 4, 4096, 8), (8, 4, 4096, 4), (64, 4, 4096, 1), (32, 4, 16384, 2),
                                                            (16, 4, 4096, 4), (1, 2, 300, 1), (1, 1, 100000, 195), (3, 8, 1024, 2)])
def test_decode_splits(tokens, kv_heads, longest, splits):
    assert kernels.decode_splits(tokens, kv_heads, longest) == splits


def test_query_tiles_go_in_twos_that_walk_about_as_many_keys():
    # one prompt of 2048 tokens from position 0 (16 tiles), a portion of 300 from position 1000, one tile alone
    tiles = [(0, offset, 128, offset) for offset in range(0, 2048, 128)]
    tiles += [(1, 2048 + offset, min(128, 300 - offset), 1000 + offset) for offset in range(0, 300, 128)] + [(2, 2348, 17, 40)]
    pairs = kernels.pair_query_tiles(list(tiles))
    covered = sorted((r, first, count) for r, a, ca, b, cb in pairs for first, count in ((a, ca), (b, cb)) if count)
    assert covered == sorted(tile[:3] for tile in tiles), "every tile once"
    of_first = [pair for pair in pairs if pair[0] == 0]
    position = {tile[1]: tile[3] for tile in tiles}
    weights = [position[a] + ca + position[b] + cb for _, a, ca, b, cb in of_first]
    assert len(of_first) == 8 and max(weights) == min(weights) == 2048 + 128, "late with early: all the same"
    assert [pair for pair in pairs if pair[0] == 2] == [(2, 2348, 17, 0, 0)]
    assert sorted(pair[1:] for pair in pairs if pair[0] == 1) == [(2048 + 128, 128, 0, 0), (2048 + 256, 44, 2048, 128)]
    keys = [position[a] + ca + (position[b] + cb if cb else 0) for _, a, ca, b, cb in pairs]
    assert keys == sorted(keys, reverse=True), "the longest first"
    # under a window neighbours go together
    adjacent = kernels.pair_query_tiles(list(tiles), adjacent=True)
    assert sorted(pair[1:] for pair in adjacent if pair[0] == 0) == [(offset, 128, offset + 128, 128) for offset in range(0, 2048, 256)]
    assert sorted(pair[1:] for pair in adjacent if pair[0] == 1) == [(2048, 128, 2048 + 128, 128), (2048 + 256, 44, 0, 0)]


@pytest.mark.parametrize("heads,kv_heads,hd,n_freq", [(4, 2, 16, 8), (3, 1, 32, 8), (28, 4, 128, 64), (2, 0, 64, 32), (5, 5, 48, 0)])
def test_rotary_pair_order_puts_partners_side_by_side(heads, kv_heads, hd, n_freq):
    order = kernels.rotary_pair_order(heads, kv_heads, hd, n_freq).tolist()
    total = (heads + 2 * kv_heads) * hd
    assert sorted(order) == list(range(total))
    for head in range(heads + 2 * kv_heads):
        rows = [row - head * hd for row in order[head * hd:(head + 1) * hd]]
        if head < heads + kv_heads:
            for pair in range(n_freq):
                assert rows[2 * pair] == pair and rows[2 * pair + 1] == pair + n_freq
            assert rows[2 * n_freq:] == list(range(2 * n_freq, hd))
        else:
            assert rows == list(range(hd)), "value heads stay as they are"


def test_parts_take_their_tensors_out_of_the_dict_as_they_bind():
    for config in (TINY_A, TINY_B):        # A ties the head to the embedding: that table is looked up twice
        spec = build_spec(config)
        model = Model(spec, Runtime(torch.float32, torch.device("cpu")))
        tensors = random_tensors(model.tensors(), init_rules(config), 0, dtype=torch.float32)
        names = set(tensors)
        untouched = dict(tensors)
        model.bind(tensors, consume=True)
        assert not tensors, "every declared tensor was handed over"
        assert model.embedding.table is untouched["model.embed_tokens.weight"]
        if config.tie_word_embeddings:
            assert model.head.weight.tensor is model.embedding.table
        # without consume the dict is left as it was
        again = Model(spec, Runtime(torch.float32, torch.device("cpu")))
        again.bind(untouched)
        assert set(untouched) == names


def test_which_product_a_linear_takes():
    plain = Weight(torch.zeros((64, 32), dtype=torch.bfloat16))          # on the host nothing is packed
    assert plain.packed is None and not takes_packed(plain, 1) and not takes_unscaled(plain, 1)
    packed = Weight(torch.zeros((64, 32), dtype=torch.bfloat16), pack=False)
    packed.packed = torch.zeros((4, 1, 4, 16, 8), dtype=torch.bfloat16)   # as on the GPU
    assert takes_packed(packed, SKINNY_ROWS) and takes_packed(packed, MEDIUM_ROWS) and not takes_packed(packed, MEDIUM_ROWS + 1)
    assert takes_packed(packed, MEDIUM_GATED_ROWS, gated=True) and not takes_packed(packed, MEDIUM_GATED_ROWS + 1, gated=True), \
        "the gated product goes to the library (and the SiLU kernel) beyond this many rows"
    assert takes_unscaled(packed, SKINNY_ROWS) and not takes_unscaled(packed, SKINNY_ROWS + 1)
    packed.tensor = None                                                   # one copy: the packed one serves every step
    assert takes_packed(packed, 5000) and takes_packed(packed, 40, gated=True)
    wide = Weight(torch.zeros((16, 8), dtype=torch.bfloat16), pack=False)
    wide.packed, wide.out_features = packed.packed, 2048 * 16
    assert takes_packed(wide, 40) and not takes_packed(wide, 41), "weights with many tiles go to the library from 41 rows on"


def test_percentile_interpolates_between_the_two_nearest_sorted_values():
    from microllm_rocm_amd.cli.hf_infer import percentile
    assert percentile([4, 1, 3, 2], 0.5) == 2.5 and percentile([7.0], 0.95) == 7.0
    assert percentile([1, 2, 3, 4, 5], 0.95) == pytest.approx(4.8) and percentile([5, 1], 0.0) == 1 and percentile([5, 1], 1.0) == 5
    with pytest.raises(ValueError):
        percentile([], 0.5)


def test_padding_a_step_to_a_graph_shape_never_changes_the_kernel_a_product_takes():
    """A mixed step is padded to fixed numbers of token rows and of wanted rows before it is replayed from a graph;
    the padded count must take the same product as the real one, for every kind of weight, or the replayed step
    would give other bits than the same step run eagerly."""
    from microllm_rocm_amd.engine.engine import MAX_GRAPH_TOKENS, MAX_GRAPH_WANTED, _token_rows, _wanted_rows
    narrow = Weight(torch.zeros((64, 32), dtype=torch.bfloat16), pack=False)
    narrow.packed = torch.zeros((4, 1, 4, 16, 8), dtype=torch.bfloat16)
    wide = Weight(torch.zeros((16, 8), dtype=torch.bfloat16), pack=False)
    wide.packed, wide.out_features = narrow.packed, 2048 * 16

    def kernel_of(weight, rows, gated):
        return (rows <= SKINNY_ROWS, takes_unscaled(weight, rows), takes_packed(weight, rows, gated), rows <= MEDIUM_ROWS)

    for pad, most in ((_token_rows, MAX_GRAPH_TOKENS), (_wanted_rows, MAX_GRAPH_WANTED)):
        for rows in range(1, most + 1):
            padded = pad(rows)
            assert rows <= padded <= max(16, 2 * rows)
            for weight in (narrow, wide):
                for gated in (False, True):
                    assert kernel_of(weight, rows, gated) == kernel_of(weight, padded, gated), (pad.__name__, rows, padded)


def test_kept_graphs_stay_bounded_and_mixed_shapes_never_push_decode_graphs_out():
    """More recurring shapes than the budget holds: captures stay bounded (a shape that was captured and evicted
    twice runs eagerly from then on), decode graphs are not evicted by mixed ones, and both budgets hold in bytes."""
    from types import SimpleNamespace
    from microllm_rocm_amd.engine.graphs import MAX_CAPTURES_A_SHAPE, GraphPolicy
    policy = GraphPolicy(decode_graphs=4, mixed_graphs=3, most_bytes=1000, seen_before_capture=2)
    captures = 0
    for key in range(4):                                   # four decode shapes, captured once each
        policy.decode.put(("decode", key), SimpleNamespace(held_bytes=100))
    assert len(policy.decode) == 4
    shapes = [("mixed", index) for index in range(10)]      # ten mixed shapes that keep coming round
    for round_number in range(40):
        for key in shapes:
            if not policy.wants_mixed(key):
                continue
            if policy.mixed.get(key) is None:
                state = SimpleNamespace(held_bytes=0)
                policy.mixed.put(key, state, policy.evicted_mixed)
                state.held_bytes = 100                      # the capture
                captures += 1
                policy.captured_mixed(key)
                policy.mixed.trim(policy.evicted_mixed, keep=key)
            assert len(policy.mixed) <= 3 and policy.mixed.held_bytes() <= 500
    assert captures <= MAX_CAPTURES_A_SHAPE * len(shapes), "no shape is captured over and over"
    assert len(policy.decode) == 4 and all(("decode", key) in policy.decode for key in range(4))
    assert all(not policy.wants_mixed(key) or key in policy.mixed for key in shapes), "evicted twice: eagerly for good"
    # a shape seen once is not captured; the second time it is
    fresh = GraphPolicy(seen_before_capture=2)
    assert not fresh.wants_mixed("s") and fresh.wants_mixed("s")
    # the budget in bytes: a graph of large logits pushes older ones out, the one in use stays
    small = GraphPolicy(decode_graphs=8, mixed_graphs=8, most_bytes=600)
    for key in range(3):
        small.decode.put(key, SimpleNamespace(held_bytes=100))
    small.decode.put("large", SimpleNamespace(held_bytes=250))
    assert "large" in small.decode and small.decode.held_bytes() <= 300 and 0 not in small.decode
