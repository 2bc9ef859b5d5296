"""Host-side rules that need no GPU: how the products split their work, the row order of a rotary weight, and how
parts take their tensors from the loader."""
import numpy as np
import pytest
import torch

from microllm_rocm_amd.architectures.qwen2 import build_spec, init_rules
from microllm_rocm_amd.ops import kernels
from microllm_rocm_amd.parts import Model, Runtime
from microllm_rocm_amd.parts.linear import MEDIUM_ROWS, SKINNY_ROWS, Weight, takes_packed, takes_unscaled
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
    assert not takes_packed(packed, SKINNY_ROWS + 1, gated=True), "the gated product of 17 to 64 rows is the library's"
    assert takes_unscaled(packed, SKINNY_ROWS) and not takes_unscaled(packed, SKINNY_ROWS + 1)
    packed.tensor = None                                                   # one copy: the packed one serves every step
    assert takes_packed(packed, 5000) and takes_packed(packed, 40, gated=True)
    wide = Weight(torch.zeros((16, 8), dtype=torch.bfloat16), pack=False)
    wide.packed, wide.out_features = packed.packed, 2048 * 16
    assert takes_packed(wide, 40) and not takes_packed(wide, 41), "weights with many tiles go to the library from 41 rows on"
