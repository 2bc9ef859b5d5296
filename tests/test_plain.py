"""Pins of the plain implementation: vectors the reference's tests hold, special cases that reduce to a
library routine, and invariants, each chosen so that a plausible mistake fails it. No GPU."""
import math

import numpy as np
import pytest

import plain_qwen2 as plain


# ---- vectors held by the reference's own tests ---------------------------------------------------
def test_rms_norm_vector():
    # tests/ops/ops_test.cpp:480-485
    out = plain.rms_norm(np.array([[3.0, 4.0]]), np.array([1.0, 2.0]), 1e-5)
    denominator = math.sqrt(12.5 + 1e-5)
    np.testing.assert_allclose(out, [[3.0 / denominator, 8.0 / denominator]], rtol=1e-12)


def test_rms_norm_eps_is_inside_the_root():
    # eps outside the root (1/(sqrt(ms)+eps)) or a weight before the scaling would give another number here
    x = np.array([[1e-3, -1e-3]])
    out = plain.rms_norm(x, np.array([1.0, 1.0]), 1e-2)
    np.testing.assert_allclose(out, x / math.sqrt(1e-6 + 1e-2), rtol=1e-12)


def test_silu_vector():
    # tests/ops/ops_test.cpp:487-495
    out = plain.silu(np.array([-1.0, 0.0, 1.0]))
    np.testing.assert_allclose(out, [-1.0 / (1.0 + math.e), 0.0, 1.0 / (1.0 + math.exp(-1.0))], rtol=1e-12)
    big = plain.silu(np.array([-800.0, 800.0]))
    assert np.all(np.isfinite(big)) and big[1] == 800.0 and abs(big[0]) < 1e-300


def test_swiglu_special_cases():
    x = np.random.default_rng(0).normal(size=(3, 4))
    eye = np.eye(4)
    # up = 1 -> silu(gate): with W_up = 0 the product is zero; with gate = 0 it is zero too
    assert np.all(plain.swiglu_ffn(x, eye, np.zeros((4, 4)), eye) == 0.0)
    assert np.all(plain.swiglu_ffn(x, np.zeros((4, 4)), eye, eye) == 0.0)
    np.testing.assert_allclose(plain.swiglu_ffn(x, eye, eye, eye), plain.silu(x) * x, rtol=1e-12)


def test_rope_split_half_vector():
    # tests/ops/ops_test.cpp:505-515: {1,2,3,4} at p=0 is unchanged; {5,6,7,8} at p=1, hd=4, base 10000
    x = np.array([[[1.0, 2.0, 3.0, 4.0]], [[5.0, 6.0, 7.0, 8.0]]])
    out = plain.rope_split_half(x, np.array([0, 1]), 10000.0)
    np.testing.assert_array_equal(out[0, 0], [1.0, 2.0, 3.0, 4.0])
    assert out[1, 0, 0] == pytest.approx(5 * math.cos(1.0) - 7 * math.sin(1.0), rel=1e-12)
    assert out[1, 0, 2] == pytest.approx(5 * math.sin(1.0) + 7 * math.cos(1.0), rel=1e-12)
    angle = 10000.0 ** (-2.0 / 4.0)
    assert out[1, 0, 1] == pytest.approx(6 * math.cos(angle) - 8 * math.sin(angle), rel=1e-12)
    assert out[1, 0, 3] == pytest.approx(6 * math.sin(angle) + 8 * math.cos(angle), rel=1e-12)


def test_embedding_vector():
    # tests/ops/ops_test.cpp:465-470
    table = np.arange(6.0).reshape(3, 2)
    np.testing.assert_array_equal(plain.embedding(table, [2, 0, 1]), [[4, 5], [0, 1], [2, 3]])


def test_attention_two_key_closed_form():
    # tests/ops/ops_test.cpp:274-296: keys = values = {3,4} then {1,0}; queries e0 and e1 share the kv head; scale 1
    k = np.array([[[3.0, 4.0]], [[1.0, 0.0]]])
    q = np.zeros((2, 2, 2))
    q[1, 0] = [1.0, 0.0]
    q[1, 1] = [0.0, 1.0]
    out = plain.causal_gqa_attention(q, k, k, 1.0)
    p1 = math.exp(3.0) / (math.exp(3.0) + math.exp(1.0))
    p2 = math.exp(4.0) / (math.exp(4.0) + 1.0)
    np.testing.assert_allclose(out[1, 0], [p1 * 3 + (1 - p1), p1 * 4], rtol=1e-12)
    np.testing.assert_allclose(out[1, 1], [p2 * 3 + (1 - p2), p2 * 4], rtol=1e-12)
    # one visible key: the output is its value
    np.testing.assert_allclose(out[0, 0], [3.0, 4.0])


def test_argmax_ties_and_sampling_rules():
    # tests/ops/ops_test.cpp:414-439: the smallest index among equal maxima
    assert plain.greedy(np.array([-2.0, 5.0, 5.0, 4.0])) == 1
    logits = np.array([0.1, 2.0, -1.0, 1.5, 0.3])
    assert plain.sample(logits, 0.0, 0, 0.7) == 1
    assert plain.sample(logits, 1.0, 1, 0.7) == 1
    # top_k = 3 never yields an excluded index (tests/inference/generator_test.cpp:31-42)
    for draw in range(200):
        assert plain.sample(logits, 1.0, 3, plain.uniform_for(7, draw)) in (1, 3, 4)
    # the same seed gives the same draws
    assert [plain.uniform_for(3, d) for d in range(5)] == [plain.uniform_for(3, d) for d in range(5)]
    assert all(0.0 <= plain.uniform_for(s, d) < 1.0 for s in range(4) for d in range(50))


def test_sampling_frequencies_follow_softmax():
    logits = np.array([1.0, 0.0, -1.0, 0.5])
    temperature = 0.8
    counts = np.zeros(4)
    draws = 20000
    for draw in range(draws):
        counts[plain.sample(logits, temperature, 0, plain.uniform_for(11, draw))] += 1
    expected = np.exp(logits / temperature)
    expected /= expected.sum()
    np.testing.assert_allclose(counts / draws, expected, atol=0.01)


# ---- special cases that reduce to a library routine -----------------------------------------------
def _softmax(x):
    e = np.exp(x - x.max(axis=-1, keepdims=True))
    return e / e.sum(axis=-1, keepdims=True)


def test_attention_equals_masked_softmax_with_repeated_heads():
    rng = np.random.default_rng(1)
    tokens, heads, kv_heads, hd = 9, 6, 2, 8
    q, k, v = rng.normal(size=(tokens, heads, hd)), rng.normal(size=(tokens, kv_heads, hd)), rng.normal(size=(tokens, kv_heads, hd))
    out = plain.causal_gqa_attention(q, k, v, 0.37)
    k_rep, v_rep = np.repeat(k, heads // kv_heads, axis=1), np.repeat(v, heads // kv_heads, axis=1)
    mask = np.triu(np.full((tokens, tokens), -np.inf), 1)
    for head in range(heads):
        expected = _softmax(q[:, head] @ k_rep[:, head].T * 0.37 + mask) @ v_rep[:, head]
        np.testing.assert_allclose(out[:, head], expected, rtol=1e-10, atol=1e-12)
    # the last query sees every key: plain attention without a mask
    last = _softmax(q[-1, 0] @ k[:, 0].T * 0.37) @ v[:, 0]
    np.testing.assert_allclose(out[-1, 0], last, rtol=1e-10)


def test_attention_scale_zero_is_the_mean_of_visible_values():
    rng = np.random.default_rng(2)
    q, k, v = rng.normal(size=(5, 2, 4)), rng.normal(size=(5, 1, 4)), rng.normal(size=(5, 1, 4))
    out = plain.causal_gqa_attention(q, k, v, 0.0)
    for p in range(5):
        np.testing.assert_allclose(out[p, 1], v[:p + 1, 0].mean(axis=0), rtol=1e-12)


def test_window_rules():
    rng = np.random.default_rng(3)
    q, k, v = rng.normal(size=(12, 2, 4)), rng.normal(size=(12, 2, 4)), rng.normal(size=(12, 2, 4))
    full = plain.causal_gqa_attention(q, k, v, 0.5)
    np.testing.assert_array_equal(plain.causal_gqa_attention(q, k, v, 0.5, window=12), full)   # W >= length: no window
    np.testing.assert_allclose(plain.causal_gqa_attention(q, k, v, 0.5, window=1), v, rtol=1e-12)  # W = 1: own value
    windowed = plain.causal_gqa_attention(q, k, v, 0.5, window=4)
    np.testing.assert_array_equal(windowed[:4], full[:4])             # the first W positions see all their keys
    expected = _softmax(q[9, 0] @ k[6:10, 0].T * 0.5) @ v[6:10, 0]    # p = 9 sees j = 6..9: p - j < 4
    np.testing.assert_allclose(windowed[9, 0], expected, rtol=1e-10)
    assert np.abs(windowed[9, 0] - full[9, 0]).max() > 1e-3


def test_attention_in_blocks_is_the_row_by_row_formula():
    """Long sequences take ``causal_gqa_attention_in_blocks``; it must be the row-by-row function, also where a
    block's first query and the window's edge fall inside a block of keys, and with sharp scores."""
    rng = np.random.default_rng(4)
    tokens, heads, kv_heads, hd = 150, 6, 2, 8
    q, k, v = rng.normal(size=(tokens, heads, hd)) * 3, rng.normal(size=(tokens, kv_heads, hd)), rng.normal(size=(tokens, kv_heads, hd))
    assert tokens <= plain.ROW_BY_ROW_LIMIT
    for window in (None, 1, 7, 64, 149, 150, 1000):
        for block in (1, 32, 37, 256):
            rows = plain.causal_gqa_attention(q, k, v, 0.4, window)
            blocks = plain.causal_gqa_attention_in_blocks(q, k, v, 0.4, window, block=block)
            np.testing.assert_allclose(blocks, rows, rtol=1e-11, atol=1e-13)
    long = plain.ROW_BY_ROW_LIMIT + 5       # beyond the limit the public function is the blocked one
    q, k, v = rng.normal(size=(long, 2, 4)), rng.normal(size=(long, 1, 4)), rng.normal(size=(long, 1, 4))
    np.testing.assert_array_equal(plain.causal_gqa_attention(q, k, v, 0.5, 100),
                                  plain.causal_gqa_attention_in_blocks(q, k, v, 0.5, 100))


def test_rope_reduces_to_a_plane_rotation_for_head_dim_two():
    x = np.array([[[1.0, 0.0]], [[0.0, 2.0]]])
    out = plain.rope_split_half(x, np.array([3, 3]), 77.0)   # hd = 2: one pair, frequency 1
    np.testing.assert_allclose(out[0, 0], [math.cos(3.0), math.sin(3.0)], rtol=1e-12)
    np.testing.assert_allclose(out[1, 0], [-2 * math.sin(3.0), 2 * math.cos(3.0)], rtol=1e-12)


# ---- invariants ---------------------------------------------------------------------------------------
def test_rope_scores_depend_on_distance_only():
    rng = np.random.default_rng(4)
    q, k = rng.normal(size=(1, 1, 16)), rng.normal(size=(1, 1, 16))

    def score(p, s):
        return float(plain.rope_split_half(q, np.array([p]), 1e4)[0, 0] @ plain.rope_split_half(k, np.array([s]), 1e4)[0, 0])

    assert score(17, 5) == pytest.approx(score(112, 100), rel=1e-9)
    assert score(17, 5) != pytest.approx(score(17, 6), rel=1e-3)
    rotated = plain.rope_split_half(q, np.array([9]), 1e4)
    assert np.linalg.norm(rotated) == pytest.approx(np.linalg.norm(q), rel=1e-12)   # a rotation keeps the norm


def _tiny_model(seed=0, tie=False, window=None, layers=2):
    rng = np.random.default_rng(seed)
    config = {"vocab_size": 50, "hidden_size": 24, "num_hidden_layers": layers, "num_attention_heads": 3,
              "num_key_value_heads": 1, "head_dim": 8, "intermediate_size": 40, "rope_theta": 1e4,
              "rms_norm_eps": 1e-5, "tie_word_embeddings": tie, "use_sliding_window": window is not None,
              "sliding_window": window, "max_window_layers": 1}
    w = {"model.embed_tokens.weight": rng.normal(0, 0.3, (50, 24)), "model.norm.weight": 1 + rng.normal(0, 0.1, 24)}
    if not tie:
        w["lm_head.weight"] = rng.normal(0, 0.3, (50, 24))
    for i in range(layers):
        p = f"model.layers.{i}"
        w[f"{p}.input_layernorm.weight"] = 1 + rng.normal(0, 0.1, 24)
        w[f"{p}.post_attention_layernorm.weight"] = 1 + rng.normal(0, 0.1, 24)
        for role, rows in (("q", 24), ("k", 8), ("v", 8)):
            w[f"{p}.self_attn.{role}_proj.weight"] = rng.normal(0, 0.3, (rows, 24))
            w[f"{p}.self_attn.{role}_proj.bias"] = rng.normal(0, 0.3, rows)
        w[f"{p}.self_attn.o_proj.weight"] = rng.normal(0, 0.3, (24, 24))
        w[f"{p}.mlp.gate_proj.weight"] = rng.normal(0, 0.3, (40, 24))
        w[f"{p}.mlp.up_proj.weight"] = rng.normal(0, 0.3, (40, 24))
        w[f"{p}.mlp.down_proj.weight"] = rng.normal(0, 0.3, (24, 40))
    return config, w


def test_causality_is_exact():
    # tests/model/model_test.cpp:263-274: changing later tokens leaves earlier logits bit-equal
    config, w = _tiny_model()
    a = plain.forward(config, w, [1, 2, 3, 4, 5, 6])
    b = plain.forward(config, w, [1, 2, 3, 4, 40, 41])
    np.testing.assert_array_equal(a[:4], b[:4])
    assert np.abs(a[4:] - b[4:]).max() > 1e-3


def test_shifting_all_positions_changes_nothing_in_a_layer():
    # Only distances count: a layer's output for positions p..p+T-1 equals that for 0..T-1. This fails when the
    # rotation pairs (i, i+1) instead of (i, i+hd/2) in only q or k, or when v is rotated.
    config, w = _tiny_model(5)
    rng = np.random.default_rng(6)
    x = rng.normal(size=(7, 24))
    base = plain.attention_layer(x, w, "model.layers.0", config, None)
    heads, kv_heads, hd = 3, 1, 8

    def shifted(offset):
        positions = np.arange(7) + offset
        def project(role, count):
            return plain.linear(x, w[f"model.layers.0.self_attn.{role}_proj.weight"],
                                w[f"model.layers.0.self_attn.{role}_proj.bias"]).reshape(7, count, hd)
        q = plain.rope_split_half(project("q", heads), positions, 1e4)
        k = plain.rope_split_half(project("k", kv_heads), positions, 1e4)
        o = plain.causal_gqa_attention(q, k, project("v", kv_heads), 1 / math.sqrt(hd))
        return plain.linear(o.reshape(7, heads * hd), w["model.layers.0.self_attn.o_proj.weight"])

    np.testing.assert_allclose(shifted(0), base, rtol=1e-12)
    np.testing.assert_allclose(shifted(1000), base, rtol=1e-7, atol=1e-9)


def test_tied_head_uses_the_embedding_and_window_changes_late_positions_only():
    config, w = _tiny_model(7, tie=True)
    logits = plain.forward(config, w, [3, 1, 4, 1, 5])
    h = plain.embedding(w["model.embed_tokens.weight"], [3, 1, 4, 1, 5])
    for i in range(2):
        h = plain.block(h, w, i, config, None)
    np.testing.assert_allclose(logits, plain.rms_norm(h, w["model.norm.weight"], 1e-5) @ w["model.embed_tokens.weight"].T,
                               rtol=1e-12)
    config_w, w_w = _tiny_model(8, window=3)
    config_n = dict(config_w, use_sliding_window=False)
    tokens = list(range(10))
    a, b = plain.forward(config_w, w_w, tokens), plain.forward(config_n, w_w, tokens)
    np.testing.assert_array_equal(a[:3], b[:3])    # within the window nothing differs
    assert np.abs(a[5:] - b[5:]).max() > 1e-4
    assert plain.layer_windows(config_w) == [None, 3]   # layer 0 < max_window_layers keeps every key


def test_block_is_pre_norm():
    # With a zero output projection and a zero down projection the block is the identity: a post-norm block,
    # or one that normalises the residual stream itself, would not be.
    config, w = _tiny_model(9)
    w["model.layers.0.self_attn.o_proj.weight"][:] = 0
    w["model.layers.0.mlp.down_proj.weight"][:] = 0
    h = np.random.default_rng(1).normal(size=(4, 24)) * 5
    np.testing.assert_array_equal(plain.block(h, w, 0, config, None), h)


def test_generate_greedy_extends_by_argmax():
    config, w = _tiny_model(10)
    out = plain.generate_greedy(config, w, [1, 2, 3], 4)
    assert len(out) == 4
    assert out[0] == int(np.argmax(plain.forward(config, w, [1, 2, 3])[-1]))
    assert out[1] == int(np.argmax(plain.forward(config, w, [1, 2, 3, out[0]])[-1]))


def test_layer_streams_end_in_the_logits():
    config, w = _tiny_model(11)
    tokens = [3, 1, 4, 1, 5, 9]
    streams = plain.layer_streams(config, w, tokens)
    assert streams.shape == (config["num_hidden_layers"], len(tokens), config["hidden_size"])
    h = plain.embedding(w["model.embed_tokens.weight"], tokens)
    np.testing.assert_array_equal(streams[0], plain.block(h, w, 0, config, plain.layer_windows(config)[0]))
    head = w["model.embed_tokens.weight"] if config["tie_word_embeddings"] else w["lm_head.weight"]
    np.testing.assert_allclose(plain.forward(config, w, tokens),
                               plain.rms_norm(streams[-1], w["model.norm.weight"], config["rms_norm_eps"]) @ head.T, rtol=1e-12)
