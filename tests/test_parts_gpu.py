"""Each part alone against its plain function, built from a spec with sizes that no tiny model uses; then
models whose run order names a layer twice or lets a layer read another layer's cache."""
import math
import os

import numpy as np
import pytest
import torch

import plain_qwen2 as plain
from tiny import TINY_B
from microllm_rocm_amd.architectures.qwen2 import build_spec
from microllm_rocm_amd.cache import CacheManager
from microllm_rocm_amd.engine import Engine, StepEntry
from microllm_rocm_amd.engine.batch import BatchBuilder
from microllm_rocm_amd.parts import LayerSpec, ModelSpec, PartSpec, RunEntry, Runtime, build_block, build_part
from microllm_rocm_amd.weights import random_tensors
from microllm_rocm_amd.weights.random_init import InitRule

pytestmark = pytest.mark.gpu

DEVICE = torch.device("cuda:0")
TOL = {torch.float32: dict(rtol=2e-5, atol=2e-5), torch.bfloat16: dict(rtol=3e-2, atol=3e-2)}


def bf16_exact(array):
    return torch.from_numpy(np.asarray(array, dtype=np.float32)).to(torch.bfloat16)


def runtime(dtype):
    return Runtime(dtype=dtype, device=DEVICE)


def bind(part, arrays, dtype):
    """Values rounded to bfloat16 so both engines and the plain functions see the same numbers."""
    tensors, exact = {}, {}
    for name, decl in part.tensors().items():
        value = bf16_exact(arrays[name])
        exact[name] = value.double().numpy()
        keep = torch.float32 if (decl.kind == "vector" or dtype == torch.float32) else torch.bfloat16
        tensors[name] = value.to(keep).to(DEVICE)
    part.bind(tensors)
    return exact


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rms_norm_part(dtype):
    rng = np.random.default_rng(0)
    part = build_part("norm", PartSpec("rms_norm", {"size": 200, "eps": 2e-4}, {"weight": "n.w"}), runtime(dtype))
    assert part.tensors()["n.w"].shape == (200,)
    exact = bind(part, {"n.w": 1 + 0.2 * rng.normal(size=200)}, dtype)
    h_ref = rng.normal(size=(9, 200)).astype(np.float32)
    delta_ref = bf16_exact(rng.normal(size=(9, 200)))
    h = torch.from_numpy(h_ref.copy()).to(DEVICE)
    out = part.forward(h, delta=delta_ref.to(dtype).to(DEVICE), write_h=True)
    total = h_ref.astype(np.float64) + delta_ref.double().numpy()
    assert out.dtype == dtype
    np.testing.assert_allclose(out.float().cpu().numpy(), plain.rms_norm(total, exact["n.w"], 2e-4), **TOL[dtype])
    np.testing.assert_allclose(h.cpu().numpy(), total, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_swiglu_part(dtype):
    rng = np.random.default_rng(1)
    names = {f"{r}_proj.weight": f"f.{r}" for r in ("gate", "up", "down")}
    part = build_part("ffn", PartSpec("swiglu", {"hidden_size": 72, "intermediate_size": 320}, names), runtime(dtype))
    exact = bind(part, {"f.gate": rng.normal(size=(320, 72)) * 0.3, "f.up": rng.normal(size=(320, 72)) * 0.3,
                        "f.down": rng.normal(size=(72, 320)) * 0.3}, dtype)
    for rows in (3, 40, 100):     # few rows take the streaming products, many the library's
        x = bf16_exact(rng.normal(size=(rows, 72)))
        out = part.forward(x.to(dtype).to(DEVICE), None)
        out = out.sum(dim=0) if out.dim() == 3 else out      # a delta may come as partial sums
        expected = plain.swiglu_ffn(x.double().numpy(), exact["f.gate"], exact["f.up"], exact["f.down"])
        np.testing.assert_allclose(out.float().cpu().numpy(), expected, rtol=TOL[dtype]["rtol"],
                                   atol=TOL[dtype]["atol"] * np.abs(expected).max())


def attention_case(dtype, heads, kv_heads, hd, hidden, window, theta, bias=True, page_size=16):
    rng = np.random.default_rng(heads * 10 + hd)
    names = {"o_proj.weight": "a.o"}
    arrays = {"a.o": rng.normal(size=(hidden, heads * hd)) * 0.2}
    for role, count in (("q", heads), ("k", kv_heads), ("v", kv_heads)):
        names[f"{role}_proj.weight"] = f"a.{role}"
        arrays[f"a.{role}"] = rng.normal(size=(count * hd, hidden)) * 0.25
        if bias:
            names[f"{role}_proj.bias"] = f"a.{role}b"
            arrays[f"a.{role}b"] = rng.normal(size=count * hd) * 0.3
    spec = PartSpec("paged_attention", {
        "hidden_size": hidden, "num_heads": heads, "num_kv_heads": kv_heads, "head_dim": hd, "qkv_bias": bias,
        "window": window, "scale": hd ** -0.5,
        "position": PartSpec("rope_split_half", {"theta": theta, "head_dim": hd})}, names)
    part = build_part("mixer", spec, runtime(dtype))
    exact = bind(part, arrays, dtype)
    weights = {"L.self_attn.o_proj.weight": exact["a.o"]}
    for role in ("q", "k", "v"):
        weights[f"L.self_attn.{role}_proj.weight"] = exact[f"a.{role}"]
        if bias:
            weights[f"L.self_attn.{role}_proj.bias"] = exact[f"a.{role}b"]
    config = {"num_attention_heads": heads, "num_key_value_heads": kv_heads, "head_dim": hd, "hidden_size": hidden,
              "rope_theta": theta}
    cache = CacheManager([part.cache_need()], [None], page_size, 12, 4, dtype=dtype, device=DEVICE)
    return part, cache, weights, config, rng


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv_heads,hd,hidden,window,bias", [(6, 2, 48, 104, None, True), (5, 1, 16, 40, 9, False),
                                                               (4, 4, 80, 96, 33, True)])
def test_attention_mixer_alone_in_portions(dtype, heads, kv_heads, hd, hidden, window, bias):
    part, cache, weights, config, rng = attention_case(dtype, heads, kv_heads, hd, hidden, window, 3e4, bias)
    assert part.cache_need().window == window and part.cache_need().kv_heads == kv_heads
    tokens = 70
    x = bf16_exact(rng.normal(size=(tokens, hidden)))
    expected = plain.attention_layer(x.double().numpy(), weights, "L", config, window)
    builder = BatchBuilder(cache, DEVICE)
    request = cache.open("r")
    binding = cache.bindings()[0]
    outputs = []
    position = 0
    for count in (17, 2, 30, 1, 1, 19):
        cache.reserve(request, count)
        ctx = builder.build([request], [[0] * count], [[]])
        out = part.forward(x[position:position + count].to(dtype).to(DEVICE), ctx, binding)
        outputs.append((out.sum(dim=0) if out.dim() == 3 else out).float().cpu())      # a delta may come as partial sums
        cache.commit(request, count)
        position += count
    got = torch.cat(outputs).numpy()
    np.testing.assert_allclose(got, expected, rtol=TOL[dtype]["rtol"], atol=TOL[dtype]["atol"] * np.abs(expected).max())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_pre_norm_block_alone(dtype):
    config = TINY_B.replace(use_sliding_window=False)
    spec = build_spec(config)
    block = build_block(spec.layers[1], runtime(dtype))
    rng = np.random.default_rng(3)
    arrays = {name: (1 + 0.1 * rng.normal(size=decl.shape)) if name.endswith("layernorm.weight")
              else rng.normal(size=decl.shape) * 0.15 for name, decl in block.tensors().items()}
    tensors, exact = {}, {}
    for name, decl in block.tensors().items():
        value = bf16_exact(arrays[name])
        exact[name] = value.double().numpy()
        keep = torch.float32 if (decl.kind == "vector" or dtype == torch.float32) else torch.bfloat16
        tensors[name] = value.to(keep).to(DEVICE)
    block.bind(tensors)
    cache = CacheManager([block.mixer.cache_need()], [None], 16, 8, 2, dtype=dtype, device=DEVICE)
    request = cache.open("r")
    cache.reserve(request, 25)
    ctx = BatchBuilder(cache, DEVICE).build([request], [[0] * 25], [[]])
    h_ref = rng.normal(size=(25, config.hidden_size)).astype(np.float32)
    h = torch.from_numpy(h_ref.copy()).to(DEVICE)
    pending = block.forward(h, None, ctx, cache.bindings()[0])
    pending = pending.sum(dim=0) if pending.dim() == 3 else pending       # a delta may come as partial sums
    total = h.double().cpu().numpy() + pending.double().cpu().numpy()      # the block hands its last delta on
    expected = plain.block(h_ref.astype(np.float64), exact, 1, config.to_dict(), None)
    np.testing.assert_allclose(total, expected, rtol=TOL[dtype]["rtol"], atol=TOL[dtype]["atol"] * np.abs(expected).max())


def test_few_rows_take_the_norm_between_two_products():
    """In bfloat16, with few rows, a block's last product begins the next norm and the next block's first product ends it."""
    from microllm_rocm_amd.parts.linear import UnscaledRows
    config = TINY_B.replace(use_sliding_window=False)
    spec = build_spec(config)
    dtype = torch.bfloat16
    rng = np.random.default_rng(5)
    blocks, exact = [], {}
    for index in (0, 1):
        block = build_block(spec.layers[index], runtime(dtype))
        tensors = {}
        for name, decl in block.tensors().items():
            array = (1 + 0.1 * rng.normal(size=decl.shape)) if name.endswith("layernorm.weight") else rng.normal(size=decl.shape) * 0.15
            value = bf16_exact(array)
            exact[name] = value.double().numpy()
            tensors[name] = value.to(torch.float32 if decl.kind == "vector" else torch.bfloat16).to(DEVICE)
        block.bind(tensors)
        blocks.append(block)
    needs = [block.mixer.cache_need() for block in blocks]
    cache = CacheManager(needs, [None, None], 16, 8, 2, dtype=dtype, device=DEVICE)
    request = cache.open("r")
    rows = 5
    cache.reserve(request, rows)
    ctx = BatchBuilder(cache, DEVICE).build([request], [[0] * rows], [[]])
    h_ref = rng.normal(size=(rows, config.hidden_size)).astype(np.float32)
    h = torch.from_numpy(h_ref.copy()).to(DEVICE)
    pending = blocks[0].forward(h, None, ctx, cache.bindings()[0], blocks[1])
    assert isinstance(pending, UnscaledRows)                   # the sum is in h already, the norm half done
    after_first = plain.block(h_ref.astype(np.float64), exact, 0, config.to_dict(), None)
    np.testing.assert_allclose(h.double().cpu().numpy(), after_first, rtol=TOL[dtype]["rtol"], atol=TOL[dtype]["atol"] * np.abs(after_first).max())
    pending = blocks[1].forward(h, pending, ctx, cache.bindings()[1], None)
    assert isinstance(pending, torch.Tensor)                   # no block follows: a plain delta (or partial sums)
    pending = pending.sum(dim=0) if pending.dim() == 3 else pending
    expected = plain.block(after_first, exact, 1, config.to_dict(), None)
    total = h.double().cpu().numpy() + pending.double().cpu().numpy()
    np.testing.assert_allclose(total, expected, rtol=TOL[dtype]["rtol"], atol=TOL[dtype]["atol"] * np.abs(expected).max())
    # with many rows the same blocks take the ordinary way
    cache.cancel_reservation(request)
    cache.close("r")
    request = cache.open("s")
    cache.reserve(request, 40)
    ctx = BatchBuilder(cache, DEVICE).build([request], [[0] * 40], [[]])
    h = torch.zeros((40, config.hidden_size), dtype=torch.float32, device=DEVICE)
    assert isinstance(blocks[0].forward(h, None, ctx, cache.bindings()[0], blocks[1]), torch.Tensor)


def qwen_like_layer(index, hidden, heads, kv_heads, hd, inter, window=None, owns_kv=True):
    prefix = f"model.layers.{index}"
    names = {"q_proj.weight": f"{prefix}.self_attn.q_proj.weight", "q_proj.bias": f"{prefix}.self_attn.q_proj.bias",
             "o_proj.weight": f"{prefix}.self_attn.o_proj.weight"}
    if owns_kv:
        for role in ("k", "v"):
            names[f"{role}_proj.weight"] = f"{prefix}.self_attn.{role}_proj.weight"
            names[f"{role}_proj.bias"] = f"{prefix}.self_attn.{role}_proj.bias"
    return LayerSpec(
        "pre_norm",
        PartSpec("rms_norm", {"size": hidden, "eps": 1e-5}, {"weight": f"{prefix}.input_layernorm.weight"}),
        PartSpec("paged_attention", {"hidden_size": hidden, "num_heads": heads, "num_kv_heads": kv_heads, "head_dim": hd,
                                     "qkv_bias": True, "window": window, "owns_kv": owns_kv,
                                     "position": PartSpec("rope_split_half", {"theta": 1e4, "head_dim": hd})}, names),
        PartSpec("rms_norm", {"size": hidden, "eps": 1e-5}, {"weight": f"{prefix}.post_attention_layernorm.weight"}),
        PartSpec("swiglu", {"hidden_size": hidden, "intermediate_size": inter},
                 {f"{r}_proj.weight": f"{prefix}.mlp.{r}_proj.weight" for r in ("gate", "up", "down")}))


def custom_model(order, owns_kv=(True, True, True)):
    hidden, heads, kv_heads, hd, inter, vocab = 48, 3, 1, 16, 80, 97
    sizes = {"vocab_size": vocab, "hidden_size": hidden}
    spec = ModelSpec("Custom", vocab, hidden, 256, PartSpec("token_embedding", sizes, {"weight": "model.embed_tokens.weight"}),
                     tuple(qwen_like_layer(i, hidden, heads, kv_heads, hd, inter, owns_kv=owns_kv[i]) for i in range(3)),
                     tuple(order), PartSpec("rms_norm", {"size": hidden, "eps": 1e-5}, {"weight": "model.norm.weight"}),
                     PartSpec("lm_head", sizes, {"weight": "lm_head.weight"}))
    config = {"vocab_size": vocab, "hidden_size": hidden, "num_hidden_layers": 3, "num_attention_heads": heads,
              "num_key_value_heads": kv_heads, "head_dim": hd, "intermediate_size": inter, "rope_theta": 1e4,
              "rms_norm_eps": 1e-5, "tie_word_embeddings": False}
    return spec, config


def custom_tensors(spec):
    from microllm_rocm_amd.parts import Model
    decls = Model(spec, Runtime(torch.float32, torch.device("cpu"))).tensors()
    rules = [InitRule("layernorm.weight", 1.0, "norm_std"), InitRule("norm.weight", 1.0, "norm_std"), InitRule("", 0.0, "std")]
    return random_tensors(decls, rules, seed=4, stds={"std": 0.15, "norm_std": 0.1})


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_layer_named_twice_runs_twice_with_a_cache_for_each_run(dtype):
    spec, config = custom_model([RunEntry(0), RunEntry(1), RunEntry(0), RunEntry(2)])
    tensors = custom_tensors(spec)
    engine = Engine(spec, tensors, dtype=dtype, max_tokens=256)
    assert len(engine.cache.groups[0].entries) == 4          # four caches for three layers
    weights = {name: value.double().numpy() for name, value in tensors.items()}
    tokens = np.random.default_rng(0).integers(0, 97, size=40).tolist()
    expected = plain.forward(config, weights, tokens, order=[0, 1, 0, 2])
    engine.open("a")
    got = [engine.step([StepEntry("a", tokens[:23], list(range(23)))]).cpu()]
    got += [engine.step([StepEntry("a", [token], [0])]).cpu() for token in tokens[23:]]
    tol = 2e-5 if dtype == "float32" else 4e-2
    assert np.abs(torch.cat(got).double().numpy() - expected).max() <= tol * np.abs(expected).max()
    different = plain.forward(config, weights, tokens, order=[0, 1, 2])
    assert np.abs(different - expected).max() > 0.05 * np.abs(expected).max()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_layer_reads_another_layers_cache(dtype):
    """Layer 2 projects queries only and attends over the keys and values that layer 0 wrote."""
    spec, config = custom_model([RunEntry(0), RunEntry(1), RunEntry(2, reads_cache_of=0)], owns_kv=(True, True, False))
    tensors = custom_tensors(spec)
    assert "model.layers.2.self_attn.k_proj.weight" not in tensors
    engine = Engine(spec, tensors, dtype=dtype, max_tokens=256)
    assert len(engine.cache.groups[0].entries) == 2
    weights = {name: value.double().numpy() for name, value in tensors.items()}
    tokens = np.random.default_rng(1).integers(0, 97, size=37).tolist()
    # plain: the same blocks, with layer 2's attention given layer 0's rotated keys and values
    h = plain.embedding(weights["model.embed_tokens.weight"], tokens)
    kept = None
    for index in range(3):
        prefix = f"model.layers.{index}"
        x = plain.rms_norm(h, weights[f"{prefix}.input_layernorm.weight"], 1e-5)
        if index == 0:
            mixed, kept = plain.attention_layer(x, weights, prefix, config, None, return_kv=True)
        elif index == 2:
            mixed = plain.attention_layer(x, weights, prefix, config, None, kv_override=kept)
        else:
            mixed = plain.attention_layer(x, weights, prefix, config, None)
        h = h + mixed
        x = plain.rms_norm(h, weights[f"{prefix}.post_attention_layernorm.weight"], 1e-5)
        h = h + plain.swiglu_ffn(x, weights[f"{prefix}.mlp.gate_proj.weight"], weights[f"{prefix}.mlp.up_proj.weight"],
                                 weights[f"{prefix}.mlp.down_proj.weight"])
    expected = plain.linear(plain.rms_norm(h, weights["model.norm.weight"], 1e-5), weights["lm_head.weight"])
    engine.open("a")
    got = [engine.step([StepEntry("a", tokens[:20], list(range(20)))]).cpu(),
           engine.step([StepEntry("a", tokens[20:22], [0, 1])]).cpu()]
    got += [engine.step([StepEntry("a", [token], [0])]).cpu() for token in tokens[22:]]
    tol = 2e-5 if dtype == "float32" else 4e-2
    assert np.abs(torch.cat(got).double().numpy() - expected).max() <= tol * np.abs(expected).max()


def test_position_embedding_and_head_parts_alone():
    rt = runtime(torch.bfloat16)
    rope = build_part("position", PartSpec("rope_split_half", {"theta": 5e4, "head_dim": 48}), rt)
    expected = 5e4 ** (-np.arange(0, 48, 2) / 48.0)
    assert rope.fused_split_half and rope.inv_freq.dtype == torch.float64
    np.testing.assert_allclose(rope.inv_freq.cpu().numpy(), expected, rtol=1e-15)
    partial = build_part("position", PartSpec("rope_split_half", {"theta": 1e4, "head_dim": 64, "rotary_dim": 32}), rt)
    assert partial.inv_freq.shape[0] == 16
    with pytest.raises(ValueError):
        build_part("position", PartSpec("rope_split_half", {"theta": 1e4, "head_dim": 64, "rotary_dim": 70}), rt)
    rng = np.random.default_rng(5)
    sizes = {"vocab_size": 331, "hidden_size": 72}
    table = bf16_exact(rng.normal(size=(331, 72)))
    embedding = build_part("embedding", PartSpec("token_embedding", sizes, {"weight": "e"}), rt)
    head = build_part("head", PartSpec("lm_head", sizes, {"weight": "e"}), rt)       # tied: the same tensor name
    assert embedding.tensors() == head.tensors()
    tensors = {"e": table.to(DEVICE)}
    embedding.bind(tensors)
    head.bind(tensors)
    ids = torch.tensor([3, 330, 0], dtype=torch.int32, device=DEVICE)
    from types import SimpleNamespace
    rows = embedding.forward(SimpleNamespace(tokens=ids))       # an embedding part is handed the step
    assert rows.dtype == torch.float32 and torch.equal(rows.cpu(), table[[3, 330, 0]].float())
    x = bf16_exact(rng.normal(size=(5, 72)))
    logits = head.forward(x.to(DEVICE))
    assert logits.dtype == torch.float32 and logits.shape == (5, 331)
    np.testing.assert_allclose(logits.cpu().numpy(), x.double().numpy() @ table.double().numpy().T, rtol=1e-4, atol=1e-4)
    with pytest.raises(KeyError, match="unknown mixer kind 'nope'"):
        build_part("mixer", PartSpec("nope"), rt)
