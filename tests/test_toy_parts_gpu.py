"""Two more toy parts, defined here and registered from here, in one model beside the package's own parts: a position
encoding that rotates neighbouring dims (applied by the part itself, not by the fused kernels) and a feed-forward
that routes every token to one of a few small experts. Nothing in the package changes for them; the cache manager,
the step function, replay in portions and the scheduler carry them as they carry the package's parts."""
import math

import numpy as np
import pytest
import torch

import plain_qwen2 as plain
from microllm_rocm_amd.engine import Engine, StepEntry
from microllm_rocm_amd.parts import (FeedForward, LayerSpec, MATRIX, ModelSpec, PartSpec, PositionEncoding, RunEntry,
                                     TensorDecl, register_part, unregister_part)

pytestmark = pytest.mark.gpu

HIDDEN, HEADS, KV_HEADS, HEAD_DIM, INTER, VOCAB, EXPERTS, THETA, EPS = 48, 3, 1, 16, 40, 101, 3, 500.0, 1e-5


class NeighbourRope(PositionEncoding):
    """Rotates dims (2i, 2i + 1) of every query and key head by position * theta^(-2i/d)."""

    def __init__(self, spec, runtime):
        super().__init__(spec, runtime)
        self.theta, self.head_dim = float(spec.params["theta"]), int(spec.params["head_dim"])

    def apply(self, qkv, positions, heads, kv_heads, head_dim):
        tokens = qkv.shape[0]
        x = qkv.view(tokens, heads + 2 * kv_heads, head_dim).clone()
        exponents = torch.arange(0, head_dim, 2, dtype=torch.float64, device=qkv.device) / head_dim
        angle = positions.to(torch.float64)[:, None] * self.theta ** -exponents[None, :]
        cos, sin = angle.cos().float()[:, None, :], angle.sin().float()[:, None, :]
        rotated = x[:, :heads + kv_heads]
        even, odd = rotated[..., 0::2].clone(), rotated[..., 1::2].clone()
        rotated[..., 0::2] = even * cos - odd * sin
        rotated[..., 1::2] = even * sin + odd * cos
        return x.view(tokens, -1)


class RoutedFeedForward(FeedForward):
    """Every token goes to the expert whose router row scores it highest; an expert is ``down(relu(up(x)))``."""

    def __init__(self, spec, runtime):
        super().__init__(spec, runtime)
        self.hidden, self.inter, self.experts = (int(spec.params[key]) for key in ("hidden_size", "intermediate_size", "experts"))
        self.routes = []

    def tensors(self):
        decls = {self.name("router"): TensorDecl((self.experts, self.hidden), MATRIX)}
        for expert in range(self.experts):
            decls[self.name(f"up.{expert}")] = TensorDecl((self.inter, self.hidden), MATRIX)
            decls[self.name(f"down.{expert}")] = TensorDecl((self.hidden, self.inter), MATRIX)
        return decls

    def bind(self, tensors):
        self.router = tensors[self.name("router")].float()
        self.up = [tensors[self.name(f"up.{expert}")].float() for expert in range(self.experts)]
        self.down = [tensors[self.name(f"down.{expert}")].float() for expert in range(self.experts)]

    def forward(self, x, ctx):
        x = x.float()
        chosen = (x @ self.router.t()).argmax(dim=1)            # router logits in float32
        self.routes.append(chosen.cpu().tolist())               # for the test: which expert every row of the step took
        out = torch.zeros_like(x)
        for expert in range(self.experts):
            rows = (chosen == expert).nonzero().flatten()
            if rows.numel():
                out[rows] = torch.relu(x[rows] @ self.up[expert].t()) @ self.down[expert].t()
        return out


@pytest.fixture
def toys_registered():
    register_part("position", "neighbour_rope", NeighbourRope)
    register_part("ffn", "routed_relu", RoutedFeedForward)
    yield
    unregister_part("position", "neighbour_rope")
    unregister_part("ffn", "routed_relu")


def toy_spec():
    layers = []
    for index in range(3):
        prefix = f"layers.{index}"
        names = {f"{role}_proj.{kind}": f"{prefix}.attn.{role}.{kind}" for role in ("q", "k", "v") for kind in ("weight", "bias")}
        names["o_proj.weight"] = f"{prefix}.attn.o.weight"
        # layers 0 and 2: the toy position encoding; layer 1: the package's own (one model, two encodings)
        position = PartSpec("neighbour_rope" if index != 1 else "rope_split_half", {"theta": THETA, "head_dim": HEAD_DIM})
        mixer = PartSpec("paged_attention", {"hidden_size": HIDDEN, "num_heads": HEADS, "num_kv_heads": KV_HEADS, "head_dim": HEAD_DIM,
                                             "qkv_bias": True, "window": None, "position": position}, names)
        if index == 1:      # layer 1: the routed feed-forward; the others: the package's SwiGLU
            ffn = PartSpec("routed_relu", {"hidden_size": HIDDEN, "intermediate_size": INTER, "experts": EXPERTS},
                           {"router": f"{prefix}.ffn.router", **{f"{w}.{e}": f"{prefix}.ffn.{w}.{e}" for w in ("up", "down") for e in range(EXPERTS)}})
        else:
            ffn = PartSpec("swiglu", {"hidden_size": HIDDEN, "intermediate_size": INTER},
                           {f"{r}_proj.weight": f"{prefix}.ffn.{r}" for r in ("gate", "up", "down")})
        layers.append(LayerSpec("pre_norm", PartSpec("rms_norm", {"size": HIDDEN, "eps": EPS}, {"weight": f"{prefix}.norm1"}),
                                mixer, PartSpec("rms_norm", {"size": HIDDEN, "eps": EPS}, {"weight": f"{prefix}.norm2"}), ffn))
    sizes = {"vocab_size": VOCAB, "hidden_size": HIDDEN}
    return ModelSpec("ToyParts", VOCAB, HIDDEN, 512, PartSpec("token_embedding", sizes, {"weight": "embed"}), tuple(layers),
                     tuple(RunEntry(index) for index in range(3)), PartSpec("rms_norm", {"size": HIDDEN, "eps": EPS}, {"weight": "norm"}),
                     PartSpec("lm_head", sizes, {"weight": "head"}))


def toy_tensors(spec):
    from microllm_rocm_amd.parts import Model, Runtime
    rng = np.random.default_rng(8)
    out = {}
    for name, decl in Model(spec, Runtime(torch.float32, torch.device("cpu"))).tensors().items():
        value = 1.0 + 0.1 * rng.normal(size=decl.shape) if "norm" in name else 0.25 * rng.normal(size=decl.shape)
        out[name] = torch.from_numpy(value).to(torch.bfloat16)      # exactly representable in both engines
    return out


def neighbour_rope(x, positions):
    """[tokens, heads, head_dim] in float64."""
    pair = np.arange(0, HEAD_DIM, 2)
    angle = positions[:, None] * THETA ** (-pair / HEAD_DIM)[None, :]
    cos, sin = np.cos(angle)[:, None, :], np.sin(angle)[:, None, :]
    out = x.copy()
    out[..., 0::2] = x[..., 0::2] * cos - x[..., 1::2] * sin
    out[..., 1::2] = x[..., 0::2] * sin + x[..., 1::2] * cos
    return out


def toy_reference(weights, tokens, routes=None):
    """The toy model whole, in float64, from the plain implementation's functions and the two toy rules. Returns the
    logits, the expert every token took and by how much its router score led. With ``routes`` the tokens take those
    experts instead of their own choice (rounding may flip a choice that leads by little, and every later position
    sees that through attention)."""
    w = {name: value.double().numpy() for name, value in weights.items()}
    h = plain.embedding(w["embed"], tokens)
    count, positions = len(tokens), np.arange(len(tokens))
    for index in range(3):
        p = f"layers.{index}"
        x = plain.rms_norm(h, w[f"{p}.norm1"], EPS)
        q = plain.linear(x, w[f"{p}.attn.q.weight"], w[f"{p}.attn.q.bias"]).reshape(count, HEADS, HEAD_DIM)
        k = plain.linear(x, w[f"{p}.attn.k.weight"], w[f"{p}.attn.k.bias"]).reshape(count, KV_HEADS, HEAD_DIM)
        v = plain.linear(x, w[f"{p}.attn.v.weight"], w[f"{p}.attn.v.bias"]).reshape(count, KV_HEADS, HEAD_DIM)
        if index != 1:
            q, k = neighbour_rope(q, positions), neighbour_rope(k, positions)
        else:
            q, k = plain.rope_split_half(q, positions, THETA), plain.rope_split_half(k, positions, THETA)
        o = plain.causal_gqa_attention(q, k, v, 1.0 / math.sqrt(HEAD_DIM), None).reshape(count, HEADS * HEAD_DIM)
        h = h + plain.linear(o, w[f"{p}.attn.o.weight"])
        x = plain.rms_norm(h, w[f"{p}.norm2"], EPS)
        if index == 1:
            scores = x @ w[f"{p}.ffn.router"].T
            chosen = np.argmax(scores, axis=1)
            ordered = np.sort(scores, axis=1)
            lead = (ordered[:, -1] - ordered[:, -2]) / np.abs(scores).max()
            own = chosen
            if routes is not None:
                chosen = np.asarray(routes)
            delta = np.stack([np.maximum(x[t] @ w[f"{p}.ffn.up.{e}"].T, 0.0) @ w[f"{p}.ffn.down.{e}"].T for t, e in enumerate(chosen)])
        else:
            delta = plain.swiglu_ffn(x, w[f"{p}.ffn.gate"], w[f"{p}.ffn.up"], w[f"{p}.ffn.down"])
        h = h + delta
    return plain.rms_norm(h, w["norm"], EPS) @ w["head"].T, own, lead


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_position_and_routed_feed_forward_in_one_model(toys_registered, dtype):
    spec = toy_spec()
    tensors = toy_tensors(spec)
    engine = Engine(spec, tensors, dtype=dtype, max_tokens=512)
    assert not engine.use_graphs, "parts that do not say they are graph-safe switch graphs off"
    tokens = np.random.default_rng(2).integers(0, VOCAB, size=90).tolist()
    tolerance = 2e-5 if dtype == "float32" else 4e-2
    routed = engine.model.blocks[1].ffn

    def check(logits, routes):
        """Against the reference that routes as the engine did; the engine's routes are the reference's own wherever
        a score leads clearly (in float32: everywhere)."""
        expected, own, lead = toy_reference(tensors, tokens, routes)
        clear = lead > (1e-4 if dtype == "float32" else 3e-2)
        assert np.array_equal(np.asarray(routes)[clear], own[clear]) and clear.sum() > len(tokens) // 2
        if dtype == "float32":
            assert list(routes) == list(own)
        assert np.abs(logits - expected).max() <= tolerance * np.abs(expected).max()

    # whole
    engine.open("whole")
    whole = engine.step([StepEntry("whole", tokens, list(range(len(tokens))))]).double().cpu().numpy()
    engine.close("whole")
    check(whole, routed.routes.pop())
    assert not routed.routes
    # in portions down to two tokens, then token by token, beside another request (few rows: the fused kernels of the
    # package's own parts run beside the toy parts)
    engine.open("cut"), engine.open("other")
    rows, routes, position = [], [], 0
    for size in (17, 2, 30, 5, 2, 3):
        entries = [StepEntry("cut", tokens[position:position + size], list(range(size)))]
        if position > 0:
            entries.append(StepEntry("other", [tokens[position % 7]], []))
        rows.append(engine.step(entries).double().cpu().numpy())
        routes += routed.routes.pop()[:size]                      # the portion's rows come first in the step
        position += size
    for token in tokens[position:]:
        rows.append(engine.step([StepEntry("other", [token], []), StepEntry("cut", [token], [0])]).double().cpu().numpy())
        routes.append(routed.routes.pop()[1])                     # the second row of the step
    check(np.concatenate(rows), routes)
    engine.cache.check()
    # the routed feed-forward really routes: every expert is chosen by some token
    w = {name: value.double().numpy() for name, value in tensors.items()}
    assert len(set(np.argmax(np.random.default_rng(0).normal(size=(200, HIDDEN)) @ w["layers.1.ffn.router"].T, axis=1))) == EXPERTS


# ---- a toy arrangement ---------------------------------------------------------------------------------------------
def parallel_block_class():
    """A toy arrangement from the package's ``Block``: mixer and feed-forward both read the first norm's output and
    their results are added to the stream together (the second norm is declared, since a layer's spec names two, and
    not used). It takes no part in the fusing of sums and norms across blocks."""
    from microllm_rocm_amd.parts import Block

    class Parallel(Block):
        def first_norm_after(self, producer, rows, h):
            return None       # the block before hands its delta on as it is

        def forward(self, h, pending, ctx, cache, next_block=None):
            x = self.mixer_norm.forward(h, delta=pending, write_h=True)
            deltas = (self.mixer.forward(x, ctx, cache), self.ffn.forward(x, ctx))
            # a delta is [rows, width] or partial sums [parts, rows, width]: all of them go on as partial sums
            return torch.cat([delta.float().reshape(-1, *h.shape) for delta in deltas])

    return Parallel


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_arrangement_beside_the_packages_own(dtype):
    from microllm_rocm_amd.parts import register_arrangement
    register_arrangement("toy_parallel", parallel_block_class(), replace=True)
    layers = []
    for index, arrangement in enumerate(("toy_parallel", "pre_norm", "toy_parallel")):
        prefix = f"layers.{index}"
        names = {f"{role}_proj.{kind}": f"{prefix}.attn.{role}.{kind}" for role in ("q", "k", "v") for kind in ("weight", "bias")}
        names["o_proj.weight"] = f"{prefix}.attn.o.weight"
        position = PartSpec("rope_split_half", {"theta": THETA, "head_dim": HEAD_DIM})
        mixer = PartSpec("paged_attention", {"hidden_size": HIDDEN, "num_heads": HEADS, "num_kv_heads": KV_HEADS, "head_dim": HEAD_DIM,
                                             "qkv_bias": True, "window": None, "position": position}, names)
        ffn = PartSpec("swiglu", {"hidden_size": HIDDEN, "intermediate_size": INTER},
                       {f"{r}_proj.weight": f"{prefix}.ffn.{r}" for r in ("gate", "up", "down")})
        layers.append(LayerSpec(arrangement, PartSpec("rms_norm", {"size": HIDDEN, "eps": EPS}, {"weight": f"{prefix}.norm1"}),
                                mixer, PartSpec("rms_norm", {"size": HIDDEN, "eps": EPS}, {"weight": f"{prefix}.norm2"}), ffn))
    sizes = {"vocab_size": VOCAB, "hidden_size": HIDDEN}
    spec = ModelSpec("ToyArrangement", VOCAB, HIDDEN, 512, PartSpec("token_embedding", sizes, {"weight": "embed"}), tuple(layers),
                     tuple(RunEntry(index) for index in range(3)), PartSpec("rms_norm", {"size": HIDDEN, "eps": EPS}, {"weight": "norm"}),
                     PartSpec("lm_head", sizes, {"weight": "head"}))
    tensors = toy_tensors(spec)
    engine = Engine(spec, tensors, dtype=dtype, max_tokens=512)
    tokens = np.random.default_rng(4).integers(0, VOCAB, size=70).tolist()

    w = {name: value.double().numpy() for name, value in tensors.items()}
    h = plain.embedding(w["embed"], tokens)
    count, positions = len(tokens), np.arange(len(tokens))
    for index, arrangement in enumerate(("toy_parallel", "pre_norm", "toy_parallel")):
        p = f"layers.{index}"

        def attention(x):
            q = plain.linear(x, w[f"{p}.attn.q.weight"], w[f"{p}.attn.q.bias"]).reshape(count, HEADS, HEAD_DIM)
            k = plain.linear(x, w[f"{p}.attn.k.weight"], w[f"{p}.attn.k.bias"]).reshape(count, KV_HEADS, HEAD_DIM)
            v = plain.linear(x, w[f"{p}.attn.v.weight"], w[f"{p}.attn.v.bias"]).reshape(count, KV_HEADS, HEAD_DIM)
            q, k = plain.rope_split_half(q, positions, THETA), plain.rope_split_half(k, positions, THETA)
            o = plain.causal_gqa_attention(q, k, v, 1.0 / math.sqrt(HEAD_DIM), None).reshape(count, HEADS * HEAD_DIM)
            return plain.linear(o, w[f"{p}.attn.o.weight"])

        def feed_forward(x):
            return plain.swiglu_ffn(x, w[f"{p}.ffn.gate"], w[f"{p}.ffn.up"], w[f"{p}.ffn.down"])

        x = plain.rms_norm(h, w[f"{p}.norm1"], EPS)
        if arrangement == "toy_parallel":
            h = h + attention(x) + feed_forward(x)
        else:
            h = h + attention(x)
            h = h + feed_forward(plain.rms_norm(h, w[f"{p}.norm2"], EPS))
    expected = plain.rms_norm(h, w["norm"], EPS) @ w["head"].T
    tolerance = 2e-5 if dtype == "float32" else 4e-2

    engine.open("whole")
    whole = engine.step([StepEntry("whole", tokens, list(range(count)))]).double().cpu().numpy()
    engine.close("whole")
    assert np.abs(whole - expected).max() <= tolerance * np.abs(expected).max()
    # in portions and then token by token (few rows: the package's blocks fuse sums and norms around the toy block)
    engine.open("cut")
    rows, position = [], 0
    for size in (33, 2, 20):
        rows.append(engine.step([StepEntry("cut", tokens[position:position + size], list(range(size)))]).double().cpu().numpy())
        position += size
    for token in tokens[position:]:
        rows.append(engine.step([StepEntry("cut", [token], [0])]).double().cpu().numpy())
    assert np.abs(np.concatenate(rows) - expected).max() <= tolerance * np.abs(expected).max()
    engine.cache.check()


# ---- a layer with a third norm, and one without a feed-forward -------------------------------------------------------
def sandwich_block_class():
    """A toy arrangement with a norm that the layer's spec carries under ``extra``: the mixer's result is normalised
    by itself before it is added to the stream."""
    from microllm_rocm_amd.parts import Block

    class Sandwich(Block):
        def first_norm_after(self, producer, rows, h):
            return None

        def forward(self, h, pending, ctx, cache, next_block=None):
            x = self.mixer_norm.forward(h, delta=pending, write_h=True)
            mixed = self.mixer.forward(x, ctx, cache)
            mixed = (mixed.sum(dim=0) if mixed.dim() == 3 else mixed).float().contiguous()
            mixed = self.extra["after_mixer"].forward(mixed, write_h=False)          # a norm of the delta alone
            x = self.ffn_norm.forward(h, delta=mixed, write_h=True)
            return self.ffn.forward(x, ctx)

    return Sandwich


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_layer_with_a_third_norm_and_a_layer_without_a_feed_forward(dtype):
    from microllm_rocm_amd.parts import register_arrangement
    register_arrangement("toy_sandwich", sandwich_block_class(), replace=True)
    arrangements = ("toy_sandwich", "pre_norm", "pre_norm", "pre_norm")
    has_ffn = (True, False, True, False)          # the last layer has none either: its mixer's delta goes to the final norm
    layers = []
    for index, arrangement in enumerate(arrangements):
        prefix = f"layers.{index}"
        names = {f"{role}_proj.{kind}": f"{prefix}.attn.{role}.{kind}" for role in ("q", "k", "v") for kind in ("weight", "bias")}
        names["o_proj.weight"] = f"{prefix}.attn.o.weight"
        position = PartSpec("rope_split_half", {"theta": THETA, "head_dim": HEAD_DIM})
        mixer = PartSpec("paged_attention", {"hidden_size": HIDDEN, "num_heads": HEADS, "num_kv_heads": KV_HEADS, "head_dim": HEAD_DIM,
                                             "qkv_bias": True, "window": None, "position": position}, names)
        norm = lambda name: PartSpec("rms_norm", {"size": HIDDEN, "eps": EPS}, {"weight": f"{prefix}.{name}"})
        ffn = PartSpec("swiglu", {"hidden_size": HIDDEN, "intermediate_size": INTER},
                       {f"{r}_proj.weight": f"{prefix}.ffn.{r}" for r in ("gate", "up", "down")})
        extra = {"after_mixer": ("norm", norm("norm_after_mixer"))} if arrangement == "toy_sandwich" else {}
        if has_ffn[index]:
            layers.append(LayerSpec(arrangement, norm("norm1"), mixer, norm("norm2"), ffn, extra=extra))
        else:
            layers.append(LayerSpec(arrangement, norm("norm1"), mixer))
    sizes = {"vocab_size": VOCAB, "hidden_size": HIDDEN}
    spec = ModelSpec("ToyLayers", VOCAB, HIDDEN, 512, PartSpec("token_embedding", sizes, {"weight": "embed"}), tuple(layers),
                     tuple(RunEntry(index) for index in range(len(layers))),
                     PartSpec("rms_norm", {"size": HIDDEN, "eps": EPS}, {"weight": "norm"}), PartSpec("lm_head", sizes, {"weight": "head"}))
    tensors = toy_tensors(spec)
    # the third norm brings the mixer's result to unit size whatever it was, its rounding with it: with a weight of
    # about a quarter the stream keeps the proportions the other toy models have (and the bound that is theirs)
    tensors["layers.0.norm_after_mixer"] = (tensors["layers.0.norm_after_mixer"].float() * 0.25).to(torch.bfloat16)
    assert "layers.0.norm_after_mixer" in tensors and "layers.1.norm2" not in tensors and "layers.1.ffn.gate" not in tensors
    engine = Engine(spec, tensors, dtype=dtype, max_tokens=512)
    tokens = np.random.default_rng(6).integers(0, VOCAB, size=60).tolist()

    w = {name: value.double().numpy() for name, value in tensors.items()}
    h = plain.embedding(w["embed"], tokens)
    count, positions = len(tokens), np.arange(len(tokens))
    for index, arrangement in enumerate(arrangements):
        p = f"layers.{index}"
        x = plain.rms_norm(h, w[f"{p}.norm1"], EPS)
        q = plain.linear(x, w[f"{p}.attn.q.weight"], w[f"{p}.attn.q.bias"]).reshape(count, HEADS, HEAD_DIM)
        k = plain.linear(x, w[f"{p}.attn.k.weight"], w[f"{p}.attn.k.bias"]).reshape(count, KV_HEADS, HEAD_DIM)
        v = plain.linear(x, w[f"{p}.attn.v.weight"], w[f"{p}.attn.v.bias"]).reshape(count, KV_HEADS, HEAD_DIM)
        q, k = plain.rope_split_half(q, positions, THETA), plain.rope_split_half(k, positions, THETA)
        o = plain.causal_gqa_attention(q, k, v, 1.0 / math.sqrt(HEAD_DIM), None).reshape(count, HEADS * HEAD_DIM)
        mixed = plain.linear(o, w[f"{p}.attn.o.weight"])
        if arrangement == "toy_sandwich":
            mixed = plain.rms_norm(mixed, w[f"{p}.norm_after_mixer"], EPS)
        h = h + mixed
        if has_ffn[index]:
            h = h + plain.swiglu_ffn(plain.rms_norm(h, w[f"{p}.norm2"], EPS), w[f"{p}.ffn.gate"], w[f"{p}.ffn.up"], w[f"{p}.ffn.down"])
    expected = plain.rms_norm(h, w["norm"], EPS) @ w["head"].T
    tolerance = 2e-5 if dtype == "float32" else 4e-2

    engine.open("whole")
    whole = engine.step([StepEntry("whole", tokens, list(range(count)))]).double().cpu().numpy()
    engine.close("whole")
    assert np.abs(whole - expected).max() <= tolerance * np.abs(expected).max()
    # in portions, then token by token from a graph (every part here says it is graph-safe): with few rows the
    # layer without a feed-forward hands its mixer's sum and the next layer's norm to the products around them
    assert engine.use_graphs
    engine.open("cut")
    rows, position = [], 0
    for size in (21, 2, 19):
        rows.append(engine.step([StepEntry("cut", tokens[position:position + size], list(range(size)))]).double().cpu().numpy())
        position += size
    for token in tokens[position:]:
        rows.append(engine.step([StepEntry("cut", [token], [0])]).double().cpu().numpy())
    assert np.abs(np.concatenate(rows) - expected).max() <= tolerance * np.abs(expected).max()
    engine.cache.check()
