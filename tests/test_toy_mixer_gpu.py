"""A mixer with state of its own, defined here, is registered, built into a model and stepped without a change
to the package: the part registry, the spec, the cache manager's state slots and the step context carry it."""
import numpy as np
import pytest
import torch

from microllm_rocm_amd.config import Architecture, register_architecture, unregister_architecture
from microllm_rocm_amd.engine import Engine, StepEntry
from microllm_rocm_amd.parts import (LayerSpec, MATRIX, Mixer, ModelSpec, PartSpec, RunEntry, StateNeed, TensorDecl,
                                     register_part, unregister_part)

pytestmark = pytest.mark.gpu


class DecayMixer(Mixer):
    """s_t = decay * s_{t-1} + x_t W_in ;  y_t = s_t W_out. The state s (one vector per request) lives in the
    request's state slot, so a request can be cut into steps anywhere."""

    def __init__(self, spec, runtime):
        super().__init__(spec, runtime)
        self.hidden, self.width, self.decay = spec.params["hidden_size"], spec.params["state_size"], spec.params["decay"]

    def tensors(self):
        return {self.name("in"): TensorDecl((self.width, self.hidden), MATRIX),
                self.name("out"): TensorDecl((self.hidden, self.width), MATRIX)}

    def bind(self, tensors):
        self.w_in, self.w_out = tensors[self.name("in")].float(), tensors[self.name("out")].float()

    def cache_need(self):
        return StateNeed((self.width,), torch.float32)

    def forward(self, x, ctx, cache):
        drive = x.float() @ self.w_in.t()
        outputs = torch.empty_like(drive)
        row = 0
        for slot, count in zip(ctx.host_slots, ctx.counts):     # requests of the step, each with its own slot
            state = cache.state[slot]
            for _ in range(count):
                state.mul_(self.decay).add_(drive[row])
                outputs[row] = state
                row += 1
        return (outputs @ self.w_out.t()).to(torch.float32)


@pytest.fixture
def toy_registered():
    register_part("mixer", "decay_state", DecayMixer)
    yield
    unregister_part("mixer", "decay_state")
    unregister_architecture("ToyStateForCausalLM")


def toy_spec(config):
    hidden, vocab, inter = config["hidden_size"], config["vocab_size"], config["intermediate_size"]
    layers = []
    for index in range(config["num_hidden_layers"]):
        prefix = f"layers.{index}"
        if index % 2 == 0:      # different mixers in different layers of one model
            mixer = PartSpec("decay_state", {"hidden_size": hidden, "state_size": config["state_size"], "decay": config["decay"]},
                             {"in": f"{prefix}.mix.in", "out": f"{prefix}.mix.out"})
        else:
            names = {f"{r}_proj.weight": f"{prefix}.attn.{r}" for r in ("q", "k", "v", "o")}
            mixer = PartSpec("paged_attention", {"hidden_size": hidden, "num_heads": 2, "num_kv_heads": 1, "head_dim": 16,
                                                 "qkv_bias": False, "window": None,
                                                 "position": PartSpec("rope_split_half", {"theta": 1e4, "head_dim": 16})}, names)
        layers.append(LayerSpec(
            "pre_norm", PartSpec("rms_norm", {"size": hidden, "eps": 1e-5}, {"weight": f"{prefix}.norm1"}), mixer,
            PartSpec("rms_norm", {"size": hidden, "eps": 1e-5}, {"weight": f"{prefix}.norm2"}),
            PartSpec("swiglu", {"hidden_size": hidden, "intermediate_size": inter},
                     {f"{r}_proj.weight": f"{prefix}.ffn.{r}" for r in ("gate", "up", "down")})))
    sizes = {"vocab_size": vocab, "hidden_size": hidden}
    return ModelSpec("ToyStateForCausalLM", vocab, hidden, 512, PartSpec("token_embedding", sizes, {"weight": "embed"}),
                     tuple(layers), tuple(RunEntry(i) for i in range(len(layers))),
                     PartSpec("rms_norm", {"size": hidden, "eps": 1e-5}, {"weight": "norm"}),
                     PartSpec("lm_head", sizes, {"weight": "embed"}))


def plain_toy(config, w, tokens):
    """Whole sequence, float64, no cache."""
    import plain_qwen2 as plain
    h = w["embed"][tokens]
    attention_config = {"num_attention_heads": 2, "num_key_value_heads": 1, "head_dim": 16, "rope_theta": 1e4}
    for index in range(config["num_hidden_layers"]):
        p = f"layers.{index}"
        x = plain.rms_norm(h, w[f"{p}.norm1"], 1e-5)
        if index % 2 == 0:
            state = np.zeros(config["state_size"])
            mixed = np.zeros_like(h)
            for t in range(len(tokens)):
                state = config["decay"] * state + w[f"{p}.mix.in"] @ x[t]
                mixed[t] = w[f"{p}.mix.out"] @ state
        else:
            weights = {f"L.self_attn.{r}_proj.weight": w[f"{p}.attn.{r}"] for r in ("q", "k", "v", "o")}
            mixed = plain.attention_layer(x, weights, "L", attention_config, None)
        h = h + mixed
        x = plain.rms_norm(h, w[f"{p}.norm2"], 1e-5)
        h = h + plain.swiglu_ffn(x, w[f"{p}.ffn.gate"], w[f"{p}.ffn.up"], w[f"{p}.ffn.down"])
    return plain.rms_norm(h, w["norm"], 1e-5) @ w["embed"].T


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_mixer_with_state_is_registered_built_and_stepped(toy_registered, tmp_path, dtype):
    import json
    from microllm_rocm_amd.parts import Model, Runtime
    from microllm_rocm_amd.weights import save_file
    config = {"architectures": ["ToyStateForCausalLM"], "vocab_size": 61, "hidden_size": 32, "intermediate_size": 56,
              "num_hidden_layers": 3, "state_size": 24, "decay": 0.9}
    register_architecture(Architecture("ToyStateForCausalLM", dict, toy_spec))
    spec = toy_spec(config)
    rng = np.random.default_rng(0)
    decls = Model(spec, Runtime(torch.float32, torch.device("cpu"))).tensors()
    tensors = {name: (torch.from_numpy(1 + 0.1 * rng.normal(size=decl.shape)) if "norm" in name
                      else torch.from_numpy(rng.normal(size=decl.shape) * 0.2)).to(torch.bfloat16)
               for name, decl in decls.items()}
    (tmp_path / "config.json").write_text(json.dumps(config))
    save_file(tensors, str(tmp_path / "model.safetensors"))
    # through the same door as every model: the folder's config.json names the architecture
    engine = Engine.from_folder(str(tmp_path), dtype=dtype, max_tokens=256, max_requests=2)
    assert [type(b.mixer).__name__ for b in engine.model.blocks] == ["DecayMixer", "PagedAttention", "DecayMixer"]
    weights = {name: value.double().numpy() for name, value in tensors.items()}
    sequences = {name: rng.integers(0, 61, size=length).tolist() for name, length in (("a", 45), ("b", 30), ("c", 38))}
    expected = {name: plain_toy(config, weights, tokens) for name, tokens in sequences.items()}
    got = {name: [] for name in sequences}

    def feed(entries):
        logits = engine.step([StepEntry(name, sequences[name][start:start + count], list(range(count)))
                              for name, start, count in entries]).cpu()
        row = 0
        for name, _, count in entries:
            got[name].append(logits[row:row + count])
            row += count

    engine.open("a")
    engine.open("b")
    feed([("a", 0, 17), ("b", 0, 2)])
    feed([("a", 17, 1), ("b", 2, 20)])
    feed([("b", 22, 8)])
    engine.close("b")                     # its slot goes back ...
    engine.open("c")                      # ... to a request that must find it zeroed
    assert engine.cache.get("c").slot != engine.cache.get("a").slot
    feed([("a", 18, 27), ("c", 0, 5)])
    for start in range(5, 38):
        feed([("c", start, 1)])
    tol = 3e-5 if dtype == "float32" else 4e-2
    for name, tokens in sequences.items():
        rows = torch.cat(got[name]).double().numpy()
        assert rows.shape == expected[name].shape
        assert np.abs(rows - expected[name]).max() <= tol * np.abs(expected[name]).max(), name
    engine.close("a")
    engine.close("c")
    engine.cache.check()
