"""Generation through the entry point, the scheduler on the real engine, and the command line."""
import json
import os
import subprocess
import sys

import numpy as np
import torch
import pytest

import plain_qwen2 as plain
from replay_tools import PlainModel
from tiny import CONFIGS, make_folder, random_tokens

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SHARP = {"std": 0.12, "norm_std": 0.1}


def engine_for(folder, dtype="float32", **options):
    from microllm_rocm_amd import Engine
    options.setdefault("max_tokens", 1024)
    return Engine.from_folder(folder, dtype=dtype, **options)


@pytest.mark.parametrize("which,lengths,new_tokens", [("A", (7, 13), 8), ("B", (5, 17, 40, 64), 16)])
def test_greedy_generation_matches_the_plain_implementation(tmp_path, which, lengths, new_tokens):
    from microllm_rocm_amd import GenerationConfig, generate, generate_serial
    folder = make_folder(tmp_path, which, SHARP)
    model = PlainModel(folder)
    config = CONFIGS[which]
    prompts = [random_tokens(1 + index, length, config.vocab_size) for index, length in enumerate(lengths)]
    expected = [prompt + plain.generate_greedy(model.config, model.weights, prompt, new_tokens) for prompt in prompts]
    engine = engine_for(folder)
    params = GenerationConfig(max_new_tokens=new_tokens, temperature=0.0)
    assert generate(engine, prompts, params, prefill_chunk=16, max_batched_tokens=24,
                    arrival_steps=[0, 1, 3, 4][:len(prompts)]) == expected
    assert [generate_serial(engine, prompt, params) for prompt in prompts] == expected
    assert generate(engine, prompts[0], params) == expected[0]          # one prompt in, one sequence out
    engine.cache.check()
    assert not engine.cache.requests
    bf16 = generate(engine_for(folder, "bfloat16"), prompts, params, prefill_chunk=16)
    same = sum(a == b for got, want in zip(bf16, expected) for a, b in zip(got, want))
    assert same >= 0.9 * sum(len(want) for want in expected)            # rounding may flip a near tie


def test_sampling_in_batches_equals_requests_run_alone_and_follows_the_plain_rule(tmp_path):
    from microllm_rocm_amd import GenerationConfig, generate, generate_serial
    folder = make_folder(tmp_path, "B", SHARP)
    model = PlainModel(folder)
    config = CONFIGS["B"]
    prompts = [random_tokens(30 + index, length, config.vocab_size) for index, length in enumerate((5, 17, 40, 64))]
    params = [GenerationConfig(max_new_tokens=16, temperature=0.8, seed=index, top_k=(0, 20)[index % 2]) for index in range(4)]
    engine = engine_for(folder)
    batched = generate(engine, prompts, params, prefill_chunk=16, max_batched_tokens=32, arrival_steps=[0, 2, 2, 5])
    alone = [generate_serial(engine, prompt, p) for prompt, p in zip(prompts, params)]
    assert batched == alone
    # every drawn token is the one the plain rule draws from the plain logits of the same prefix
    for sequence, prompt, p in zip(batched, prompts, params):
        for draw in range(16):
            prefix = sequence[:len(prompt) + draw]
            expected = plain.sample(model.logits(prefix)[-1], p.temperature, p.top_k, plain.uniform_for(p.seed, draw))
            if expected != sequence[len(prompt) + draw]:
                # float32 against float64 logits: only a draw that falls on an interval's edge may differ
                weights = plain.sampling_weights(model.logits(prefix)[-1], p.temperature, p.top_k)
                cumulative = np.cumsum(weights) / weights.sum()
                target = plain.uniform_for(p.seed, draw)
                assert min(abs(cumulative - target)) < 1e-4
                break


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_every_replay_of_a_decode_graph_equals_the_eager_step(tmp_path, dtype):
    """Decode steps replayed from HIP graphs, with eager steps (a portion of a prompt beside decoded tokens, requests
    that come and go, a wider block table) and synchronisations between the replays: every replay gives the bits
    of the same step run without graphs."""
    from microllm_rocm_amd.engine import StepEntry
    folder = make_folder(tmp_path, "B", SHARP)
    config = CONFIGS["B"]
    graphs = engine_for(folder, dtype, use_graphs=True)
    eager = engine_for(folder, dtype, use_graphs=False)
    rng = np.random.default_rng(7)
    prompts = {name: random_tokens(60 + index, length, config.vocab_size) for index, (name, length) in
               enumerate({"a": 20, "b": 33, "c": 50}.items())}

    def both(entries):
        out = [engine.step([StepEntry(*entry) for entry in entries]) for engine in (graphs, eager)]
        torch.cuda.synchronize()
        assert (out[0] is None) == (out[1] is None)
        if out[0] is not None:
            assert torch.equal(out[0], out[1]), "a replayed step differs from the eager step"
        return out[0]

    for engine in (graphs, eager):
        engine.open("a"), engine.open("b")
    both([("a", prompts["a"], [19]), ("b", prompts["b"], [32])])
    replays = 0
    for step in range(40):
        tokens = rng.integers(0, config.vocab_size, size=3).tolist()
        if step == 10:      # an eager step between replays: a new request's prompt beside two decoded tokens
            for engine in (graphs, eager):
                engine.open("c")
            both([("a", [tokens[0]], [0]), ("c", prompts["c"][:30], []), ("b", [tokens[1]], [0])])
            both([("c", prompts["c"][30:], [19])])
            continue
        if step == 25:      # a request leaves: the graph for two requests again
            for engine in (graphs, eager):
                engine.close("b")
        if step == 31:      # a request ends and another comes under its name, as long as the old one was
            for engine in (graphs, eager):
                length = engine.cache.get("a").num_tokens
                engine.close("a"), engine.open("a")
            both([("a", random_tokens(99, length, config.vocab_size), [])])
        live = [name for name in ("a", "b", "c") if graphs.is_open(name)]
        wanted = [[0], [], [0]] if step % 7 == 3 else [[0]] * 3        # logits of some requests only
        both([(name, [token], want) for name, token, want in zip(live, tokens, wanted)])
        replays += 1
    assert graphs.graph_replays == replays and eager.graph_replays == 0
    # most replays found their metadata built while the step before ran (not the first of a graph, not those at a
    # page's edge or after another kind of step), and none took what was built for other requests
    assert replays // 2 < graphs.steps_built_ahead < replays
    assert graphs.kept_graphs >= 2, "more than one graph was captured (two and three requests)"
    for engine in (graphs, eager):
        engine.cache.check()


def test_few_pages_preempt_and_recompute_to_the_same_tokens(tmp_path):
    from microllm_rocm_amd import GenerationConfig, generate
    folder = make_folder(tmp_path, "A", SHARP)
    config = CONFIGS["A"]
    prompts = [random_tokens(50 + index, 30, config.vocab_size) for index in range(3)]
    params = GenerationConfig(max_new_tokens=40, temperature=0.0)
    roomy = generate(engine_for(folder, max_tokens=1024), prompts, params)
    tight_engine = engine_for(folder, num_pages=9, max_tokens=None)           # 9 pages of 16: three requests of 70 do not fit
    tight, scheduler = generate(tight_engine, prompts, params, return_scheduler=True)
    assert scheduler.metrics.preemptions >= 1
    assert tight == roomy
    assert tight_engine.cache.free_pages() == [9]


def test_stop_tokens_and_limits(tmp_path):
    from microllm_rocm_amd import GenerationConfig, Scheduler, generate
    folder = make_folder(tmp_path, "A", SHARP)
    engine = engine_for(folder)
    prompt = random_tokens(9, 11, CONFIGS["A"].vocab_size)
    free_run = generate(engine, prompt, GenerationConfig(max_new_tokens=12, temperature=0.0))[len(prompt):]
    stopped = generate(engine, prompt, GenerationConfig(max_new_tokens=12, temperature=0.0, stop_tokens=(free_run[3],)))
    assert stopped[len(prompt):] == free_run[:free_run.index(free_run[3]) + 1]
    with pytest.raises(ValueError, match="max positions"):
        Scheduler(engine).submit(prompt, GenerationConfig(max_new_tokens=200))
    with pytest.raises(ValueError, match="outside the vocabulary"):
        generate(engine, [[999]], GenerationConfig(max_new_tokens=1))


def test_command_line(tmp_path):
    folder = make_folder(tmp_path, "B", SHARP)
    model = PlainModel(folder)
    prompt = random_tokens(3, 9, CONFIGS["B"].vocab_size)
    expected = plain.generate_greedy(model.config, model.weights, prompt, 6)
    logits_path = tmp_path / "last.f32"
    command = [sys.executable, os.path.join(ROOT, "bin", "microllm_hf_infer"), "--config", os.path.join(folder, "config.json"),
               "--weights", os.path.join(folder, "model.safetensors"), "--tokens", ",".join(map(str, prompt)),
               "--device", "hip", "--dtype", "float32", "--new-tokens", "6", "--logits-output", str(logits_path)]
    result = subprocess.run(command, capture_output=True, text=True, timeout=300)
    assert result.returncode == 0, result.stderr
    report = json.loads(result.stdout.strip().splitlines()[-1])
    assert report["generated_tokens"] == expected and report["prompt_tokens"] == len(prompt)
    last = np.fromfile(logits_path, dtype="<f4")
    reference = model.logits(prompt)[-1]
    assert np.abs(last - reference).max() <= 2e-5 * np.abs(reference).max()
    bad = subprocess.run(command + ["--bogus", "1"], capture_output=True, text=True, timeout=120)
    assert bad.returncode != 0 and "bogus" in bad.stderr
    continuous = subprocess.run(command[:6] + ["--tokens", ",".join(map(str, prompt)), "--device", "hip", "--dtype", "float32",
                                               "--workload", "continuous", "--continuous-prompt-lengths", "5,9,7",
                                               "--continuous-new-token-lengths", "4,6,3", "--continuous-arrival-steps", "0,1,1",
                                               "--continuous-slots", "2", "--warmup", "1", "--steps", "2"],
                                capture_output=True, text=True, timeout=300)
    assert continuous.returncode == 0, continuous.stderr
    report = json.loads(continuous.stdout.strip().splitlines()[-1])
    assert report["completed_requests"] == 3 and [len(r) for r in report["generated"]] == [4, 6, 3]
    # latencies as the reference reports them (apps/hf_infer.cpp:988-995): medians and 95th percentiles of the lists
    for key in ("request_ttft", "request_completion"):
        values = sorted(report[f"{key}_ms"])
        assert len(values) == 3 and abs(report[f"{key}_p50_ms"] - values[1]) <= 2e-3
        assert values[1] - 2e-3 <= report[f"{key}_p95_ms"] <= values[2] + 2e-3
    assert 0 < report["kv_cache_byte_utilization"] <= 1
    # the workload ran once untimed and twice timed, with the same tokens both times
    assert report["warmup"] == 1 and report["steps"] == 2 and report["measured_tokens"] == 2 * 13 and report["warmup_ms"] > 0
    for generated, length, new in zip(report["generated"], (5, 9, 7), (4, 6, 3)):
        cyclic = [prompt[i % len(prompt)] for i in range(length)]
        assert generated == plain.generate_greedy(model.config, model.weights, cyclic, new)


def test_command_line_ways_of_generating(tmp_path, capsys):
    """The reference's switches for how tokens are generated: without the cache, the prompt token by token, argmax on
    the host, every prompt position's logits, the weights' precision by --bf16-ffn and --bf16-attention. All give
    the plain implementation's tokens; the cached run's last logits are those of the last generated position."""
    from microllm_rocm_amd.cli import hf_infer
    folder = make_folder(tmp_path, "A", SHARP)
    model = PlainModel(folder)
    prompt = random_tokens(5, 11, CONFIGS["A"].vocab_size)
    expected = plain.generate_greedy(model.config, model.weights, prompt, 5)
    base = ["--model", folder, "--tokens", ",".join(map(str, prompt)), "--new-tokens", "5", "--batch", "2"]
    cache_logits = tmp_path / "cache.f32"

    def run(*more):
        capsys.readouterr()
        assert hf_infer.main(base + list(more)) == 0
        return json.loads(capsys.readouterr().out.strip().splitlines()[-1])

    for more in (["--bf16-ffn", "false", "--bf16-attention", "false", "--use-cache", "false"],
                 ["--dtype", "float32", "--use-cache", "false", "--batch-argmax-mode", "host"],
                 ["--dtype", "float32", "--cache-prefill-mode", "token", "--cache-logits-output", str(cache_logits), "--steps", "2"],
                 ["--dtype", "float32", "--prefill-logits", "full", "--batch-argmax-mode", "host"]):
        report = run(*more)
        assert report["compute_dtype"] == "float32" and report["generated_tokens"] == expected, more
    # the logits that chose the last token: position prompt + 4 of the sequence, for both rows of the batch
    written = np.fromfile(cache_logits, dtype="<f4").reshape(2, -1)
    reference = model.logits(prompt + expected[:4])[-1]
    assert np.abs(written - reference[None, :]).max() <= 2e-5 * np.abs(reference).max()
    assert run("--bf16-ffn", "true", "--bf16-attention", "true")["compute_dtype"] == "bfloat16"
    for bad in (["--bf16-ffn", "true", "--bf16-attention", "false"], ["--bf16-ffn", "true"], ["--prefill-logits", "some"],
                ["--use-cache", "false", "--cache-logits-output", str(cache_logits)],
                ["--use-cache", "false", "--temperature", "0.7"]):
        assert hf_infer.main(base + bad) == 2, bad
        assert "microllm_hf_infer:" in capsys.readouterr().err


def test_command_line_value_trace(tmp_path, capsys):
    """--trace-output: one JSON line per layer with the residual stream after it and one for the logits, with the
    reference's field names; values and statistics against the plain implementation."""
    from microllm_rocm_amd.cli import hf_infer
    folder = make_folder(tmp_path, "B", SHARP)
    model = PlainModel(folder)
    config = CONFIGS["B"]
    prompt = random_tokens(8, 21, config.vocab_size)
    trace = tmp_path / "deep" / "trace.jsonl"
    base = ["--model", folder, "--tokens", ",".join(map(str, prompt)), "--dtype", "float32", "--workload", "prefill",
            "--trace-output", str(trace)]
    capsys.readouterr()
    assert hf_infer.main(base + ["--trace-max-elements", "50"]) == 0
    report = json.loads(capsys.readouterr().out.strip().splitlines()[-1])
    records = [json.loads(line) for line in trace.read_text().splitlines()]
    assert report["trace_records"] == len(records) == config.num_hidden_layers + 1
    streams = plain.layer_streams(model.config, model.weights, prompt)
    for layer, record in enumerate(records[:-1]):
        assert (record["sequence"], record["kind"], record["shape"]) == (layer, "layer", [1, len(prompt), config.hidden_size])
        assert record["values_truncated"] and len(record["values"]) == 50
        expected = streams[layer].reshape(-1)
        scale = np.abs(expected).max()
        assert np.abs(np.array(record["values"]) - expected[:50]).max() <= 2e-5 * scale
        statistics = record["statistics"]
        assert statistics["numel"] == statistics["finite_count"] == expected.size
        assert abs(statistics["l2_norm"] - np.sqrt((expected ** 2).sum())) <= 2e-5 * np.sqrt((expected ** 2).sum())
        assert abs(statistics["minimum"] - expected.min()) <= 2e-5 * scale and abs(statistics["maximum"] - expected.max()) <= 2e-5 * scale
    last = records[-1]
    reference = model.logits(prompt)[-1]
    assert last["kind"] == "model" and last["shape"] == [1, config.vocab_size]
    assert np.abs(np.array(last["values"]) - reference[:50]).max() <= 2e-5 * np.abs(reference).max()
    for bad in (["--trace-max-elements", "0"], ["--prefill-steps", "2"], ["--workload", "both"]):
        assert hf_infer.main(base + bad) == 2, bad
        assert "microllm_hf_infer:" in capsys.readouterr().err


def test_step_refuses_bad_batches_and_leaves_the_cache_as_it_was(tmp_path):
    from microllm_rocm_amd import StepEntry
    from microllm_rocm_amd.cache import OutOfPages
    folder = make_folder(tmp_path, "A", SHARP)
    engine = engine_for(folder, num_pages=4, max_tokens=None, max_requests=3)      # 64 positions in all
    engine.open("a")
    engine.open("b")
    with pytest.raises(ValueError, match="twice"):
        engine.step([StepEntry("a", [1]), StepEntry("a", [2])])
    with pytest.raises(ValueError, match="no tokens"):
        engine.step([StepEntry("a", [])])
    with pytest.raises(ValueError, match="outside the vocabulary"):
        engine.step([StepEntry("a", [1, 256])])
    with pytest.raises(ValueError, match="wanted place"):
        engine.step([StepEntry("a", [1, 2], [2])])
    with pytest.raises(KeyError, match="not open"):
        engine.step([StepEntry("zzz", [1])])
    with pytest.raises(ValueError, match="max positions"):
        engine.step([StepEntry("a", [1] * 129)])
    assert engine.cache.free_pages() == [4] and engine.cache.get("a").num_tokens == 0
    # the second entry does not fit: nothing of the first is kept either
    with pytest.raises(OutOfPages):
        engine.step([StepEntry("a", [1] * 40), StepEntry("b", [2] * 30)])
    assert engine.cache.free_pages() == [4] and engine.cache.get("a").reserved == 0 and engine.cache.get("a").num_tokens == 0
    engine.cache.check()
    logits = engine.step([StepEntry("a", [1] * 40, [39]), StepEntry("b", [2] * 10)])
    assert logits.shape == (1, 256) and engine.cache.free_pages() == [0]
    engine.open("c")
    with pytest.raises(OutOfPages, match="slots"):
        engine.open("d")
    engine.close("a")
    engine.close("b")
    engine.close("c")
    engine.cache.check()


def test_non_finite_logits_are_an_error(tmp_path):
    import torch
    from microllm_rocm_amd import GenerationConfig, generate
    from microllm_rocm_amd.sampling import NonFiniteLogits
    from microllm_rocm_amd.weights import SafetensorsFile, save_file
    folder = make_folder(tmp_path, "A", SHARP)
    path = os.path.join(folder, "model.safetensors")
    handle = SafetensorsFile(path)
    tensors = {name: handle.tensor(name).clone() for name in handle.names()}
    tensors["model.norm.weight"][3] = float("nan")
    save_file(tensors, path)
    engine = engine_for(folder)
    with pytest.raises(NonFiniteLogits):        # src/inference/scheduler.cpp:918-920
        generate(engine, [[1, 2, 3]], GenerationConfig(max_new_tokens=2, temperature=0.0))
    with pytest.raises(NonFiniteLogits):
        generate(engine_for(folder, "bfloat16"), [[1, 2, 3]], GenerationConfig(max_new_tokens=2, temperature=0.7))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_few_pages_preempt_with_a_window_and_seeded_sampling(tmp_path, dtype):
    """Tiny B (window 24 in layers 1 and 2, so two cache groups) with temperature 0.8 and top-k: requests that are
    thrown out for want of pages and run again continue their own stream of draws."""
    from microllm_rocm_amd import GenerationConfig, generate
    folder = make_folder(tmp_path, "B", SHARP)
    config = CONFIGS["B"]
    prompts = [random_tokens(70 + index, length, config.vocab_size) for index, length in enumerate((30, 41, 25, 36))]
    params = [GenerationConfig(max_new_tokens=40, temperature=0.8, top_k=(0, 20)[index % 2], seed=10 + index) for index in range(4)]
    roomy = generate(engine_for(folder, dtype, max_tokens=2048), prompts, params, prefill_chunk=16)
    tight_engine = engine_for(folder, dtype, num_pages=12, max_tokens=None)     # 192 positions for 4 requests of up to 81
    tight, scheduler = generate(tight_engine, prompts, params, prefill_chunk=16, return_scheduler=True)
    assert scheduler.metrics.preemptions >= 1
    model = PlainModel(folder)

    def same_streams(got, expected):
        """Equal token for token in float32. In bfloat16 a request that is run again takes other kernels for the
        tokens it had generated (a portion instead of single tokens), which round differently: a draw may then fall
        on the other side of an interval's edge, and from there on the streams are different samples. The first
        difference of a request must be such a draw: its uniform lies within 2e-2 of an edge of the plain rule's
        cumulative distribution over the shared prefix (bfloat16 logits move the edges by about that much)."""
        if dtype == "float32":
            assert got == expected
            return
        exact = 0
        for sequence, other, prompt, p in zip(got, expected, prompts, params):
            if sequence == other:
                exact += 1
                continue
            first = next(index for index, (a, b) in enumerate(zip(sequence, other)) if a != b)
            assert first >= len(prompt)
            weights = plain.sampling_weights(model.logits(sequence[:first])[-1], p.temperature, p.top_k)
            cumulative = np.cumsum(weights) / weights.sum()
            assert min(abs(cumulative - plain.uniform_for(p.seed, first - len(prompt)))) < 2e-2
        assert exact >= len(got) // 2

    same_streams(tight, roomy)
    assert len(tight_engine.cache.groups) == 2 and tight_engine.cache.free_pages() == [12, 12]
    tight_engine.cache.check()
    # the same with the windowed group's pool sized for portions of 16: 4 slots x ceil((24 - 1 + 16) / 16) + 1 pages
    sized = engine_for(folder, dtype, num_pages=40, max_tokens=None, max_requests=4, max_portion=16)
    assert [group.pool.num_pages for group in sized.cache.groups] == [40, 16]
    same_streams(generate(sized, prompts, params, prefill_chunk=64), roomy)     # the scheduler keeps to the engine's portion
    assert sized.cache.free_pages() == [40, 16]
    with pytest.raises(ValueError, match="portions of at most 16"):
        sized.open("long")
        sized.step([("long", list(range(17)), [])])
    sized.close("long")


def test_a_step_that_fails_inside_the_model_is_rolled_back(tmp_path):
    """A part that raises in ``forward`` when told to, registered from here and put into the second layer: the
    failed step leaves no reservation, no page and no position behind, and the next step gives what it should."""
    from microllm_rocm_amd import Engine, StepEntry
    from microllm_rocm_amd.config.registry import load_config
    from microllm_rocm_amd.parts import FeedForward, PartSpec, register_part, unregister_part
    from microllm_rocm_amd.parts.feedforward import SwiGLU
    from microllm_rocm_amd.weights import load_folder
    import dataclasses

    class Moody(SwiGLU):
        fail = False

        def forward(self, x, ctx, residual=None):
            if Moody.fail:
                raise RuntimeError("the feed-forward refuses")
            return super().forward(x, ctx, residual=residual)

    register_part("ffn", "moody_swiglu", Moody)
    try:
        folder = make_folder(tmp_path, "A", SHARP)
        architecture, config = load_config(folder)
        spec = architecture.build_spec(config)
        layers = list(spec.layers)
        layers[1] = dataclasses.replace(layers[1], ffn=dataclasses.replace(layers[1].ffn, kind="moody_swiglu"))
        spec = dataclasses.replace(spec, layers=tuple(layers))
        from microllm_rocm_amd.parts import Model, Runtime
        for dtype in (torch.float32, torch.bfloat16):
            tensors = load_folder(folder, Model(spec, Runtime(dtype, torch.device("cpu"))).tensors(), dtype, torch.device("cuda:0"))
            engine = Engine(spec, tensors, dtype=dtype, num_pages=8, tensors_placed=True)
            reference = engine_for(folder, dtype, num_pages=8, max_tokens=None)
            prompt_a, prompt_b = random_tokens(1, 40, 256), random_tokens(2, 21, 256)
            for e in (engine, reference):
                e.open("a"), e.open("b")
                e.step([StepEntry("a", prompt_a[:30], [])])
            Moody.fail = True
            for entries in ([StepEntry("a", prompt_a[30:], [9]), StepEntry("b", prompt_b, [20])],      # a mixed step
                            [StepEntry("a", [prompt_a[30]], [0])]):                                      # a decode step (graph)
                with pytest.raises(RuntimeError, match="refuses"):
                    engine.step(entries)
                engine.cache.check()
                assert engine.cache.get("a").num_tokens == 30 and engine.cache.get("a").reserved == 0
                assert engine.cache.get("b").num_tokens == 0 and engine.cache.get("b").reserved == 0
                assert engine.cache.held_pages() == [2]
            Moody.fail = False
            got = engine.step([StepEntry("a", prompt_a[30:], [9]), StepEntry("b", prompt_b, [20])])
            expected = reference.step([StepEntry("a", prompt_a[30:], [9]), StepEntry("b", prompt_b, [20])])
            assert torch.equal(got, expected)
            token = int(got[0].argmax())
            assert torch.equal(engine.step([StepEntry("a", [token], [0])]), reference.step([StepEntry("a", [token], [0])]))
            engine.cache.check()
    finally:
        Moody.fail = False
        unregister_part("ffn", "moody_swiglu")


def test_logits_of_a_step_are_the_callers_to_keep(tmp_path):
    """Decode steps are replayed from a graph that writes its logits to the same buffer every time: what ``step``
    returns is a copy unless the caller says it only borrows."""
    from microllm_rocm_amd import StepEntry
    folder = make_folder(tmp_path, "A", SHARP)
    engine = engine_for(folder, "bfloat16")
    assert engine.use_graphs
    engine.open("a")
    engine.step([StepEntry("a", [5, 6, 7], [])])
    kept, copies = [], []
    for token in (9, 10, 11, 12):
        logits = engine.step([StepEntry("a", [token], [0])])
        kept.append(logits)
        copies.append(logits.clone())
    assert engine.graph_replays >= 3
    for logits, copy in zip(kept, copies):
        assert torch.equal(logits, copy)
    assert not torch.equal(kept[0], kept[1])
    borrowed = engine.step([StepEntry("a", [13], [0])], borrow_logits=True)
    before = borrowed.clone()
    engine.step([StepEntry("a", [14], [0])], borrow_logits=True)
    assert not torch.equal(borrowed, before)          # the buffer of the graph: the next step has overwritten it


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["A", "B"])
def test_mixed_steps_replayed_from_graphs_equal_eager_steps(tmp_path, dtype, which):
    """Steps that mix portions of prompts with single tokens are padded to a fixed shape and replayed from a graph once
    the shape has come twice: every such step gives the bits of the same step run eagerly, whatever the padding
    (the numbers of tokens, requests, wanted rows and attention tiles change from step to step within a shape), and
    the keys and values it stores are what later steps read."""
    from microllm_rocm_amd.engine import StepEntry
    folder = make_folder(tmp_path, which, SHARP)
    config = CONFIGS[which]
    graphs = engine_for(folder, dtype, use_graphs=True, num_pages=24, max_tokens=None, max_requests=8)
    eager = engine_for(folder, dtype, use_graphs=False, num_pages=24, max_tokens=None, max_requests=8)
    rng = np.random.default_rng(3)

    def both(entries):
        out = [engine.step([StepEntry(*entry) for entry in entries]) for engine in (graphs, eager)]
        torch.cuda.synchronize()
        assert (out[0] is None) == (out[1] is None)
        if out[0] is not None:
            assert out[0].shape == out[1].shape and torch.equal(out[0], out[1]), "a replayed step differs from the eager step"

    def tokens(count):
        return rng.integers(0, config.vocab_size, size=count).tolist()

    for round_index in range(6):
        names = [f"r{round_index}_{index}" for index in range(4)]
        for engine in (graphs, eager):
            for name in names:
                engine.open(name)
        # two requests decode while the other two bring portions of 9 to 16 and 17 to 24 tokens: the same padded
        # shapes in every round (16, 32 or 48 rows of tokens; 4 requests), other contents
        both([(names[0], tokens(5), [4]), (names[1], tokens(11), [10])])
        for step in range(5):
            first, second = int(rng.integers(9, 17)), int(rng.integers(17, 25))
            wanted = [[0], [0], [first - 1], []] if step % 2 else [[0], [], [0, first - 1], [second - 1]]
            both([(names[0], tokens(1), wanted[0]), (names[1], tokens(1), wanted[1]),
                  (names[2], tokens(first), wanted[2]), (names[3], tokens(second), wanted[3])])
        both([(name, tokens(1), [0]) for name in names])          # and a decode step over what the mixed steps stored
        both([(names[2], tokens(2), [1]), (names[0], tokens(1), [0])])
        for engine in (graphs, eager):
            for name in names:
                engine.close(name)
            engine.cache.check()
    assert graphs.mixed_graph_replays >= 15 and eager.graph_replays == 0
    pool = graphs.cache.groups[0].pool
    assert pool.total_taken > pool.num_pages, "pages were used again"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_step_copies_its_metadata_once_and_nothing_back(tmp_path, dtype):
    """The copies between host and device that the engine makes are counted: a step moves one packed buffer of
    metadata to the device and nothing to the host (a decode step from a graph: its tokens, and the next step's
    metadata built ahead); selecting tokens moves the chosen ids back, one copy a step. The reference holds a
    forward to no copy to the host the same way (tests/inference/hip_shape_matrix_test.cpp:101-136)."""
    from microllm_rocm_amd import GenerationConfig, generate
    from microllm_rocm_amd.engine import StepEntry
    from microllm_rocm_amd.ops.transfers import reset_transfer_stats, transfer_stats
    folder = make_folder(tmp_path, "B", SHARP)
    config = CONFIGS["B"]
    engine = engine_for(folder, dtype)
    prompts = {name: random_tokens(60 + index, length, config.vocab_size) for index, (name, length) in enumerate((("a", 40), ("b", 9), ("c", 21)))}
    for name in prompts:
        engine.open(name)
    reset_transfer_stats()
    logits = engine.step([StepEntry("a", prompts["a"], [39]), StepEntry("b", prompts["b"][:5], [])])      # portions of prompts
    moved = transfer_stats()
    assert (moved.host_to_device_calls, moved.device_to_host_calls) == (1, 0) and 0 < moved.host_to_device_bytes < 4096
    engine.step([StepEntry("a", [3], [0]), StepEntry("b", prompts["b"][5:], [3]), StepEntry("c", prompts["c"], [])])   # mixed
    moved = transfer_stats()
    assert (moved.host_to_device_calls, moved.device_to_host_calls) == (2, 0)
    for _ in range(4):                                                                                        # single tokens
        before = transfer_stats()
        logits = engine.step([StepEntry(name, [5], [0]) for name in prompts], borrow_logits=True)
        moved = transfer_stats()
        assert moved.device_to_host_calls == 0 and 1 <= moved.host_to_device_calls - before.host_to_device_calls <= 2
    assert engine.graph_replays == 4 and engine.steps_built_ahead >= 2
    torch.cuda.synchronize()
    assert torch.isfinite(logits).all()
    for name in prompts:
        engine.close(name)
    reset_transfer_stats()
    generate(engine, [prompts["b"]], GenerationConfig(max_new_tokens=6, temperature=0.0))
    moved = transfer_stats()
    assert moved.device_to_host_calls == 6 and moved.device_to_host_bytes == 6 * 4, "the chosen id of every step, nothing else"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_lookahead_generates_the_same_tokens(tmp_path, dtype):
    """Steps launched before the host has seen the tokens of the step before (they take them from the device) give
    what waiting for every token gives: greedy and sampled, prompts in portions beside decoding, arrivals at
    different steps, and a pool so small that requests are preempted and run again from ids the host must have."""
    from microllm_rocm_amd import GenerationConfig, generate
    folder = make_folder(tmp_path, "B", SHARP)
    config = CONFIGS["B"]
    prompts = [random_tokens(80 + index, length, config.vocab_size) for index, length in enumerate((5, 17, 40, 64, 9, 33))]
    params = [GenerationConfig(max_new_tokens=20 + index, temperature=(0.0, 0.8)[index % 2], seed=index, top_k=(0, 20, 0)[index % 3])
              for index in range(len(prompts))]
    for options in ({"max_tokens": 2048}, {"num_pages": 9, "max_tokens": None}):
        engine = engine_for(folder, dtype, max_requests=4, **options)
        common = dict(prefill_chunk=16, max_batched_tokens=32, arrival_steps=[0, 0, 2, 3, 9, 9], return_scheduler=True)
        waited, slow = generate(engine, prompts, params, lookahead=False, **common)
        ahead, fast = generate(engine, prompts, params, lookahead=True, **common)
        assert ahead == waited
        assert fast.metrics.preemptions == slow.metrics.preemptions and (fast.metrics.preemptions > 0) == ("num_pages" in options)
        assert all(token >= 0 for output in ahead for token in output)
        engine.cache.check()
        assert not engine.cache.requests


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_timed_decode_loop_gives_the_same_tokens_with_and_without_lookahead(tmp_path, dtype):
    """The benchmark's decode loop, which takes a step's tokens from the ids that the step before left on the
    device, decodes what the loop that waits for every step's ids decodes, and leaves the cache as it found it."""
    from microllm_rocm_amd.engine.benchmark import decode_throughput
    folder = make_folder(tmp_path, "A", SHARP)
    results = []
    for lookahead, warmup in ((False, 2), (True, 2), (True, 0), (False, 0)):
        engine = engine_for(folder, dtype, max_tokens=4 * 128, max_requests=4)      # the same pages for the same requests
        torch.manual_seed(5)       # the caches are filled with random keys and values
        results.append(decode_throughput(engine, 3, 40, steps=9, warmup=warmup, seed=1, lookahead=lookahead))
        engine.cache.check()
        assert not engine.cache.requests
    assert results[0]["last_tokens"] == results[1]["last_tokens"] and len(results[0]["last_tokens"]) == 3
    assert results[2]["last_tokens"] == results[3]["last_tokens"]
    assert all(result["tokens_per_second"] > 0 for result in results)
