"""The scheduler's decisions, with a stand-in for the engine that keeps the cache's books but runs no model.
No GPU: logits are a fixed function of the tokens a request has fed so far, so that running a request again
after a preemption must give the same tokens."""
import hashlib
from types import SimpleNamespace

import numpy as np
import pytest
import torch

import plain_qwen2 as plain
from microllm_rocm_amd.cache import CacheManager
from microllm_rocm_amd.engine.scheduler import CompletionReason, RequestState, Scheduler
from microllm_rocm_amd.parts import PagedKVNeed
from microllm_rocm_amd.sampling import SamplingParams

VOCAB = 40


def logits_after(tokens):
    digest = hashlib.sha256(repr(list(tokens)).encode()).digest()
    return np.random.default_rng(int.from_bytes(digest[:8], "little")).normal(size=VOCAB)


class FakeEngine:
    def __init__(self, num_pages=16, page_size=4, max_requests=4, max_positions=256, window=None):
        need = PagedKVNeed(1, 8, window)
        self.cache = CacheManager([need], [None], page_size, num_pages, max_requests, device=None)
        self.spec = SimpleNamespace(vocab_size=VOCAB, max_positions=max_positions)
        self.fed = {}
        self.batches = []
        self.from_device = 0

    def step(self, entries, reserved=False, borrow_logits=False, device_tokens=None):
        assert reserved
        rows = []
        self.batches.append([(entry.request_id, len(entry.tokens)) for entry in entries])
        self.from_device += sum(entry.token_from is not None for entry in entries)
        for entry in entries:
            request = self.cache.get(entry.request_id)
            history = self.fed.setdefault(entry.request_id, [])
            if request.num_tokens == 0:
                history.clear()               # run again after a preemption
            assert len(history) == request.num_tokens
            tokens = list(entry.tokens)
            if entry.token_from is not None:  # an id the host has not seen: the step reads it where it was selected
                assert len(tokens) == 1
                tokens = [int(device_tokens[entry.token_from])]
            assert all(0 <= token < VOCAB for token in tokens)
            history.extend(tokens)
            for place in entry.want:
                rows.append(logits_after(history[:request.num_tokens + place + 1]))
            self.cache.commit(request, len(entry.tokens))
        self.cache.check()
        return torch.tensor(np.array(rows), dtype=torch.float32) if rows else None


class PlainSampler:
    def select(self, logits, params, draws):
        return [plain.sample(row.numpy().astype(np.float64), p.temperature, p.top_k, plain.uniform_for(p.seed, d))
                for row, p, d in zip(logits, params, draws)]

    def select_later(self, logits, params, draws):
        """What ``Sampler.select_later`` returns: the ids where the next step can read them, and a way to ask for
        them; asked, it counts, so that a test can tell whether the scheduler waited."""
        chosen = self.select(logits, params, draws)
        sampler = self

        class Later:
            device = torch.tensor(chosen, dtype=torch.int32)

            def tokens(self):
                sampler.asked_later = getattr(sampler, "asked_later", 0) + 1
                return list(chosen)

        return Later()


def alone(prompt, params):
    """What one request generates when nothing else runs: the oracle every schedule must match."""
    tokens = list(prompt)
    out = []
    for draw in range(params.max_new_tokens):
        token = plain.sample(logits_after(tokens), params.temperature, params.top_k, plain.uniform_for(params.seed, draw))
        tokens.append(token)
        out.append(token)
        if token in params.stop_tokens:
            break
    return out


def scheduler(engine=None, **options):
    return Scheduler(engine or FakeEngine(), sampler=PlainSampler(), **options)


GREEDY = SamplingParams(max_new_tokens=5, temperature=0.0)


def test_single_request_chunks_its_prompt_under_the_budget():
    engine = FakeEngine()
    s = scheduler(engine, max_batched_tokens=8, prefill_chunk=6)
    rid = s.submit(list(range(15)), GREEDY)
    s.run_until_idle()
    assert [batch for batch in engine.batches[:3]] == [[(rid, 6)], [(rid, 6)], [(rid, 3)]]
    assert all(batch == [(rid, 1)] for batch in engine.batches[3:]) and len(engine.batches) == 3 + 4
    request = s.request(rid)
    assert request.generated == alone(range(15), GREEDY)
    assert request.state == RequestState.COMPLETED and request.completion_reason == CompletionReason.LENGTH
    assert engine.cache.free_pages() == [16] and engine.cache.slots.num_free == 4
    assert s.metrics.prefill_tokens == 15 and s.metrics.decode_tokens == 4 and s.metrics.completed_requests == 1


def test_decodes_go_first_and_prompts_share_the_rest_of_the_budget():
    engine = FakeEngine(num_pages=64)
    s = scheduler(engine, max_batched_tokens=10, prefill_chunk=8)
    first = s.submit([1, 2, 3], SamplingParams(max_new_tokens=6, temperature=0.0))
    s.step()                                           # first is prefilled whole and decodes from now on
    second = s.submit(list(range(20)), GREEDY)
    third = s.submit(list(range(5)), GREEDY)
    s.step()
    assert engine.batches[-1] == [(first, 1), (second, 8), (third, 1)]   # 10 tokens: 1 + 8 + what is left
    s.step()
    assert engine.batches[-1] == [(first, 1), (second, 8), (third, 1)]
    s.step()
    assert engine.batches[-1] == [(first, 1), (second, 4), (third, 3)]
    s.run_until_idle()
    for rid, prompt, params in ((first, [1, 2, 3], SamplingParams(max_new_tokens=6, temperature=0.0)),
                                (second, range(20), GREEDY), (third, range(5), GREEDY)):
        assert s.request(rid).generated == alone(prompt, params)


def test_admission_is_first_come_first_served_and_respects_slots_and_arrivals():
    engine = FakeEngine(max_requests=2, num_pages=64)
    s = scheduler(engine)
    ids = [s.submit([i + 1, i + 2], SamplingParams(max_new_tokens=2 + i, temperature=0.0)) for i in range(3)]
    late = s.submit([9, 9], GREEDY, arrival_step=6)
    s.step()
    assert [r for r, _ in engine.batches[-1]] == ids[:2]
    assert s.request(ids[2]).state == RequestState.PENDING_PREFILL and not s.request(ids[2]).admitted
    s.step()                                           # the first finishes (2 tokens), freeing a slot
    assert s.request(ids[0]).state == RequestState.COMPLETED
    s.step()
    assert ids[2] in [r for r, _ in engine.batches[-1]]
    s.run_until_idle()
    assert s.request(late).admission_order == 3 and s.request(late).completion_step >= 6
    assert min(index for index, batch in enumerate(engine.batches) if late in [r for r, _ in batch]) >= 3
    assert s.metrics.peak_active_requests == 2


def test_stop_tokens_cancel_and_zero_length():
    engine = FakeEngine()
    s = scheduler(engine)
    free_run = alone([5, 6, 7], SamplingParams(max_new_tokens=8, temperature=0.0))
    stop = free_run[2]
    params = SamplingParams(max_new_tokens=8, temperature=0.0, stop_tokens=(stop,))
    rid = s.submit([5, 6, 7], params)
    empty = s.submit([1], SamplingParams(max_new_tokens=0))
    assert s.request(empty).state == RequestState.COMPLETED and s.request(empty).generated == []
    doomed = s.submit([2, 3], GREEDY)
    s.step()
    assert s.cancel(doomed) is True and s.cancel(doomed) is False     # terminal and idempotent
    assert s.request(doomed).state == RequestState.CANCELLED and len(s.request(doomed).generated) == 1
    with pytest.raises(KeyError):
        s.cancel(999)
    s.run_until_idle()
    request = s.request(rid)
    first_stop = free_run.index(stop)
    assert request.generated == free_run[:first_stop + 1]             # the stop token is emitted, then it stops
    assert request.completion_reason == CompletionReason.STOP_TOKEN and s.metrics.stop_completed_requests == 1
    assert engine.cache.free_pages() == [16] and engine.cache.slots.num_free == 4
    waiting = s.submit([4], GREEDY, arrival_step=100)
    assert s.cancel(waiting) is True and not s.has_work()


def test_submit_validation():
    s = scheduler(FakeEngine(num_pages=4, page_size=4, max_positions=32))
    with pytest.raises(ValueError, match="at least one token"):
        s.submit([])
    with pytest.raises(ValueError, match="outside the vocabulary"):
        s.submit([VOCAB])
    with pytest.raises(ValueError, match="max positions"):
        s.submit([1] * 30, SamplingParams(max_new_tokens=3))
    with pytest.raises(ValueError, match="more than the cache holds"):
        s.submit([1] * 10, SamplingParams(max_new_tokens=7))
    for bad in (SamplingParams(max_new_tokens=-1), SamplingParams(temperature=-0.5), SamplingParams(temperature=float("nan")),
                SamplingParams(top_k=VOCAB + 1), SamplingParams(stop_tokens=(3, 3)), SamplingParams(stop_tokens=(VOCAB,))):
        with pytest.raises(ValueError):
            s.submit([1], bad)


def test_running_out_of_pages_preempts_the_latest_and_recomputes():
    # 8 pages of 4 tokens. Two requests of 10 + 12 tokens each need 6 pages in the end: they cannot both finish.
    engine = FakeEngine(num_pages=8, page_size=4)
    s = scheduler(engine, max_batched_tokens=64, prefill_chunk=64)
    params = [SamplingParams(max_new_tokens=12, temperature=0.9, seed=3), SamplingParams(max_new_tokens=12, temperature=0.0)]
    prompts = [list(range(10)), list(range(20, 30))]
    ids = [s.submit(prompt, p) for prompt, p in zip(prompts, params)]
    s.run_until_idle(maximum_steps=200)
    assert s.metrics.preemptions >= 1 and s.request(ids[1]).preemptions >= 1 and s.request(ids[0]).preemptions == 0
    for rid, prompt, p in zip(ids, prompts, params):
        assert s.request(rid).generated == alone(prompt, p)           # recomputation continues the same stream
    assert engine.cache.free_pages() == [8] and engine.cache.slots.num_free == 4
    # the preempted request was run again from position 0 with its prompt and what it had generated
    again = [batch for batch in engine.batches if any(r == ids[1] and n > 10 for r, n in batch)]
    assert again


def test_a_preempted_request_waits_for_room_instead_of_being_thrown_out_again_and_again():
    # 8 pages of 4 tokens. The older request grows to 10 + 20 = 30 tokens (8 pages): it needs every page the
    # younger one holds, one after the other. The younger one is preempted once and comes back when the older has
    # finished; it is not admitted into the page or two that are free meanwhile, which would cost a recomputation
    # of its prompt for every page the older one takes.
    engine = FakeEngine(num_pages=8, page_size=4)
    s = scheduler(engine, max_batched_tokens=64, prefill_chunk=4)     # portions of one page: one always "fits"
    older = s.submit(list(range(10)), SamplingParams(max_new_tokens=20, temperature=0.0))
    young = SamplingParams(max_new_tokens=16, temperature=0.7, seed=1)
    younger = s.submit(list(range(20, 26)), young)
    s.run_until_idle(maximum_steps=200)
    assert s.request(older).preemptions == 0 and s.request(younger).preemptions == 1
    assert s.metrics.preemptions == 1
    assert s.request(younger).generated == alone(range(20, 26), young)
    assert s.request(older).generated == alone(range(10), SamplingParams(max_new_tokens=20, temperature=0.0))
    # tokens run through the model: both requests once, and the younger one's prompt and what it had generated again
    fed_younger = sum(n for batch in engine.batches for r, n in batch if r == younger)
    assert fed_younger <= 2 * (6 + 16)
    assert s.metrics.prefill_tokens + s.metrics.decode_tokens == sum(n for batch in engine.batches for _, n in batch)
    assert engine.cache.free_pages() == [8]


class FailingEngine(FakeEngine):
    """Raises inside the step whose number is given, after the scheduler has reserved its pages."""

    def __init__(self, fail_at, state=False, **options):
        super().__init__(**options)
        self.fail_at = fail_at
        self.calls = 0
        if state:
            from microllm_rocm_amd.parts import StateNeed
            self.cache = CacheManager([PagedKVNeed(1, 8, None), StateNeed((2,))], [None, None], 4, 16, 4, device=None)

    def step(self, entries, reserved=False, borrow_logits=False, device_tokens=None):
        self.calls += 1
        if self.calls == self.fail_at:
            # what Engine.step does when the model raises: the step's reservations are given back
            for entry in entries:
                self.cache.cancel_reservation(self.cache.get(entry.request_id))
            raise RuntimeError("a kernel refused its arguments")
        return super().step(entries, reserved, device_tokens=device_tokens)


@pytest.mark.parametrize("state", [False, True])
def test_a_failed_step_counts_for_nothing_and_the_next_one_goes_on(state):
    engine = FailingEngine(fail_at=3, state=state)
    s = scheduler(engine, max_batched_tokens=8, prefill_chunk=4)
    params = SamplingParams(max_new_tokens=4, temperature=0.0)
    first, second = s.submit(list(range(9)), params), s.submit(list(range(30, 35)), params)
    s.step()
    s.step()
    before = (s.metrics.prefill_tokens, s.metrics.decode_tokens, s.metrics.engine_steps)
    with pytest.raises(RuntimeError, match="refused"):
        s.step()
    assert (s.metrics.prefill_tokens, s.metrics.decode_tokens, s.metrics.engine_steps) == before and s.metrics.failed_steps == 1
    engine.cache.check()
    assert all(request.reserved == 0 for request in engine.cache.requests.values())
    if state:      # per-request state may hold a part of the failed step: every request of it starts again
        assert not engine.cache.requests and [r.computed for r in s.requests.values()] == [0, 0]
        assert s.metrics.preemptions == 0
    else:          # pages hold nothing beyond the positions that count: the requests go on where they were
        assert sorted(r.computed for r in s.requests.values()) == sorted(
            engine.cache.get(rid).num_tokens for rid in (first, second))
    s.run_until_idle(maximum_steps=100)
    assert s.request(first).generated == alone(range(9), params)
    assert s.request(second).generated == alone(range(30, 35), params)
    assert engine.cache.free_pages() == [16] and engine.cache.slots.num_free == 4


def test_a_request_alone_always_fits_and_idle_limit_is_an_error():
    engine = FakeEngine(num_pages=4, page_size=4)
    s = scheduler(engine, max_batched_tokens=5, prefill_chunk=5)
    rid = s.submit(list(range(9)), SamplingParams(max_new_tokens=7, temperature=0.0))    # 16 tokens = all 4 pages
    s.run_until_idle()
    assert s.request(rid).generated == alone(range(9), SamplingParams(max_new_tokens=7, temperature=0.0))
    s.submit(list(range(9)), GREEDY)
    with pytest.raises(RuntimeError, match="did not become idle"):
        s.run_until_idle(maximum_steps=2)


@pytest.mark.parametrize("lookahead", [False, True])
@pytest.mark.parametrize("seed", range(6))
def test_random_workloads_match_requests_run_alone(seed, lookahead):
    """Also with ``lookahead``, where the host learns a step's tokens while the next step runs: the pool is small
    enough for preemptions (recomputation needs the ids on the host), some requests have stop tokens (waited for
    as ever), and every token must be what the request generates alone."""
    rng = np.random.default_rng(seed)
    engine = FakeEngine(num_pages=int(rng.integers(10, 24)), page_size=4, max_requests=3, window=None if seed % 2 else 12)
    s = scheduler(engine, max_batched_tokens=int(rng.integers(4, 20)), prefill_chunk=int(rng.integers(2, 12)), lookahead=lookahead)
    jobs = []
    for index in range(8):
        prompt = rng.integers(0, VOCAB, size=int(rng.integers(1, 14))).tolist()
        stops = tuple(rng.choice(VOCAB, size=3, replace=False).tolist()) if seed >= 4 and index % 3 == 0 else ()
        params = SamplingParams(max_new_tokens=int(rng.integers(1, 12)), temperature=float(rng.choice([0.0, 0.8])),
                                top_k=int(rng.choice([0, 5])), seed=index, stop_tokens=stops)
        jobs.append((s.submit(prompt, params, arrival_step=int(rng.integers(0, 10))), prompt, params))
    s.run_until_idle(maximum_steps=2000)
    for rid, prompt, params in jobs:
        assert s.request(rid).generated == alone(prompt, params)
        assert s.request(rid).first_token_time > 0 and s.request(rid).completion_time >= s.request(rid).first_token_time
    assert engine.cache.free_pages() == [engine.cache.groups[0].pool.num_pages]
    if not lookahead:
        assert engine.from_device == 0
    elif seed < 4:      # (a step that selects for a request with stop tokens waits, for all its requests)
        assert engine.from_device > 0, "with lookahead steps take tokens that the host has not seen"


def test_lookahead_learns_a_step_s_tokens_one_step_late_and_all_of_them_in_the_end():
    engine = FakeEngine(num_pages=32, page_size=4)
    sampler = PlainSampler()
    s = Scheduler(engine, sampler=sampler, lookahead=True)
    params = SamplingParams(max_new_tokens=6, temperature=0.0)
    first, second = s.submit([1, 2, 3], params), s.submit([4, 5], params)
    s.step()                                      # both prompts; their first tokens are selected, not waited for
    assert s.request(first).generated == [-1] and getattr(sampler, "asked_later", 0) == 0
    s.step()                                      # launched with ids from the device, then the first step's are learnt
    assert sampler.asked_later == 1 and s.request(first).generated[0] >= 0 and s.request(first).generated[1] == -1
    assert engine.from_device == 2
    s.run_until_idle()
    assert s.request(first).generated == alone([1, 2, 3], params) and s.request(second).generated == alone([4, 5], params)
    assert all(token >= 0 for rid in (first, second) for token in s.request(rid).generated)
    # a request with stop tokens is waited for in the step that selects for it
    stopping = SamplingParams(max_new_tokens=6, temperature=0.0, stop_tokens=(alone([7, 8], params)[2],))
    third = s.submit([7, 8], stopping)
    s.run_until_idle()
    assert s.request(third).generated == alone([7, 8], stopping) and len(s.request(third).generated) == 3
    assert s.request(third).completion_reason.value == "stop_token"
