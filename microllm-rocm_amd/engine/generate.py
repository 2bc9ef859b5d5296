"""Generation: the Python entry point above the scheduler.

``generate`` is the reference's call (src/inference/generator.cpp:71-151): token
ids in, the prompt followed by the new tokens out; here it takes several prompts
at once and runs them through the continuous-batching scheduler.
``generate_serial`` runs one request at a time, the way the reference's serial
scheduler does (src/inference/scheduler.cpp:195-230); batched generation must
give the same tokens.
"""
from __future__ import annotations

from typing import List, Optional, Sequence, Union

from ..sampling import Sampler, SamplingParams
from .batch import StepEntry
from .engine import Engine
from .scheduler import Scheduler

GenerationConfig = SamplingParams  # the reference's name (include/microllm/inference/generator.h:11)


def _params_list(params, count: int) -> List[SamplingParams]:
    if params is None:
        params = SamplingParams()
    if isinstance(params, SamplingParams):
        return [params] * count
    params = list(params)
    if len(params) != count:
        raise ValueError("one SamplingParams per prompt, or one for all")
    return params


def generate(engine: Engine, prompts: Sequence[Sequence[int]],
             params: Union[None, SamplingParams, Sequence[SamplingParams]] = None,
             max_batched_tokens: int = 2048, prefill_chunk: int = 512, max_requests: Optional[int] = None,
             arrival_steps: Optional[Sequence[int]] = None, return_scheduler: bool = False, lookahead: bool = True):
    """Prompt plus generated tokens for every prompt, in input order. With ``lookahead`` (the default: nobody looks
    at a token before the end) a step is launched before the host has seen the tokens of the step before
    (``Scheduler``); the tokens are the same."""
    single = bool(prompts) and isinstance(prompts[0], int)
    if single:
        prompts = [prompts]
    param_list = _params_list(params, len(prompts))
    scheduler = Scheduler(engine, max_batched_tokens=max_batched_tokens, prefill_chunk=prefill_chunk,
                          max_requests=max_requests, lookahead=lookahead)
    ids = []
    for index, (prompt, request_params) in enumerate(zip(prompts, param_list)):
        arrival = arrival_steps[index] if arrival_steps is not None else None
        ids.append(scheduler.submit(prompt, request_params, arrival_step=arrival))
    scheduler.run_until_idle()
    outputs = [list(scheduler.request(i).prompt) + list(scheduler.request(i).generated) for i in ids]
    if return_scheduler:
        return (outputs[0] if single else outputs), scheduler
    return outputs[0] if single else outputs


def generate_serial(engine: Engine, prompt: Sequence[int], params: Optional[SamplingParams] = None,
                    sampler: Optional[Sampler] = None) -> List[int]:
    """One request alone: the whole prompt in one step, then one token a step."""
    params = params or SamplingParams()
    params.validate(engine.spec.vocab_size)
    sampler = sampler or Sampler()
    tokens = [int(token) for token in prompt]
    if not tokens:
        raise ValueError("generation prompt cannot be empty")
    if len(tokens) + params.max_new_tokens > engine.spec.max_positions:
        raise ValueError("prompt plus generated tokens exceeds model context")
    if params.max_new_tokens == 0:
        return tokens
    request_id = ("serial", id(tokens))
    engine.open(request_id)
    try:
        logits = engine.step([StepEntry(request_id, tokens, [len(tokens) - 1])])
        for generated in range(params.max_new_tokens):
            token = sampler.select(logits, [params], [generated])[0]
            tokens.append(token)
            if token in params.stop_tokens or generated + 1 == params.max_new_tokens:
                break
            logits = engine.step([StepEntry(request_id, [token], [0])], borrow_logits=True)
    finally:
        engine.close(request_id)
    return tokens
