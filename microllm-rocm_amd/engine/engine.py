"""The engine: a model, its cache and the one step function.

``step`` takes a batch of (request, its next tokens, wanted places): portions of
prompts beside single decoded tokens, cut anywhere. It runs only those tokens,
as one batch, against what earlier steps left in the cache, and returns the
float32 logits at the wanted places. The reference has five entry points, each
with its own batch shape (src/model/model.cpp:1091-1135, 1263-1303, 1316-1354,
1419-1439, 1448-1572); this is the one that replaces them.
"""
from __future__ import annotations

import os
from typing import Dict, Hashable, List, Mapping, Optional, Sequence, Union

import numpy as np
import torch

from ..cache.manager import CacheManager, RequestCache, pages_of_group
from ..cache.pages import OutOfPages
from ..config.registry import architecture_named, load_config
from ..ops import kernels, library
from ..ops.transfers import device_copy, on_device
from ..parts import Model, ModelSpec, Runtime
from ..weights import load_folder, place_all, random_tensors
from .batch import BatchBuilder, FixedShape, HostBatch, StepContext, StepEntry
from .graphs import GraphPolicy

_DTYPES = {"float32": torch.float32, "fp32": torch.float32, "bfloat16": torch.bfloat16, "bf16": torch.bfloat16}


def parse_dtype(dtype: Union[str, torch.dtype]) -> torch.dtype:
    if isinstance(dtype, torch.dtype):
        if dtype not in (torch.float32, torch.bfloat16):
            raise ValueError(f"the engine runs in float32 or bfloat16, not {dtype}")
        return dtype
    if dtype not in _DTYPES:
        raise ValueError(f"unknown dtype {dtype!r}; use float32 or bfloat16")
    return _DTYPES[dtype]


MAX_GRAPH_REQUESTS = 256
MIN_GRAPH_WIDTH = 16
DECODE_GRAPHS = 32          # captured steps of single tokens kept at a time; the one replayed longest ago goes first
MIXED_GRAPHS = 48           # and captured mixed steps, which have a budget of their own (engine/graphs.py)
GRAPH_LOGITS_BYTES = 2 << 30    # what the kept graphs' logits may hold together
MAX_GRAPH_TOKENS = 4096     # mixed steps of more tokens run eagerly: their launches no longer cost more than their kernels
MAX_GRAPH_WANTED = 256
SHAPE_SEEN_TWICE = 2        # a mixed step's shape is captured when it comes for the second time
WANTED_ROWS = (1, 2, 4, 8, 16, 32, 40, 48, 64, 128, 256)    # what the wanted rows of a mixed step are padded to


def _power_of_two(value: int, least: int = 1) -> int:
    return max(least, 1 << (max(value, 1) - 1).bit_length())


def _token_rows(tokens: int) -> int:
    """Rows a mixed step of ``tokens`` tokens is padded to: steps of 16 up to 128 (and 40), of 64 up to 1024, then
    of 256 (at most an eighth more rows than tokens from 128 on). No padded count lies on the other side of a row
    count at which a product changes its kernel (16, 40, 48, 64; ``parts.linear``) than the count itself: the
    padded step then gives the bits of the step run as it is."""
    if 32 < tokens <= 40:
        return 40
    step = 16 if tokens <= 128 else (64 if tokens <= 1024 else 256)
    return -(-tokens // step) * step


def _wanted_rows(wanted: int) -> int:
    """Rows the head's product is padded to in a mixed step; the same rule about kernels' row counts."""
    return next(rows for rows in WANTED_ROWS if rows >= max(wanted, 1))


class _DecodeGraph:
    """One captured decode step: its own metadata buffers, the graph and the logits it writes."""

    def __init__(self, engine: "Engine", width: int):
        self.builder = BatchBuilder(engine.cache, engine.device, engine.model.step_planners())
        self.width = width
        self.graph: Optional[torch.cuda.CUDAGraph] = None
        self.logits: Optional[torch.Tensor] = None
        self.held_bytes = 0         # of its logits, once captured


class _BuiltAhead:
    """The metadata of the decode step that is likely to come next, built while the GPU runs this one: the same
    requests, one more token each. What it was built from is kept, to tell whether it still holds."""

    def __init__(self, state: _DecodeGraph, ctx: StepContext, requests: List[RequestCache]):
        self.state, self.ctx, self.requests = state, ctx, requests
        self.num_tokens = [request.num_tokens for request in requests]
        self.page_counts = [[len(pages) for pages in request.pages] for request in requests]

    def holds_for(self, state: _DecodeGraph, requests: List[RequestCache]) -> bool:
        return (state is self.state and len(requests) == len(self.requests)
                and all(now is then for now, then in zip(requests, self.requests))
                and all(request.num_tokens == count for request, count in zip(requests, self.num_tokens))
                and all([len(pages) for pages in request.pages] == counts for request, counts in zip(requests, self.page_counts)))


class Engine:
    def __init__(self, spec: ModelSpec, tensors: Mapping[str, torch.Tensor], dtype: Union[str, torch.dtype] = "bfloat16",
                 device: Union[str, torch.device] = "cuda:0", page_size: int = 16,
                 max_tokens: Optional[int] = None, num_pages: Optional[int] = None, max_requests: int = 64,
                 tensors_placed: bool = False, use_graphs: bool = True, weight_copies: str = "auto",
                 consume_tensors: bool = False, tune_library: bool = False, max_portion: Optional[int] = None,
                 graph_mixed_steps: bool = True):
        """``max_portion``: the most tokens a step brings one request, if the caller keeps to one (a scheduler's
        prefill chunk): cache groups with a window then get pools no larger than their requests can fill.
        ``weight_copies``: a bfloat16 weight is kept ``"both"`` as stored (for the library's product of steps
        with many rows) and packed (for the streaming products), or ``"packed"`` only, where memory is short;
        ``"auto"`` keeps both if two copies and the cache fit the GPU's memory. With ``consume_tensors`` the
        entries of ``tensors`` (a dict) are taken out as the parts take them. ``tune_library``: the library times
        its candidates for the large products of prompts (``kernels.set_library_tuning``; global to the process)."""
        if not torch.cuda.is_available():
            raise RuntimeError("no GPU is visible; this engine has no CPU path")
        library.load()  # fail now, and loudly, if the kernels are missing and cannot be built
        self._ahead: Optional[_BuiltAhead] = None
        self._borrow = False
        self._entries: Sequence[StepEntry] = ()
        self._device_tokens: Optional[torch.Tensor] = None     # of the step that is running, if it takes tokens from there
        self.steps_built_ahead = 0      # decode steps whose metadata was ready when they came
        self._last_graph: Optional[_DecodeGraph] = None
        if tune_library and not kernels.library_tuning():
            kernels.set_library_tuning(True)
        self.dtype = parse_dtype(dtype)
        self.device = torch.device(device)
        torch.cuda.set_device(self.device)
        self.spec = spec
        self._policy = GraphPolicy(DECODE_GRAPHS, MIXED_GRAPHS, GRAPH_LOGITS_BYTES, SHAPE_SEEN_TWICE)
        if num_pages is None:
            if max_tokens is None:
                raise ValueError("give max_tokens or num_pages: the cache pool is sized once")
            num_pages = max(1, -(-max_tokens // page_size))
        if weight_copies not in ("auto", "both", "packed"):
            raise ValueError("weight_copies is 'auto', 'both' or 'packed'")
        probe = Model(spec, Runtime(dtype=self.dtype, device=self.device))
        decls = probe.tensors()
        if weight_copies == "auto":
            weight_copies = "both" if self._two_copies_fit(probe, decls, num_pages, page_size, max_requests, max_portion) else "packed"
        self.weight_copies = weight_copies
        self.runtime = Runtime(dtype=self.dtype, device=self.device, keep_plain_weights=weight_copies == "both")
        self.model = Model(spec, self.runtime)
        placed = tensors if tensors_placed else place_all(tensors, decls, self.dtype, self.device, consume=consume_tensors)
        consume = consume_tensors or not tensors_placed
        self.model.bind(placed if isinstance(placed, dict) else dict(placed), consume=consume)
        del tensors, placed
        reads = [entry.reads_cache_of for entry in spec.order]
        self.max_portion = max_portion
        self.cache = CacheManager(self.model.cache_needs(), reads, page_size, num_pages, max_requests,
                                  dtype=self.dtype, device=self.device,
                                  max_blocks=-(-spec.max_positions // page_size), max_portion=max_portion)
        self._bindings = self.cache.bindings()
        self._builder = BatchBuilder(self.cache, self.device, self.model.step_planners())
        self.steps_run = 0
        # Steps in which every request brings one token are replayed from HIP graphs, one per (number of
        # requests, block-table width): the launches of a decode step cost more host time than GPU time.
        self.use_graphs = use_graphs and all(part.graph_safe for part in self.model.parts())
        self._graphs_allowed = self.use_graphs
        # All captures share one memory pool: a graph's activations live only while it runs, so the next graph may
        # have them; what a graph hands out (its logits) stays its own while the graph is kept. How many are kept,
        # and of which kind, is the policy's business (continuous batching walks through many numbers of
        # requests): each holds its logits [rows, vocabulary] in float32 and its metadata buffers.
        self._graph_pool = None
        self.graph_replays = 0
        self.graphs_captured = 0
        # Steps that mix portions of prompts with single tokens are padded to one of a few shapes and replayed
        # from graphs too, once a shape has come twice: for small models such a step's launches cost the host
        # more time than its kernels cost the GPU.
        self.graph_mixed_steps = graph_mixed_steps
        self.mixed_graph_replays = 0

    def _two_copies_fit(self, model: Model, decls, num_pages: int, page_size: int, max_requests: int,
                        max_portion: Optional[int]) -> bool:
        """Whether the weights as stored, their packed copies and the cache pool fit the GPU with a tenth to spare."""
        if self.dtype != torch.bfloat16:
            return True     # a float32 engine has no packed copies
        weights = sum(2 * int(torch.Size(decl.shape).numel()) for decl in decls.values())
        cache = 0
        for need in model.cache_needs():
            if need is None:
                continue
            if need.paged:
                cache += pages_of_group(need, num_pages, page_size, max_requests, max_portion) * page_size * need.bytes_per_position(self.dtype)
            else:
                cache += max_requests * need.bytes_per_request(self.dtype)
        # What graphs keep: their logits up to the policy's bound, and one pool with the activations of the largest
        # captured step (a few dozen float32 rows of the stream's width per token covers every part here).
        graphs = self._policy.most_bytes + MAX_GRAPH_TOKENS * model.spec.hidden_size * 64
        total = torch.cuda.get_device_properties(self.device).total_memory
        return 2 * weights + cache + graphs <= 0.9 * total

    # ---- construction --------------------------------------------------------------------
    @classmethod
    def from_folder(cls, folder: str, dtype: Union[str, torch.dtype] = "bfloat16", device="cuda:0", **options) -> "Engine":
        """Read ``config.json``, choose the model by its architecture name, load ``model.safetensors``."""
        architecture, config = load_config(folder)
        spec = architecture.build_spec(config)
        engine_dtype = parse_dtype(dtype)
        probe = Model(spec, Runtime(dtype=engine_dtype, device=torch.device("cpu")))
        tensors = load_folder(folder, probe.tensors(), engine_dtype, torch.device(device))
        engine = cls(spec, tensors, dtype=engine_dtype, device=device, tensors_placed=True, consume_tensors=True, **options)
        engine.config = config
        return engine

    @classmethod
    def from_random(cls, config, seed: int = 0, dtype: Union[str, torch.dtype] = "bfloat16", device="cuda:0",
                    stds: Optional[Mapping[str, float]] = None, on_device: bool = False, **options) -> "Engine":
        """Random weights drawn in memory (on the GPU when ``on_device``: for sizes too large to draw on the host)."""
        architecture = architecture_named(config.architecture)
        spec = architecture.build_spec(config)
        engine_dtype = parse_dtype(dtype)
        probe = Model(spec, Runtime(dtype=engine_dtype, device=torch.device("cpu")))
        tensors = random_tensors(probe.tensors(), architecture.init_rules(config), seed, dtype=torch.bfloat16,
                                 stds=stds, device=device if on_device else "cpu")
        engine = cls(spec, tensors, dtype=engine_dtype, device=device, consume_tensors=True, **options)
        engine.config = config
        return engine

    # ---- requests ------------------------------------------------------------------------
    def open(self, request_id: Hashable) -> RequestCache:
        return self.cache.open(request_id)

    def close(self, request_id: Hashable) -> None:
        self.cache.close(request_id)

    def is_open(self, request_id: Hashable) -> bool:
        return request_id in self.cache.requests

    @property
    def kept_graphs(self) -> int:
        """Captured steps held at the moment, of both kinds."""
        return len(self._policy)

    # ---- decode steps from graphs ---------------------------------------------------------
    def _graph_step(self, requests: List[RequestCache], entries: Sequence[StepEntry]) -> Optional[torch.Tensor]:
        n = len(entries)
        widest = -(-(max(request.num_tokens for request in requests) + 1) // self.cache.page_size)
        width = max(MIN_GRAPH_WIDTH, 1 << (max(widest, 1) - 1).bit_length())
        key = (n, width)
        state = self._policy.decode.get(key)
        if state is None:
            state = _DecodeGraph(self, width)
            self._policy.decode.put(key, state)
        every_row = [[0]] * n   # the graph computes the logits of every row; the wanted ones are picked after
        ahead, self._ahead = self._ahead, None
        if ahead is not None and state.graph is not None and ahead.holds_for(state, requests):
            state.builder.fill_tokens([entry.tokens[0] for entry in entries])
            ctx = ahead.ctx
            self.steps_built_ahead += 1
        else:
            ctx = state.builder.build(requests, [entry.tokens for entry in entries], every_row, fixed_width=width)
        self._last_graph = state
        self._tokens_from_device(ctx.tokens, entries, list(range(n)))
        if state.graph is None:
            self._capture(state, ctx)
            self._policy.decode.trim(keep=key)
        state.graph.replay()
        self.graph_replays += 1
        wanted = [index for index, entry in enumerate(entries) if len(entry.want) > 0]
        if not wanted:
            return None
        if len(wanted) == n:
            return state.logits if self._borrow else device_copy(state.logits)
        return state.logits[on_device(wanted, self.device, dtype=torch.int64)]

    # ---- mixed steps from graphs -----------------------------------------------------------
    def _fixed_shape(self, batch: HostBatch) -> Optional[FixedShape]:
        """The shape a mixed step is padded to, or None if it is too large for that and runs as it is. Whether
        the padded step is then replayed from a graph or run eagerly is the policy's choice (most shapes of a
        changing workload come once); it is padded either way, so that the kernels' choices that follow the number
        of rows (which product, how a reduction is cut) are the same both times and a step gives the same bits
        whether its shape happens to be captured or not. A planner's array that is empty stays empty: the kernel it
        would feed (single tokens beside a prompt that has none) is then not launched at all."""
        step = batch.step
        wanted = int(batch.want_rows.size)
        if step.n_tokens > MAX_GRAPH_TOKENS or step.n_seqs > MAX_GRAPH_REQUESTS or wanted > MAX_GRAPH_WANTED:
            return None
        return FixedShape(tokens=_token_rows(step.n_tokens), requests=_power_of_two(step.n_seqs),
                          wanted=_wanted_rows(wanted), width=_power_of_two(batch.blocks_needed, MIN_GRAPH_WIDTH),
                          planned={name: _power_of_two(rows) if rows else 0 for name, rows in batch.planned_rows().items()})

    def _padded_step(self, shape: FixedShape, batch: HostBatch) -> Optional[torch.Tensor]:
        """The step in its fixed shape, run eagerly."""
        ctx = self._builder.upload(batch, fixed=shape)
        self._tokens_from_device(ctx.tokens, self._entries, batch.step.cu[:-1].tolist())
        logits = self.model.forward(ctx, self._bindings, ctx.want_rows)
        wanted = int(batch.want_rows.size)
        return logits[:wanted] if wanted else None

    def _tokens_from_device(self, tokens: torch.Tensor, entries: Sequence[StepEntry], places: List[int]) -> None:
        """Put the tokens that entries take from ``device_tokens`` into the step's token list on the device
        (``places[i]`` is where entry ``i``'s first token lies in it), after the host's stand-ins were copied there."""
        source = self._device_tokens
        if source is None:
            return
        taking = [(places[index], entry.token_from) for index, entry in enumerate(entries) if entry.token_from is not None]
        if not taking:
            return
        count = len(taking)
        if [place for place, _ in taking] == list(range(count)) and [row for _, row in taking] == list(range(count)):
            tokens[:count].copy_(source[:count])      # the same requests in the same order as the step before
            return
        both = on_device(np.asarray(taking, dtype=np.int64).T.copy(), self.device)
        tokens.index_copy_(0, both[0], source.index_select(0, both[1]))

    def _mixed_graph_step(self, shape: FixedShape, batch: HostBatch) -> Optional[torch.Tensor]:
        key = shape.key()
        state = self._policy.mixed.get(key)
        if state is None:
            state = _DecodeGraph(self, shape.width)
            self._policy.mixed.put(key, state, self._policy.evicted_mixed)
        ctx = state.builder.upload(batch, fixed=shape)
        self._tokens_from_device(ctx.tokens, self._entries, batch.step.cu[:-1].tolist())
        if state.graph is None:
            self._capture(state, ctx)
            self._policy.captured_mixed(key)
            self._policy.mixed.trim(self._policy.evicted_mixed, keep=key)
        state.graph.replay()
        self.graph_replays += 1
        self.mixed_graph_replays += 1
        wanted = int(batch.want_rows.size)
        if wanted == 0:
            return None
        logits = state.logits[:wanted]
        return logits if self._borrow else device_copy(logits)

    def _capture(self, state: "_DecodeGraph", ctx: StepContext) -> None:
        """Once eagerly (libraries create their handles and workspaces), then the capture. The step writes the same
        keys and values to the same slots each time, so running it again changes nothing."""
        self.model.forward(ctx, self._bindings, ctx.want_rows)
        torch.cuda.synchronize(self.device)
        ctx.memo.clear()     # what the parts computed once for the step is computed inside the graph too
        if self._graph_pool is None:
            self._graph_pool = torch.cuda.graph_pool_handle()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, pool=self._graph_pool):
            state.logits = self.model.forward(ctx, self._bindings, ctx.want_rows)
        state.graph = graph
        state.held_bytes = state.logits.numel() * state.logits.element_size() if state.logits is not None else 0
        self.graphs_captured += 1

    # ---- the step ------------------------------------------------------------------------
    def step(self, entries: Sequence[StepEntry], reserved: bool = False, borrow_logits: bool = False,
             device_tokens: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
        """Run one batch; returns float32 logits ``[wanted, vocab]`` in the order of entries and of ``want``.

        ``device_tokens`` (int32, on the device): where entries with ``token_from`` take their token from, so that
        a step can be launched before the ids that the step before chose have reached the host. Such an id is not
        checked against the vocabulary here; an id that is none (-1, from logits that were not finite) embeds as a
        row that is not finite either.

        With ``reserved`` the caller (a scheduler) has already taken the pages for every portion. The result is the
        caller's to keep. With ``borrow_logits`` it may be the buffer that a captured decode step writes, which the
        next step overwrites in place: for callers that select their tokens before they step again (the scheduler,
        the generation loop, the benchmark) and save the copy. If the model raises, the step counts for nothing:
        see ``_roll_back``.
        """
        self._borrow = borrow_logits
        entries = [entry if isinstance(entry, StepEntry) else StepEntry(*entry) for entry in entries]
        if not entries:
            return None
        requests: List[RequestCache] = []
        seen = set()
        for entry in entries:
            if entry.request_id in seen:
                raise ValueError(f"request {entry.request_id!r} appears twice in one step")
            seen.add(entry.request_id)
            request = self.cache.get(entry.request_id)
            if request.broken:
                raise ValueError(f"request {entry.request_id!r} was in a step that failed after its state may have "
                                 "changed; close it and run it again from its first token")
            count = len(entry.tokens)
            if count == 0:
                raise ValueError(f"request {entry.request_id!r} brings no tokens")
            if entry.token_from is not None:
                if count != 1 or device_tokens is None or not 0 <= entry.token_from < device_tokens.shape[0]:
                    raise ValueError(f"request {entry.request_id!r}: a token from the device is one token, a row of device_tokens")
                lowest = highest = 0
            elif count == 1:
                lowest = highest = int(entry.tokens[0])
            else:
                lowest, highest = int(min(entry.tokens)), int(max(entry.tokens))
            if lowest < 0 or highest >= self.spec.vocab_size:
                bad = next(token for token in entry.tokens if not 0 <= int(token) < self.spec.vocab_size)
                raise ValueError(f"token {bad} of request {entry.request_id!r} is outside the vocabulary")
            if self.max_portion is not None and count > self.max_portion:
                raise ValueError(f"request {entry.request_id!r} brings {count} tokens; this engine's cache was sized "
                                 f"for portions of at most {self.max_portion}")
            if request.num_tokens + count > self.spec.max_positions:
                raise ValueError(f"request {entry.request_id!r} would pass max positions {self.spec.max_positions}")
            for place in entry.want:
                if not 0 <= place < count:
                    raise ValueError(f"wanted place {place} of request {entry.request_id!r} is outside its {count} tokens")
            requests.append(request)
        if reserved:
            for request, entry in zip(requests, entries):
                if request.reserved < len(entry.tokens):
                    raise ValueError(f"request {entry.request_id!r} has no pages reserved for its portion")
        else:
            taken: List[RequestCache] = []
            try:
                for request, entry in zip(requests, entries):
                    self.cache.reserve(request, len(entry.tokens))
                    taken.append(request)
            except OutOfPages:
                for request in taken:
                    self.cache.cancel_reservation(request)
                raise
        self._device_tokens = device_tokens if any(entry.token_from is not None for entry in entries) else None
        try:
            if self.use_graphs and len(entries) <= MAX_GRAPH_REQUESTS and all(len(entry.tokens) == 1 for entry in entries):
                logits = self._graph_step(requests, entries)
            else:
                self._last_graph = None
                self._entries = entries
                batch = self._builder.prepare(requests, [entry.tokens for entry in entries], [entry.want for entry in entries])
                shape = self._fixed_shape(batch) if self.use_graphs and self.graph_mixed_steps else None
                if shape is not None and self._policy.wants_mixed(shape.key()):
                    logits = self._mixed_graph_step(shape, batch)
                elif shape is not None:
                    logits = self._padded_step(shape, batch)
                else:
                    ctx = self._builder.upload(batch)
                    self._tokens_from_device(ctx.tokens, entries, batch.step.cu[:-1].tolist())
                    logits = self.model.forward(ctx, self._bindings, ctx.want_rows)
        except BaseException:
            self._roll_back(requests)
            raise
        for request, entry in zip(requests, entries):
            self.cache.commit(request, len(entry.tokens))
        self.steps_run += 1
        if self._last_graph is not None:
            self._build_ahead(self._last_graph, requests)
        return logits

    def observe_layers(self, observer) -> None:
        """Call ``observer(run entry, stream)`` after every run entry of every step from now on, ``stream`` being
        the float32 residual stream ``[tokens, hidden]`` with that entry's result added (a fresh tensor); None
        switches it off. Steps run eagerly meanwhile: a graph's replay calls nothing on the host."""
        if observer is None:
            self.model.observer = None
            self.use_graphs = self._graphs_allowed
            return

        def after_entry(index, h, pending):
            stream = h.clone()
            if isinstance(pending, torch.Tensor):   # else the entry's last product added its result itself
                for part in (pending if pending.dim() == 3 else pending.unsqueeze(0)):
                    stream += part.to(torch.float32)
            observer(index, stream)

        self.model.observer = after_entry
        self.use_graphs = False

    def _roll_back(self, requests: List[RequestCache]) -> None:
        """A step failed inside the model (a kernel refused its arguments, a part raised): nothing of it counts.

        Every request of the step gives back the pages that only this step needed, whoever reserved them, and
        keeps the positions it had; keys and values that the step wrote beyond them are never read, since
        lengths, not contents, say what is valid. Per-request state has no such rule: a part may have changed it
        before the failure, so with state in the model the step's requests are marked broken and refused from
        then on; whoever runs them closes them and runs them again from their first token (the scheduler does).
        The reference resets the cache on any failure of a forward (src/model/model.cpp:1131-1134)."""
        self._ahead = None
        self._last_graph = None
        for request in requests:
            if request.closed:
                continue
            self.cache.cancel_reservation(request)
            if self.cache.has_state:
                request.broken = True

    def _build_ahead(self, state: _DecodeGraph, requests: List[RequestCache]) -> None:
        """After a decode step from a graph: the next one's metadata (positions, slots, block tables), while the
        GPU is busy with this one. Only where every request has room for one more position in the pages it holds
        and the block tables keep their width; the tokens are filled in when the step comes."""
        self._last_graph = None
        if state.graph is None or any(need for request in requests for need in self.cache.pages_needed(request, 1)):
            return
        widest = -(-(max(request.num_tokens for request in requests) + 1) // self.cache.page_size)
        if max(MIN_GRAPH_WIDTH, 1 << (max(widest, 1) - 1).bit_length()) != state.width:
            return
        count = len(requests)
        ctx = state.builder.build(requests, [[0]] * count, [[0]] * count, fixed_width=state.width)
        self._ahead = _BuiltAhead(state, ctx, list(requests))
