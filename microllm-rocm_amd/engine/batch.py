"""The batch of one step: a flat list of tokens with, for every request in it, where its portion starts.

A step holds portions of prompts beside single decoded tokens. Everything a
kernel needs to find a token's request, position and pages is packed into one
int32 buffer on the host and copied to the device in one transfer (the reference
packs tokens, positions and rows the same way, src/model/model.cpp:1522-1538).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from types import SimpleNamespace
from typing import Any, Dict, Hashable, List, Mapping, Optional, Sequence, Tuple

import numpy as np
import torch

from ..cache.manager import CacheManager, RELEASED, RequestCache
from ..ops.transfers import copy_to_device, on_device


@dataclass
class StepEntry:
    """One request's next tokens and the places among them whose logits are wanted.

    ``token_from``: the entry's one token is not known on the host yet; it is row ``token_from`` of the
    ``device_tokens`` that the step is given (ids chosen on the device by the step before), and ``tokens`` holds a
    stand-in."""
    request_id: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = ()
    token_from: Optional[int] = None


@dataclass
class PagedView:
    """One cache group as the step sees it."""
    block_table: torch.Tensor   # int32 [requests, width]; RELEASED where a window has passed
    slot_mapping: torch.Tensor  # int32 [tokens]: page * page_size + offset of every token's key and value
    page_size: int
    width: int


@dataclass
class HostStep:
    """A step as the host sees it: what a part that plans its launches from the batch's shape (tiles of queries,
    work lists) is given. ``cu[i]`` is where request ``i``'s portion starts in the flat token list, ``starts[i]``
    the position of its first token, ``totals[i]`` the request's length once the step is done."""
    n_tokens: int
    n_seqs: int
    page_size: int
    counts: List[int]
    starts: List[int]
    totals: List[int]
    cu: np.ndarray

    @property
    def single_tokens_only(self) -> bool:
        return self.n_tokens == self.n_seqs


PADDING = -1     # request of a token, or slot of its key and value, where the row only pads a step to a fixed shape


@dataclass
class HostBatch:
    """A step prepared on the host (``BatchBuilder.prepare``): its arrays and its planners' plans, not yet copied."""
    step: HostStep
    tokens: np.ndarray
    positions: np.ndarray
    seq_of_token: np.ndarray
    starts_array: np.ndarray
    totals_array: np.ndarray
    slots: np.ndarray
    want_rows: np.ndarray
    blocks_needed: int
    plans: list          # (planner, arrays, values)

    def planned_rows(self) -> Dict[Tuple[Hashable, str], int]:
        return {(planner.key, name): int(array.shape[0]) for planner, arrays, _ in self.plans for name, array in arrays.items()}


@dataclass(frozen=True)
class FixedShape:
    """The shape a step is padded to so that it can be replayed from a graph: rows of tokens, of requests and of
    wanted logits, the block tables' width and the rows of every planner's arrays. Padding rows hold token 0 at
    position 0 of request ``PADDING`` with slot ``PADDING`` (nothing is stored for them and attention passes them
    over); padding requests hold no tokens; a planner pads its arrays with the values it names in ``padding``."""
    tokens: int
    requests: int
    wanted: int
    width: int
    planned: Mapping[Tuple[Hashable, str], int]

    def key(self) -> tuple:
        return (self.tokens, self.requests, self.wanted, self.width, tuple(sorted(self.planned.items(), key=repr)))


class StepPlanner:
    """What a part gives the engine if its kernels need metadata of their own for a step.

    ``plan(host)`` returns ``(arrays, values)``: int32 numpy arrays that go to the device with the step's other
    metadata, in the same single copy, and host values (numbers that choose launches). Parts whose planners have
    equal ``key`` share one plan a step. For a step in which every request brings one token the arrays' sizes may
    depend on the number of requests alone (such steps are replayed from graphs at fixed addresses)."""
    key: Hashable = None
    padding: Dict[str, int] = {}      # array name -> the value of rows that pad it to a fixed number of rows

    def plan(self, host: HostStep) -> Tuple[Dict[str, np.ndarray], Dict[str, Any]]:
        raise NotImplementedError


@dataclass
class StepContext:
    n_tokens: int
    n_seqs: int
    tokens: torch.Tensor        # int32 [tokens]
    positions: torch.Tensor     # int32 [tokens]: absolute position of every token in its request
    seq_of_token: torch.Tensor  # int32 [tokens]: index into this step's requests
    cu_tokens: torch.Tensor     # int32 [requests + 1]: where each request's portion starts in the flat list
    seq_start: torch.Tensor     # int32 [requests]: position of the portion's first token
    seq_total: torch.Tensor     # int32 [requests]: positions in the cache once this step is done
    slots: torch.Tensor         # int32 [requests]: state slot of every request
    want_rows: Optional[torch.Tensor]  # int32 [wanted]: rows of the flat list whose logits are wanted
    paged: List[PagedView]
    # the same on the host, for parts written in Python and for choosing kernels
    starts: List[int] = field(default_factory=list)
    counts: List[int] = field(default_factory=list)
    host_slots: List[int] = field(default_factory=list)
    max_count: int = 0
    max_total: int = 0
    planned_total: int = 0      # the longest request this step's launch shapes are planned for (>= max_total)
    host: Optional[HostStep] = None
    fixed: bool = False         # the step was padded to a fixed shape: n_tokens and n_seqs count the padding too
    # the plans of the parts' planners (key: the planner's): device arrays and host values as attributes
    planned: Dict[Hashable, SimpleNamespace] = field(default_factory=dict)
    # what a part computes once for the step and its likes in other layers take from here (key: the part's choice)
    memo: dict = field(default_factory=dict)

    def plan_of(self, planner: StepPlanner) -> SimpleNamespace:
        """The plan of ``planner`` for this step: made with the step if the engine knew the planner (the model's
        parts name theirs), else made now, with a copy of its own to the device (a part run outside an engine)."""
        plan = self.planned.get(planner.key)
        if plan is None:
            arrays, values = planner.plan(self.host)
            device = self.tokens.device
            plan = SimpleNamespace(**values, **{name: on_device(np.ascontiguousarray(array, dtype=np.int32), device)
                                                for name, array in arrays.items()})
            self.planned[planner.key] = plan
        return plan


class BatchBuilder:
    """Packs a step's metadata and moves it to the device through one pinned staging buffer.

    With ``fixed_width`` every block table is padded to that many columns, so that the layout of the packed
    buffer depends on the numbers of tokens and requests alone: a step that is replayed from a HIP graph
    finds every array at the address it had when the graph was captured.
    """

    def __init__(self, cache: CacheManager, device: torch.device, planners: Sequence[StepPlanner] = ()):
        self.cache = cache
        self.device = device
        self.planners: List[StepPlanner] = []
        for planner in planners:       # one plan a key
            if all(planner.key != known.key for known in self.planners):
                self.planners.append(planner)
        self._staging: Optional[torch.Tensor] = None
        self._device_buffer: Optional[torch.Tensor] = None
        self._copied = None

    def _buffers(self, size: int):
        if self._staging is None or self._staging.numel() < size:
            capacity = max(4096, 1 << (size - 1).bit_length())
            self._staging = torch.empty(capacity, dtype=torch.int32, pin_memory=True)
            self._device_buffer = torch.empty(capacity, dtype=torch.int32, device=self.device)
            self._copied = None
        if self._copied is not None:
            self._copied.synchronize()  # the last step's copy has left the staging buffer
        return self._staging, self._device_buffer

    def fill_tokens(self, tokens: Sequence[int]) -> None:
        """Put the tokens of a step of single tokens into the buffers that ``build`` filled for it ahead of time
        (with any tokens): they lie first in the packed buffer."""
        count = len(tokens)
        if self._copied is not None:
            self._copied.synchronize()
        self._staging.numpy()[:count] = tokens
        copy_to_device(self._device_buffer[:count], self._staging[:count], non_blocking=True)
        self._copied = torch.cuda.Event()
        self._copied.record()

    def build(self, requests: Sequence[RequestCache], token_lists: Sequence[Sequence[int]],
              wants: Sequence[Sequence[int]], fixed_width: Optional[int] = None) -> StepContext:
        """The step's metadata on the device; with ``fixed_width`` every block table has that many columns."""
        return self.upload(self.prepare(requests, token_lists, wants), fixed_width=fixed_width)

    def prepare(self, requests: Sequence[RequestCache], token_lists: Sequence[Sequence[int]],
                wants: Sequence[Sequence[int]]) -> "HostBatch":
        """Everything about the step that is worked out on the host, the planners' plans included; nothing is
        copied yet. Whoever wants the step in a fixed shape reads the sizes here, chooses the shape (``FixedShape``)
        and hands both to ``upload``, of this builder or of another that knows the same planners."""
        page_size = self.cache.page_size
        n_seqs = len(requests)
        counts = [len(tokens) for tokens in token_lists]
        n_tokens = sum(counts)
        slots = np.fromiter((request.slot for request in requests), dtype=np.int32, count=n_seqs)
        starts_array = np.fromiter((request.num_tokens for request in requests), dtype=np.int32, count=n_seqs)
        starts = starts_array.tolist()
        if n_tokens == n_seqs:      # every request brings one token: nothing to concatenate
            counts_array = np.ones(n_seqs, dtype=np.int32)
            tokens = np.fromiter((tokens[0] for tokens in token_lists), dtype=np.int32, count=n_seqs)
            positions = starts_array
            seq_of_token = np.arange(n_seqs, dtype=np.int32)
        else:
            counts_array = np.asarray(counts, dtype=np.int32)
            tokens = np.concatenate([np.asarray(t, dtype=np.int32) for t in token_lists]) if n_tokens else np.zeros(0, np.int32)
            positions = np.concatenate([np.arange(s, s + c, dtype=np.int32) for s, c in zip(starts, counts)]) \
                if n_tokens else np.zeros(0, np.int32)
            seq_of_token = np.repeat(np.arange(n_seqs, dtype=np.int32), counts)
        totals_array = starts_array + counts_array
        totals = totals_array.tolist()
        cu = np.zeros(n_seqs + 1, dtype=np.int32)
        np.cumsum(counts_array, out=cu[1:])
        if all(len(want) == 1 and want[0] == 0 for want in wants) and n_tokens == n_seqs:
            want_rows = np.arange(n_seqs, dtype=np.int32)
        else:
            want_rows = np.asarray([cu[index] + place for index, want in enumerate(wants) for place in want],
                                   dtype=np.int32)
        blocks_needed = int((int(totals_array.max()) + page_size - 1) // page_size) if n_seqs else 1
        host_step = HostStep(n_tokens=n_tokens, n_seqs=n_seqs, page_size=page_size, counts=counts, starts=starts,
                             totals=totals, cu=cu)
        plans = [(planner, *planner.plan(host_step)) for planner in self.planners]
        return HostBatch(host_step, tokens, positions, seq_of_token, starts_array, totals_array, slots, want_rows,
                         max(1, blocks_needed), plans)

    def upload(self, batch: "HostBatch", fixed_width: Optional[int] = None,
               fixed: Optional["FixedShape"] = None) -> StepContext:
        """Pack the prepared step into the staging buffer and copy it to the device. With ``fixed`` every array is
        padded to that shape (see ``FixedShape``), so that the packed buffer's layout depends on the shape alone."""
        step = batch.step
        page_size, n_seqs, n_tokens = step.page_size, step.n_seqs, step.n_tokens
        if fixed is not None:
            fixed_width = fixed.width
            if n_tokens > fixed.tokens or n_seqs > fixed.requests or batch.want_rows.size > fixed.wanted:
                raise ValueError("the step is larger than the fixed shape")
        rows_tokens = fixed.tokens if fixed is not None else n_tokens
        rows_seqs = fixed.requests if fixed is not None else n_seqs

        def padded(array: np.ndarray, rows: int, fill: int) -> np.ndarray:
            if array.shape[0] == rows:
                return array
            out = np.full((rows,) + array.shape[1:], fill, dtype=np.int32)
            out[:array.shape[0]] = array
            return out

        tokens = padded(batch.tokens, rows_tokens, 0)
        positions = padded(batch.positions, rows_tokens, 0)
        seq_of_token = padded(batch.seq_of_token, rows_tokens, PADDING)
        cu = padded(step.cu, rows_seqs + 1, n_tokens)
        starts_array = padded(batch.starts_array, rows_seqs, 0)
        totals_array = padded(batch.totals_array, rows_seqs, 0)
        slots = padded(batch.slots, rows_seqs, 0)
        want_rows = padded(batch.want_rows, fixed.wanted, 0) if fixed is not None else batch.want_rows
        tables, mappings, widths = [], [], []
        for group in self.cache.groups:
            width = batch.blocks_needed
            if fixed_width is not None:
                if width > fixed_width:
                    raise ValueError("a block table is wider than the fixed width")
                width = fixed_width
            rows = group.tables[batch.slots]                      # [requests, most blocks a request can hold]
            if width <= rows.shape[1]:
                table = np.ascontiguousarray(rows[:, :width])
            else:
                table = np.full((n_seqs, width), RELEASED, dtype=np.int32)
                table[:, :rows.shape[1]] = rows
            mapping = table[batch.seq_of_token, batch.positions // page_size] * page_size + batch.positions % page_size
            tables.append(padded(table, rows_seqs, RELEASED))
            mappings.append(padded(mapping.astype(np.int32, copy=False), rows_tokens, PADDING))
            widths.append(width)
        pieces = [tokens, positions, seq_of_token, cu, starts_array, totals_array, slots, want_rows]
        for table, mapping in zip(tables, mappings):
            pieces += [table.reshape(-1), mapping]
        plans = []          # (key, host values, {name: (piece index, shape)})
        for planner, arrays, values in batch.plans:
            places = {}
            for name, array in arrays.items():
                array = np.ascontiguousarray(array, dtype=np.int32)
                if fixed is not None:
                    array = padded(array, fixed.planned[(planner.key, name)], planner.padding[name])
                places[name] = (len(pieces), array.shape)
                pieces.append(array.reshape(-1))
            plans.append((planner.key, values, places))
        offsets, cursor = [], 0
        for piece in pieces:
            offsets.append(cursor)
            cursor += (piece.size + 3) // 4 * 4  # keep every piece 16-byte aligned
        staging, device_buffer = self._buffers(max(cursor, 1))
        host = staging.numpy()
        for offset, piece in zip(offsets, pieces):
            host[offset:offset + piece.size] = piece
        copy_to_device(device_buffer[:cursor], staging[:cursor], non_blocking=True)
        self._copied = torch.cuda.Event()
        self._copied.record()

        def piece_at(index: int, shape=None) -> torch.Tensor:
            view = device_buffer[offsets[index]:offsets[index] + pieces[index].size]
            return view if shape is None else view.view(shape)

        paged = []
        for g, group in enumerate(self.cache.groups):
            paged.append(PagedView(piece_at(8 + 2 * g, (rows_seqs, widths[g])), piece_at(9 + 2 * g),
                                   page_size, widths[g]))
        planned = {key: SimpleNamespace(**values, **{name: piece_at(index, shape) for name, (index, shape) in places.items()})
                   for key, values, places in plans}
        longest = max(step.totals) if step.totals else 0
        return StepContext(
            n_tokens=rows_tokens, n_seqs=rows_seqs, tokens=piece_at(0), positions=piece_at(1), seq_of_token=piece_at(2),
            cu_tokens=piece_at(3), seq_start=piece_at(4), seq_total=piece_at(5), slots=piece_at(6),
            want_rows=piece_at(7) if want_rows.size else None, paged=paged,
            starts=step.starts, counts=step.counts, host_slots=batch.slots.tolist(),
            max_count=max(step.counts) if step.counts else 0, max_total=longest,
            planned_total=longest if fixed_width is None else fixed_width * page_size, host=step, planned=planned,
            fixed=fixed is not None)
