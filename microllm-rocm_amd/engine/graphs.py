"""Which captured steps are kept: host logic only, no GPU call.

Steps of single tokens (decoding) carry most of a serving run's time and have few shapes (requests x block-table
width); steps that mix portions with single tokens have many (token rows x requests x wanted x width x the
planners' rows) and most come once. The two kinds therefore have budgets of their own, so that no run of mixed
shapes pushes the decode graphs out, and both are bounded in bytes as well: a kept graph holds its float32
logits ``[rows, vocabulary]``. A mixed shape is captured when it has come ``seen_before_capture`` times; one
that was evicted has to come that often again, and one that was evicted after having been captured
``MAX_CAPTURES_A_SHAPE`` times runs eagerly from then on: a workload that cycles through more shapes than the
budget holds would otherwise pay an eager run, a capture and a replay every time a shape comes back.
"""
from __future__ import annotations

from collections import OrderedDict
from typing import Callable, Dict, Hashable, Optional

MAX_CAPTURES_A_SHAPE = 2


class KeptGraphs:
    """An LRU of captured steps with a budget in entries and in bytes (``state.held_bytes``, 0 until captured)."""

    def __init__(self, most: int, most_bytes: int):
        self.most, self.most_bytes = most, most_bytes
        self.entries: "OrderedDict[Hashable, object]" = OrderedDict()
        self.evicted = 0

    def __len__(self) -> int:
        return len(self.entries)

    def __contains__(self, key: Hashable) -> bool:
        return key in self.entries

    def held_bytes(self) -> int:
        return sum(getattr(state, "held_bytes", 0) for state in self.entries.values())

    def get(self, key: Hashable):
        state = self.entries.get(key)
        if state is not None:
            self.entries.move_to_end(key)
        return state

    def put(self, key: Hashable, state, on_evict: Optional[Callable[[Hashable], None]] = None) -> None:
        self.entries[key] = state
        self.entries.move_to_end(key)
        self.trim(on_evict, keep=key)

    def trim(self, on_evict: Optional[Callable[[Hashable], None]] = None, keep: Hashable = None) -> None:
        """Drop the entries replayed longest ago until both budgets hold; ``keep`` (the one in use) stays."""
        while len(self.entries) > 1 and (len(self.entries) > self.most or self.held_bytes() > self.most_bytes):
            oldest = next(iter(self.entries))
            if oldest == keep:
                self.entries.move_to_end(oldest)
                oldest = next(iter(self.entries))
            del self.entries[oldest]
            self.evicted += 1
            if on_evict is not None:
                on_evict(oldest)


class GraphPolicy:
    """The engine's two sets of kept graphs and the rule for capturing a mixed step's shape."""

    def __init__(self, decode_graphs: int = 32, mixed_graphs: int = 16, most_bytes: int = 2 << 30,
                 seen_before_capture: int = 2):
        self.decode = KeptGraphs(decode_graphs, most_bytes // 2)
        self.mixed = KeptGraphs(mixed_graphs, most_bytes // 2)
        self.seen_before_capture = seen_before_capture
        self._seen: Dict[Hashable, int] = {}
        self._captures: Dict[Hashable, int] = {}

    @property
    def most_bytes(self) -> int:
        return self.decode.most_bytes + self.mixed.most_bytes

    def __len__(self) -> int:
        return len(self.decode) + len(self.mixed)

    def wants_mixed(self, key: Hashable) -> bool:
        """Whether a mixed step of this shape is replayed from a graph (captured now if need be) or runs eagerly."""
        if key in self.mixed:
            return True
        if self._captures.get(key, 0) >= MAX_CAPTURES_A_SHAPE:
            return False                     # it was captured and pushed out before: eagerly for good
        if len(self._seen) > 4096:
            self._seen.clear()
        seen = self._seen[key] = self._seen.get(key, 0) + 1
        return seen >= self.seen_before_capture

    def captured_mixed(self, key: Hashable) -> None:
        self._captures[key] = self._captures.get(key, 0) + 1

    def evicted_mixed(self, key: Hashable) -> None:
        self._seen.pop(key, None)            # it has to come twice again before it is captured again
