"""The model a ``ModelSpec`` describes: embedding, layers run in the spec's order, final norm, head.

Nothing here names an architecture. The run order is data: an entry names a
layer (perhaps one that an earlier entry named too) and either owns a cache or
reads an earlier entry's. Logits are computed in float32 for the wanted rows only
(the reference projects the last row only, src/model/model.cpp:1118-1128).
"""
from __future__ import annotations

from typing import Dict, List, Mapping, Optional

import torch

from ..ops import kernels
from .base import CacheNeed, MATRIX, Part, Runtime, TensorDecl
from .block import Block, build_block
from .linear import Weight, linear
from .registry import build_part, register_part
from .spec import ModelSpec, PartSpec


class TokenEmbedding(Part):
    """``h0[t] = E[id_t]`` widened to float32 (src/model/model.cpp:1111). An embedding part is handed the whole
    step, so that one which also needs positions or requests (learned positions, token types) finds them."""
    category = "embedding"
    graph_safe = True

    def __init__(self, spec: PartSpec, runtime: Runtime):
        super().__init__(spec, runtime)
        self.vocab = int(spec.params["vocab_size"])
        self.width = int(spec.params["hidden_size"])
        self.table: Optional[torch.Tensor] = None

    def tensors(self):
        return {self.name("weight"): TensorDecl((self.vocab, self.width), MATRIX)}

    def bind(self, tensors):
        self.table = tensors[self.name("weight")]

    def forward(self, ctx) -> torch.Tensor:
        return kernels.embedding(self.table, ctx.tokens)

    def bytes_read(self, rows: int, context: int) -> int:
        return rows * self.width * self.table.element_size()     # a row per token, not the table


class LMHead(Part):
    """``logits = x W^T`` in float32; a tied head names the embedding's table as its weight
    (src/model/model.cpp:1121-1128)."""
    category = "head"
    graph_safe = True

    def __init__(self, spec: PartSpec, runtime: Runtime):
        super().__init__(spec, runtime)
        self.vocab = int(spec.params["vocab_size"])
        self.width = int(spec.params["hidden_size"])
        self.weight: Optional[torch.Tensor] = None

    def tensors(self):
        return {self.name("weight"): TensorDecl((self.vocab, self.width), MATRIX)}

    def bind(self, tensors):
        self.weight = Weight(tensors[self.name("weight")], keep_plain=self.runtime.keep_plain_weights)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return linear(x, self.weight, out_dtype=torch.float32)

    def flops(self, tokens: int, wanted: int = 1) -> float:
        return 2.0 * self.vocab * self.width * wanted     # logits at the wanted rows only


register_part("embedding", "token_embedding", TokenEmbedding)
register_part("head", "lm_head", LMHead)


class _HandOver:
    """A mapping that lets go of an entry when it has been looked up as often as parts declared it."""

    def __init__(self, tensors: dict, declarations):
        self._tensors = tensors
        self._uses: Dict[str, int] = {}
        for declared in declarations:
            for name in declared:
                self._uses[name] = self._uses.get(name, 0) + 1

    def __getitem__(self, name: str) -> torch.Tensor:
        self._uses[name] = self._uses.get(name, 1) - 1
        return self._tensors.pop(name) if self._uses[name] <= 0 else self._tensors[name]

    def __contains__(self, name: str) -> bool:
        return name in self._tensors


class Model:
    def __init__(self, spec: ModelSpec, runtime: Runtime):
        spec.validate()
        self.spec = spec
        self.runtime = runtime
        self.embedding = build_part("embedding", spec.embedding, runtime)
        self.blocks: List[Block] = [build_block(layer, runtime) for layer in spec.layers]
        self.final_norm = build_part("norm", spec.final_norm, runtime)
        self.head = build_part("head", spec.head, runtime)
        # Called as observer(run entry, h, pending) after every entry of a step when set (the replay tool's dump of
        # the stream layer by layer; the reference traces tensors by name, include/microllm/profiling/trace.h:63).
        self.observer = None

    # ---- tensors -------------------------------------------------------------------------
    def tensors(self) -> Dict[str, TensorDecl]:
        decls: Dict[str, TensorDecl] = {}

        def add(new: Mapping[str, TensorDecl]) -> None:
            for name, decl in new.items():
                if name in decls and decls[name] != decl:
                    raise ValueError(f"tensor {name!r} is declared twice with different shapes or kinds")
                decls[name] = decl

        add(self.embedding.tensors())
        for block in self.blocks:
            add(block.tensors())
        add(self.final_norm.tensors())
        add(self.head.tensors())
        return decls

    def bind(self, tensors: Mapping[str, torch.Tensor], consume: bool = False) -> None:
        """Hand every part its tensors. With ``consume`` (``tensors`` must be a dict) an entry is taken out of
        ``tensors`` when the last part that declared it has looked it up, so that what a part does not keep
        (a weight it only needed to pack or stack) is freed at once, not when loading ends."""
        if consume:
            tensors = _HandOver(tensors, [part.tensors() for part in self.parts()])
        self.embedding.bind(tensors)
        for block in self.blocks:
            block.bind(tensors)
        self.final_norm.bind(tensors)
        self.head.bind(tensors)

    def parts(self) -> List[Part]:
        """Every part the model runs, the parts' own sub-parts included."""
        found: List[Part] = []

        def add(part: Part) -> None:
            found.append(part)
            for inner in part.sub_parts():
                add(inner)

        for part in (self.embedding, self.final_norm, self.head):
            add(part)
        for block in self.blocks:
            for part in block.parts():
                add(part)
        return found

    def step_planners(self) -> list:
        """The planners of the parts that want step metadata of their own, one per key."""
        planners = []
        for part in self.parts():
            planner = part.step_planner()
            if planner is not None and all(planner.key != known.key for known in planners):
                planners.append(planner)
        return planners

    def cache_needs(self) -> List[Optional[CacheNeed]]:
        """The cache need of every run entry; None for an entry that owns none."""
        needs: List[Optional[CacheNeed]] = []
        for entry in self.spec.order:
            need = self.blocks[entry.layer].mixer.cache_need()
            needs.append(None if entry.reads_cache_of is not None else need)
        return needs

    # ---- forward -------------------------------------------------------------------------
    def forward(self, ctx, caches, want_rows: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
        """Run the step's tokens through every entry; logits ``[wanted, vocab]`` in float32.

        ``caches[i]`` is the cache binding of run entry ``i`` (its own, or the one it reads).
        ``want_rows`` indexes the step's flat token list; None or empty skips the head.
        """
        h = self.embedding.forward(ctx)
        pending = None
        order = self.spec.order
        for index, entry in enumerate(order):
            next_block = self.blocks[order[index + 1].layer] if index + 1 < len(order) else None
            pending = self.blocks[entry.layer].forward(h, pending, ctx, caches[index], next_block)
            if self.observer is not None:
                self.observer(index, h, pending)
        if want_rows is None or want_rows.numel() == 0:
            return None
        x = self.final_norm.forward(h, delta=pending, write_h=False, rows=want_rows)
        return self.head.forward(x)
