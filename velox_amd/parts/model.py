"""A decoder described as data, and the object built from that description.

``ModelSpec`` is what an architecture produces from its configuration: one
``LayerSpec`` per weight-owning layer (each naming its own mixer, feed-forward and
norm kinds with their constants), shared position encodings, and ``schedule``, the
order in which layers run.  The schedule is a list of ``ScheduleEntry``: an entry may
name a layer that an earlier entry already named (the layer's weights run twice, each
run with a cache of its own), or set ``cache_from`` to an earlier entry to read that
entry's cache instead of owning one.

``DecoderModel`` runs the whole thing the way the reference's ``QwenDecoderModel``
does (``src/transformer.py:43-52``): embed, blocks in schedule order, final norm; the
output head is a separate call on chosen rows (``src/transformer.py:67-68``).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple

import torch

from . import block as _block  # noqa: F401  (registers the built-in arrangement)
from .base import Embedding, OutputHead, Param, Part, PartSpec, make_part, register_part, single


@dataclass(frozen=True)
class LayerSpec:
    prefix: str
    mixer: PartSpec
    feed_forward: PartSpec
    mixer_norm: PartSpec
    ff_norm: PartSpec
    position: Optional[str] = None  # key into ModelSpec.positions handed to the mixer
    arrangement: str = "pre_norm"
    # where each part's tensors stand in the checkpoint, below the layer's prefix (an architecture sets its own names)
    mixer_prefix: str = "mixer."
    feed_forward_prefix: str = "feed_forward."
    mixer_norm_prefix: str = "mixer_norm."
    ff_norm_prefix: str = "feed_forward_norm."


@dataclass(frozen=True)
class ScheduleEntry:
    layer: int
    cache_from: Optional[int] = None


@dataclass
class ModelSpec:
    vocab_size: int
    hidden_size: int
    max_position: int
    layers: List[LayerSpec]
    schedule: List[ScheduleEntry]
    final_norm: PartSpec
    positions: Dict[str, PartSpec] = field(default_factory=dict)
    embedding_position: Optional[str] = None  # a position encoding applied to the embeddings
    tie_head: bool = False
    embed_name: str = "embedding.weight"
    head_name: str = "head.weight"
    final_norm_prefix: str = "final_norm."
    eos_token_ids: Tuple[int, ...] = ()
    # The parts at the two ends, chosen like every other part.  None = the plain ones: a table that is looked up
    # (``embed_name``) and a product without bias (``head_name``, or the table itself with ``tie_head``).  A kind
    # registered under "embedding" / "head" gets its ``args`` plus ``name``, ``vocab_size``, ``hidden_size`` and, for a
    # head, ``tied_to`` (the table's checkpoint name or None).
    embedding: Optional[PartSpec] = None
    head: Optional[PartSpec] = None

    def validate(self) -> None:
        if not self.layers:
            raise ValueError("a model needs at least one layer")
        for index, entry in enumerate(self.schedule):
            if not 0 <= entry.layer < len(self.layers):
                raise ValueError(f"schedule[{index}] names layer {entry.layer}, but there are {len(self.layers)}")
            if entry.cache_from is not None:
                if not 0 <= entry.cache_from < index:
                    raise ValueError(f"schedule[{index}].cache_from must name an earlier entry")
                if self.schedule[entry.cache_from].cache_from is not None:
                    raise ValueError(f"schedule[{index}].cache_from must name an entry that owns its cache")


class TableEmbedding(Embedding):
    """``h[t] = E[ids[t]]``, no scaling (reference ``src/transformer.py:27,44``)."""

    def __init__(self, name: str, vocab_size: int, hidden_size: int) -> None:
        super().__init__("")
        self.name = name
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size
        self.table: Optional[torch.Tensor] = None

    def params(self) -> Dict[str, Param]:
        return {"table": single(self.name, (self.vocab_size, self.hidden_size), product=False)}

    def forward(self, token_ids: torch.Tensor, ctx) -> torch.Tensor:
        return ctx.ops.embed(token_ids, self.table)


class LinearHead(OutputHead):
    """``logits = hidden @ W^T`` without bias; ``W`` is the embedding table when tied
    (reference ``src/transformer.py:60-62``).  Logits are returned in float32."""

    def __init__(self, name: str, vocab_size: int, hidden_size: int, tied_to: Optional[str] = None) -> None:
        super().__init__("")
        self.name = name
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size
        self.tied_to = tied_to
        self.weight: Optional[torch.Tensor] = None

    def params(self) -> Dict[str, Param]:
        base = single(self.name, (self.vocab_size, self.hidden_size))
        if self.tied_to is None:
            return {"weight": base}
        return {"weight": Param(base.shape, base.sources, base.source_shapes, base.role, base.init, alias_of=self.tied_to)}

    def prepare_kernels(self, ops) -> None:
        self.prepare_weight(ops, "weight")

    def forward(self, hidden_rows: torch.Tensor, ctx) -> torch.Tensor:
        return ctx.ops.linear(hidden_rows, self.operand("weight"), None, torch.float32)


register_part("embedding", "table", TableEmbedding)
register_part("head", "linear", LinearHead)


class DecoderModel(Part):
    def __init__(self, spec: ModelSpec) -> None:
        super().__init__("")
        spec.validate()
        self.spec = spec
        self.positions = {key: make_part("position", ps.kind, **ps.kwargs()) for key, ps in spec.positions.items()}
        embedding = spec.embedding or PartSpec.of("table")
        self.embedding = make_part("embedding", embedding.kind, name=spec.embed_name, vocab_size=spec.vocab_size, hidden_size=spec.hidden_size, **embedding.kwargs())
        self.blocks = []
        for layer in spec.layers:
            mixer_kwargs = layer.mixer.kwargs()
            if layer.position is not None:
                mixer_kwargs["position"] = self.positions[layer.position]
            mixer = make_part("mixer", layer.mixer.kind, prefix=layer.prefix + layer.mixer_prefix, **mixer_kwargs)
            ff = make_part("feed_forward", layer.feed_forward.kind, prefix=layer.prefix + layer.feed_forward_prefix, **layer.feed_forward.kwargs())
            norm1 = make_part("norm", layer.mixer_norm.kind, prefix=layer.prefix + layer.mixer_norm_prefix, **layer.mixer_norm.kwargs())
            norm2 = make_part("norm", layer.ff_norm.kind, prefix=layer.prefix + layer.ff_norm_prefix, **layer.ff_norm.kwargs())
            self.blocks.append(make_part("arrangement", layer.arrangement, prefix=layer.prefix, mixer=mixer, feed_forward=ff, mixer_norm=norm1, ff_norm=norm2))
        self.final_norm = make_part("norm", spec.final_norm.kind, prefix=spec.final_norm_prefix, **spec.final_norm.kwargs())
        head = spec.head or PartSpec.of("linear")
        self.head = make_part("head", head.kind, name=spec.head_name, vocab_size=spec.vocab_size, hidden_size=spec.hidden_size,
                              tied_to=spec.embed_name if spec.tie_head else None, **head.kwargs())
        self.schedule = list(spec.schedule)

    # -- structure ----------------------------------------------------------------------
    def children(self) -> Tuple[Part, ...]:
        return (self.embedding, *self.positions.values(), *self.blocks, self.final_norm, self.head)

    def all_parts(self) -> List[Part]:
        out: List[Part] = []

        def walk(part: Part) -> None:
            out.append(part)
            for child in part.children():
                walk(child)

        for child in self.children():
            walk(child)
        return out

    def allows_capture(self) -> bool:
        """Whether every part allows its ``forward`` to be captured into a HIP graph (``Part.graph_safe``)."""
        return all(part.graph_safe for part in self.all_parts())

    def cache_needs(self) -> List[object]:
        """One entry per schedule entry: the mixer's need, or None when it reads another entry's cache."""
        needs = []
        for entry in self.schedule:
            need = self.blocks[entry.layer].cache_need()
            needs.append(need if entry.cache_from is None else None)
        return needs

    # -- arithmetic ---------------------------------------------------------------------
    def embed(self, token_ids: torch.Tensor, ctx) -> torch.Tensor:
        """The residual stream before the first block: float32 ``[T, H]``."""
        residual = self.embedding.forward(token_ids, ctx)
        if self.spec.embedding_position is not None:
            residual = self.positions[self.spec.embedding_position].on_embeddings(residual, ctx)
        return residual

    def run_schedule(self, residual: torch.Tensor, pending, ctx, first: int = 0, last: Optional[int] = None):
        """Runs schedule entries ``first .. last - 1`` on ``residual`` (updated in place); takes and returns ``pending``,
        the sub-layer output that the next norm still has to add."""
        last = len(self.schedule) if last is None else last
        for index in range(first, last):
            entry = self.schedule[index]
            owner = index if entry.cache_from is None else entry.cache_from
            cache = ctx.cache_view(owner)
            # the norm that reads this block's output: the one the next entry's block begins with, if it begins with one
            # (the final norm works on chosen rows and takes its input as it is)
            following = self.blocks[self.schedule[index + 1].layer].input_norm() if index + 1 < len(self.schedule) else None
            pending = self.blocks[entry.layer].forward(residual, pending, ctx, cache, entry.cache_from is None, next_norm=following)
        return pending

    def forward(self, token_ids: torch.Tensor, ctx):
        """Runs every block; returns ``(residual float32 [T, H], pending [T, H])``."""
        residual = self.embed(token_ids, ctx)
        return residual, self.run_schedule(residual, None, ctx)

    def logits(self, residual: torch.Tensor, pending, rows: torch.Tensor, ctx) -> torch.Tensor:
        """Final norm and output head on ``rows`` (int32 [R]) only: float32 [R, vocab]."""
        hidden = self.final_norm.forward(residual, pending, ctx, rows=rows)
        return self.head.forward(hidden, ctx)
