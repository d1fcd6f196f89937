"""Interfaces of the parts a decoder is put together from.

A *part* owns tensors (declared as :class:`Param`) and one piece of arithmetic.
It is given its sizes and constants at construction and never learns which
model it sits in.  Six families exist, each with a registry from a kind name to a
class so that an architecture (or a test) can add its own:

``Mixer``
    mixes information between the tokens of a sequence (attention here).  It
    declares what it needs of the cache manager through :meth:`cache_need`.
``FeedForward``
    ``[T, H] -> [T, H]`` per token (dense gated MLP here; routed experts would
    be another kind behind the same call).
``Norm``
    owns the residual update: ``residual += delta; return normalise(residual)``.
``PositionEncoding``
    either changes the embeddings (absolute encodings) or hands rotary tables to
    the mixer, which fuses the rotation into its cache write.

``Embedding``
    token ids -> the residual stream, float32 ``[T, H]``.
``OutputHead``
    normalised rows -> float32 logits ``[R, vocab]``.

``Block`` arranges one mixer, one feed-forward and their norms; arrangements have a
registry of their own (``register_arrangement``).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Dict, Optional, Tuple

import torch


# ----------------------------------------------------------------------------------------
# parameters
# ----------------------------------------------------------------------------------------
@dataclass(frozen=True)
class Param:
    """One tensor a part owns and where it comes from in a checkpoint.

    ``sources`` are checkpoint tensor names relative to the part's prefix; more
    than one means "concatenate along dim 0" (the reference fuses q/k/v and
    gate/up the same way, ``src/weight_loader.py:91-98``).  ``role`` decides the
    dtype it is held in: a ``matrix`` takes the run's dtype whatever the checkpoint
    stores, a ``vector`` (norm weights, biases) is always held in float32, a
    ``stored`` tensor stays in 32-bit when the checkpoint holds it so (a router's
    weights, say) and takes the run dtype otherwise.  ``product`` = False marks a
    matrix that no matrix product reads (a table that is only looked up).  ``init`` names the random-weights law: ``normal`` is
    N(0, 0.02), ``one_plus_normal`` is 1 + N(0, 0.02).
    """

    shape: Tuple[int, ...]
    sources: Tuple[str, ...]
    source_shapes: Tuple[Tuple[int, ...], ...]
    role: str = "matrix"
    init: str = "normal"
    alias_of: Optional[str] = None  # absolute checkpoint name this falls back to (tied head)
    product: bool = True


def single(name: str, shape: Tuple[int, ...], role: str = "matrix", init: str = "normal", product: bool = True) -> Param:
    return Param(shape=tuple(shape), sources=(name,), source_shapes=(tuple(shape),), role=role, init=init, product=product)


def fused_rows(names: Tuple[str, ...], shapes: Tuple[Tuple[int, ...], ...], role: str = "matrix") -> Param:
    rows = sum(s[0] for s in shapes)
    return Param(shape=(rows,) + tuple(shapes[0][1:]), sources=tuple(names), source_shapes=tuple(tuple(s) for s in shapes), role=role)


class Part:
    """Base of every part: a prefix in the checkpoint's name space plus declared tensors."""

    # Whether ``forward`` may be recorded into a HIP graph and replayed: it then reads nothing on the host that changes
    # from step to step (no ``.tolist()``, ``.item()`` or Python loop over a step's values) and launches the same kernels
    # on the same addresses every time.  One part that says False keeps the whole model's decode steps uncaptured.
    graph_safe = True

    def __init__(self, prefix: str = "") -> None:
        self.prefix = prefix
        self._prepared: Dict[str, object] = {}

    def params(self) -> Dict[str, Param]:
        """attribute name -> Param; the loader sets ``self.<attribute>`` to the bound tensor."""
        return {}

    def children(self) -> Tuple["Part", ...]:
        return ()

    def finalize(self, device: torch.device, dtype: torch.dtype) -> None:
        """Called once after the weights are bound (build tables, derived tensors)."""

    def prepare_kernels(self, ops) -> None:
        """Called once with the kernels' handle, after the weights are bound: a part hands the weights that its
        decode-sized products read to ``self.prepare_weight(ops, "<attribute>", ...)`` and from then on passes
        ``self.operand("<attribute>")`` where it passed the tensor.  Nothing has to be done here."""

    def prepare_weight(self, ops, attr: str, **options) -> None:
        """Lets the kernels make what they want of ``self.<attr>`` (copies in the order their lanes read, say); the
        part owns the result.  ``options`` are ``ops.prepare_weight``'s; several calls for one attribute add up."""
        prepare = getattr(ops, "prepare_weight", None)
        tensor = getattr(self, attr, None)
        if prepare is None or tensor is None:
            return
        known = self._prepared.get(attr)
        if known is not None and getattr(known, "weight", None) is not tensor:
            known = None  # bound again since: start over
        handle = prepare(tensor, handle=known, **options)
        if handle is not None:
            self._prepared[attr] = handle
        else:
            self._prepared.pop(attr, None)

    def operand(self, attr: str):
        """``self.<attr>`` as the kernels take it: what ``prepare_weight`` made of it, or the tensor itself.  A tensor
        that was bound again behind a prepared one is an error, not a silent fall to the slow path."""
        tensor = getattr(self, attr)
        handle = self._prepared.get(attr)
        if handle is None:
            return tensor
        if handle.weight is not tensor:
            raise RuntimeError(f"{type(self).__name__}.{attr} ({self.prefix!r}) was bound again after the kernels prepared it; "
                               "call ops.prepare(model, dtype) again")
        return handle

    def capture_key_bounds(self, ops, batch: int, max_model_len: int):
        """Context lengths below ``max_model_len`` for which a captured step of ``batch`` one-token rows should exist a
        second time, because this part's kernels would be launched differently when every sequence is that short (a
        capture fixes launch shapes; the step function replays the capture with the smallest bound that covers the
        step).  Default: none."""
        return ()

    def workspace_needs(self, ops, limits) -> Dict[str, int]:
        """Scratch this part may ask ``ctx.workspace`` for: buffer name -> the most float32 elements, for any step within
        ``limits`` (``max_num_tokens``, ``max_num_seqs``, ``max_model_len``).  The step function reserves these before it
        runs or captures anything and refuses to grow them later, because captured steps hold their addresses."""
        return {}


# ----------------------------------------------------------------------------------------
# what a mixer needs of the cache manager
# ----------------------------------------------------------------------------------------
PAGE = -1  # stands in a page tensor's shape for the dimension that runs over the tokens of a page


@dataclass(frozen=True)
class PagedNeed:
    """Memory that grows by one entry per token, kept in pages.

    ``tensors``: what a page holds, ``(name, shape of one page, dtype)`` per tensor; ``PAGE`` in a shape marks the
    dimension that runs over the page's tokens (its size is the page size, which the cache manager decides), dtype
    None = the run dtype.  The mixer decides the layout: attention keeps keys as ``(kv_heads, PAGE, head_dim)`` and
    values transposed (``parts.attention.kv_pages``); a mixer that caches one latent vector per token would name a
    single ``(PAGE, width)`` tensor.  Entries of the schedule with equal needs share a pool of pages.

    ``window`` = None keeps every token; an integer keeps the last ``window`` of them (a query at position p reads
    positions p-window+1 .. p), so pages wholly behind the window can be given back while the request is still running.
    """

    tensors: Tuple[Tuple[str, Tuple[int, ...], Optional[torch.dtype]], ...]
    window: Optional[int] = None

    def __post_init__(self) -> None:
        if not self.tensors:
            raise ValueError("a PagedNeed names at least one tensor per page")
        for name, shape, _ in self.tensors:
            if tuple(shape).count(PAGE) != 1:
                raise ValueError(f"page tensor {name!r}: its shape {tuple(shape)} must hold PAGE exactly once")
        if self.window is not None and self.window < 1:
            raise ValueError(f"window={self.window} must be at least 1")


@dataclass(frozen=True)
class StateNeed:
    """Per-request state of fixed size: ``(name, shape, dtype)`` per tensor, dtype None = run dtype."""

    tensors: Tuple[Tuple[str, Tuple[int, ...], Optional[torch.dtype]], ...]


@dataclass
class ResidualSink:
    """Where a sub-layer's last product may put its result itself: ``residual`` (float32 [T, H]) is what the output is
    to be added to and ``norm`` the norm that reads the sum next.  A mixer or feed-forward that sets
    ``accepts_sink = True`` takes ``sink=`` in ``forward`` and hands it to its last ``ops.linear(...,
    residual_norm=sink)`` (one that sets ``accepts_deferred = True`` is in turn ready to be given a ``DeferredNorm``
    as its input; others get a plain tensor); what comes back is either the product as always, or, when the kernels could fuse the add and
    the norm's first half into the product, a ``DeferredNorm`` (the residual is then already updated)."""

    residual: torch.Tensor
    norm: "Norm"


@dataclass
class DeferredNorm:
    """Normalised activations that have not been computed as such: ``x`` holds ``residual * weight`` in the run dtype and
    ``sums`` what is needed for each row's ``rsqrt(mean(residual^2) + eps)``; the products that read them
    (``ops.linear``, ``ops.linear_silu_mul``, ``ops.qkv_rope_write``) scale their result rows, which is the same thing.
    ``ops.materialize`` turns it into a plain tensor for anything else."""

    x: torch.Tensor  # [T, H]
    sums: torch.Tensor  # float32 [16, blocks]: sums of squares of the residual, per row and block of columns
    width: int
    eps: float
    norm: "Norm"  # the norm whose weight is already applied

    @property
    def shape(self):
        return self.x.shape

    @property
    def dtype(self):
        return self.x.dtype


class Mixer(Part):
    def cache_need(self):
        """``PagedNeed``, ``StateNeed`` or None."""
        return None

    def forward(self, x: torch.Tensor, ctx, cache, owns_cache: bool = True) -> torch.Tensor:
        """``x`` [T, H] in the run dtype -> [T, H] (or float32 partial sums [S, T, H] that the next norm adds up: what
        ``ops.linear(..., partials_ok=True)`` returns may be handed on as it is).

        ``cache`` is this schedule entry's view of the cache (or the entry's it reads
        from when ``owns_cache`` is false: then nothing may be written to it).
        """
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, x: torch.Tensor, ctx) -> torch.Tensor:
        """[T, H] -> [T, H], or float32 partial sums [S, T, H] (see ``Mixer.forward``)."""
        raise NotImplementedError


class Norm(Part):
    def deferred_form(self):
        """``(weight float32 [H], eps)`` if this norm is ``x * rsqrt(mean(x^2) + eps) * weight`` and may therefore be split
        into a product's epilogue (weight) and the next product's row scale; None otherwise."""
        return None

    def forward(self, residual: torch.Tensor, delta: Optional[torch.Tensor], ctx, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        """``residual`` [T, H] float32.

        ``delta`` is [T, H] or float32 partial sums [S, T, H], which are added first to last, or a ``DeferredNorm`` made
        for this very norm (then the residual is up to date and the ``DeferredNorm`` itself is what comes back).
        With ``rows`` None: ``residual += delta`` in place (delta may be None) and the
        normalised residual comes back in the run dtype, [T, H].  With ``rows`` (int32
        [R]): nothing is changed and ``normalise(residual[rows] + delta[rows])`` comes back.
        """
        raise NotImplementedError


class PositionEncoding(Part):
    def on_embeddings(self, hidden: torch.Tensor, ctx) -> torch.Tensor:
        return hidden

    def rotary_tables(self) -> Optional[Tuple[torch.Tensor, torch.Tensor]]:
        """(cos, sin), float32 [max_position, rotary_dim/2], or None when nothing rotates."""
        return None


class Embedding(Part):
    def forward(self, token_ids: torch.Tensor, ctx) -> torch.Tensor:
        """int32 ``[T]`` -> the residual stream before the first block, float32 ``[T, H]`` (a fresh tensor: blocks
        update it in place)."""
        raise NotImplementedError


class OutputHead(Part):
    def forward(self, hidden_rows: torch.Tensor, ctx) -> torch.Tensor:
        """``[R, H]`` in the run dtype (the final norm's output on the wanted rows) -> float32 logits ``[R, vocab]``."""
        raise NotImplementedError


class Block(Part):
    """One schedule entry's arithmetic: an arrangement of a mixer, a feed-forward and their norms around the residual.

    The residual stream is a float32 ``[T, H]`` tensor that blocks update in place.  What a block's last sub-layer
    produced may be handed on instead of added: ``forward`` takes the previous block's ``pending`` and returns its own
    (None when it has added everything itself), and whoever normalises next adds it inside the norm's kernel."""

    mixer: "Mixer"

    def input_norm(self) -> Optional["Norm"]:
        """The norm that reads this block's input first, if the block begins with one that the block before may hand its
        output to (``next_norm``); None if it does not (then it is given a plain ``pending`` and no sink is offered)."""
        return None

    def cache_need(self):
        return self.mixer.cache_need()

    def forward(self, residual: torch.Tensor, pending, ctx, cache, owns_cache: bool, next_norm: Optional["Norm"] = None):
        raise NotImplementedError


# ----------------------------------------------------------------------------------------
# registries of kinds
# ----------------------------------------------------------------------------------------
_MIXERS: Dict[str, Callable[..., Mixer]] = {}
_FEED_FORWARDS: Dict[str, Callable[..., FeedForward]] = {}
_NORMS: Dict[str, Callable[..., Norm]] = {}
_POSITIONS: Dict[str, Callable[..., PositionEncoding]] = {}
_EMBEDDINGS: Dict[str, Callable[..., Embedding]] = {}
_HEADS: Dict[str, Callable[..., OutputHead]] = {}
_ARRANGEMENTS: Dict[str, Callable[..., Block]] = {}
_TABLES = {"mixer": _MIXERS, "feed_forward": _FEED_FORWARDS, "norm": _NORMS, "position": _POSITIONS, "embedding": _EMBEDDINGS, "head": _HEADS,
           "arrangement": _ARRANGEMENTS}


def register_part(family: str, kind: str, factory: Callable[..., Part]) -> None:
    table = _TABLES[family]
    table[kind] = factory


def register_arrangement(kind: str, factory: Callable[..., Block]) -> None:
    """``factory(prefix, mixer, feed_forward, mixer_norm, ff_norm) -> Block``."""
    register_part("arrangement", kind, factory)


def make_part(family: str, kind: str, **kwargs) -> Part:
    table = _TABLES[family]
    if kind not in table:
        raise KeyError(f"unknown {family} kind {kind!r}; registered: {sorted(table)}")
    return table[kind](**kwargs)


@dataclass(frozen=True)
class PartSpec:
    """A kind name plus the constants handed to its constructor."""

    kind: str
    args: Tuple[Tuple[str, object], ...] = ()

    @staticmethod
    def of(kind: str, **kwargs) -> "PartSpec":
        return PartSpec(kind, tuple(sorted(kwargs.items())))

    def kwargs(self) -> Dict[str, object]:
        return dict(self.args)
