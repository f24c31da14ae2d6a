"""Interfaces of the parts and the registries they are built through.

A part is built from its specification alone, says which tensors it owns
(``params``), takes them (``bind``) and runs on the packed tokens of one step
(``forward``). It never sees the model or the architecture it is used in.

Adding a part of a new kind: subclass the interface, and call ``register_mixer`` /
``register_feed_forward`` / ``register_norm`` / ``register_position`` with the kind
name that its specification carries.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, Dict, Optional

import torch

from .specs import CacheSpec, ParamSpec, StateSpec


class Part:
    """Common face of every part."""

    # Whether steps of every shape (prompt portions beside decoded tokens), not only those of one token per
    # request, may be captured with this part in them and replayed: its ``forward`` then neither
    # synchronises nor allocates outside ``batch.workspace`` for any batch, takes from the host side of the
    # batch nothing but its sizes, and passes over what pads a captured step: rows without a request
    # (``row_slot`` -1, possibly without tokens) and tokens that see no keys and are cached nowhere
    # (``kv_hi`` 0, slot -1). A model is replayed that way only if all of its parts say so.
    replays_every_step: bool = False

    def __init__(self, spec) -> None:
        self.spec = spec

    def params(self) -> Dict[str, ParamSpec]:
        """Local tensor name -> its shape and role."""
        return {}

    def bind(self, tensors: Dict[str, torch.Tensor], dtype: torch.dtype, device: torch.device) -> None:
        """Take the loaded tensors (on ``device``); ``dtype`` is the precision of activations."""


class Norm(Part):
    def forward(self, x: torch.Tensor, out: torch.Tensor, rows: Optional[torch.Tensor] = None) -> None:
        """Normalise fp32 rows of ``x`` (all, or those in ``rows``) into ``out``."""
        raise NotImplementedError

    def layernorm_operands(self):
        """Optional. A norm that computes ``(x - mean) / sqrt(var + eps) * weight + bias`` over the last axis
        says so here: ``(weight fp32 [dim], bias fp32 [dim] or None, eps)``. The linear kernels that can
        normalise their input rows themselves, or the rows they have just finished, then take the norm
        into their launch (a block's first norm in decode steps, the final norm before the head).
        ``None`` (the default): the norm is always run through ``forward``, in a launch of its own."""
        return None


@dataclass(frozen=True)
class Rotation:
    """A rotary encoding as the attention mixer and its kernels take it.

    ``table``: fp32 ``[positions, R]``, row ``p`` = the cosines of the ``R / 2`` angles of position
    ``p``, then their sines; the first ``R`` channels of every query and key head are turned.
    ``pairing``: which two channels angle ``i`` turns: ``"halves"`` = ``i`` and ``i + R / 2``,
    ``"interleaved"`` = ``2 i`` and ``2 i + 1``.
    """

    table: torch.Tensor
    pairing: str = "halves"


class PositionEncoding(Part):
    """How positions are encoded, inside a mixer (``AttentionSpec.position``) or once for the whole
    model (``ModelPlan.position``). An encoding that turns pairs of channels by angles that grow with
    the position offers ``rotation``; one that adds something to the embeddings before the first block
    overrides ``add_to_embeddings``; one that offers neither is applied nowhere (order then comes from
    elsewhere, or from nowhere).

    ``axes``: how many numbers say where a token stands. 1: its place in the sequence, which every
    step carries as ``StepBatch.positions`` ``[tokens]``. More (rows and columns of an image patch, time):
    the step then also carries ``StepBatch.position_axes`` ``[tokens, axes]``, taken from
    ``StepEntry.positions`` where an entry gives them and else the place in the sequence on every axis."""

    axes: int = 1

    def rotation(self, device: torch.device) -> Optional[Rotation]:
        return None

    def add_to_embeddings(self, x: torch.Tensor, batch) -> None:
        """Model-level encodings: add the encoding of every token's position into the fp32 rows ``x``
        ``[tokens, dim]`` in place (``batch.positions``, ``batch.position_axes``). Under replayed graphs
        (``batch.decode_only``) this must neither synchronise nor allocate."""


@dataclass
class LayerCache:
    """What one run of a layer may touch of the cache manager's memory.

    ``group``: key into ``StepBatch.groups`` (block table, slots, window start) or ``None``
    if the mixer keeps nothing per token; ``tensors``: the paged tensors its cache
    specification named, each ``[pages, *shape of a page]`` (for attention ``k``:
    ``[pages, Hkv, page_size, hd]`` and ``v``: ``[pages, Hkv, hd, page_size]``, also reachable as
    ``.k`` and ``.v``); ``writes``: ``False`` when this run reads the cache of another run; ``state``:
    ``[slots + 1, *shape]`` per-request state, indexed by ``StepBatch.row_slot``; its last row is
    a spare for rows without a request (slot -1: what index -1 means to torch), whose content
    nobody reads.
    """

    group: Optional[int] = None
    tensors: Dict[str, torch.Tensor] = field(default_factory=dict)
    writes: bool = True
    state: Optional[torch.Tensor] = None

    @property
    def k(self) -> Optional[torch.Tensor]:
        return self.tensors.get("k")

    @property
    def v(self) -> Optional[torch.Tensor]:
        return self.tensors.get("v")


@dataclass
class SideLinear:
    """``out = act(a @ weight.T + bias)``: a piece of a block's work that depends on nothing the mixer
    computes (the first linear of a feed-forward that reads the same normalised input ``a``). A mixer
    that says so (``Mixer.takes_beside``) is handed it with ``attend`` and runs it in its own launch,
    on the compute units that its core leaves idle."""

    a: torch.Tensor                       # [n, in], the block's normalised input
    weight: torch.Tensor                  # [out, in]
    bias: Optional[torch.Tensor]
    out: torch.Tensor                     # [n, out]
    act: int                              # activation code of ``ops.linear``


class Mixer(Part):
    def cache_spec(self) -> Optional[CacheSpec]:
        """Keys and values kept per token, or ``None``."""
        return None

    def state_spec(self) -> Optional[StateSpec]:
        """Fixed-size state kept per request, or ``None``."""
        return None

    def query_tile(self) -> Optional[int]:
        """If the mixer's kernel wants the queries of a row in blocks of a size of its own: that
        size. The step then lists the blocks of that size in ``StepBatch.query_blocks[size]``
        (called after ``bind``: the size may depend on the precision)."""
        return None

    def forward(self, h: torch.Tensor, batch, cache: LayerCache, residual: torch.Tensor) -> None:
        """Add the mixer's output for the normalised input ``h`` into fp32 ``residual``."""
        raise NotImplementedError

    # Optional: a mixer that is "linear, core, linear" may offer its stages one by one. A block can
    # then run the first linear together with its norm and the feed-forward's first linear, and
    # the last linear together with the feed-forward's last (one kernel launch each when few rows
    # are decoded). A mixer without these is always run through ``forward``.
    def input_projection(self):
        """``(weight [out, in], bias or None, out)`` of the first linear, or ``None``."""
        return None

    def attend(self, projected: torch.Tensor, batch, cache: LayerCache, beside: Optional[SideLinear] = None) -> torch.Tensor:
        """The core on the projected input; returns the input of the output projection. ``beside``
        is only ever given after ``takes_beside`` said yes, and is done when this returns."""
        raise NotImplementedError

    def takes_beside(self, job: SideLinear, batch, cache: LayerCache) -> bool:
        """Whether ``attend`` would run ``job`` inside its own launch for this batch."""
        return False

    def output_projection(self):
        """``(weight, bias or None)`` of the last linear, whose result is added to the residual."""
        return None


class FeedForward(Part):
    def forward(self, h: torch.Tensor, batch, residual: torch.Tensor) -> None:
        """Add the feed-forward output for ``h`` into fp32 ``residual``."""
        raise NotImplementedError

    # Optional, as for mixers: a feed-forward that is "linear + activation, linear".
    def input_projection(self):
        """``(weight, bias or None, out, activation code)`` of the first linear, or ``None``."""
        return None

    def output_projection(self):
        """``(weight, bias or None)`` of the last linear, whose result is added to the residual."""
        return None


_REGISTRIES: Dict[str, Dict[str, Callable]] = {"mixer": {}, "feed_forward": {}, "norm": {}, "position": {}}


def _register(family: str, kind: str, cls: Callable) -> None:
    _REGISTRIES[family][kind] = cls


def register_mixer(kind: str, cls: Callable) -> None:
    _register("mixer", kind, cls)


def register_feed_forward(kind: str, cls: Callable) -> None:
    _register("feed_forward", kind, cls)


def register_norm(kind: str, cls: Callable) -> None:
    _register("norm", kind, cls)


def register_position(kind: str, cls: Callable) -> None:
    _register("position", kind, cls)


def build_part(family: str, spec) -> Part:
    """The part registered for ``spec.kind`` in ``family``."""
    kinds = _REGISTRIES[family]
    kind = getattr(spec, "kind", None)
    if kind not in kinds:
        raise ValueError(f"no {family} of kind {kind!r} is registered; known: {', '.join(sorted(kinds)) or 'none'}")
    return kinds[kind](spec)


def known_kinds(family: str):
    return sorted(_REGISTRIES[family])
