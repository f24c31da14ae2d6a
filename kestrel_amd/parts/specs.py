"""Parameters of the parts a model is put together from.

A specification is plain data: sizes and constants, nothing about the model it
ends up in. An architecture turns its ``config.json`` into a ``ModelPlan`` made of
these; the parts are then built from the plan through the registries of
``kestrel_amd.parts.base``. A specification of a kind that is not listed here (a
test's toy mixer, another feed-forward) is any object with a ``kind`` attribute
whose part class is registered under that kind.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Mapping, Optional, Tuple


@dataclass(frozen=True)
class ParamSpec:
    """One tensor a part owns.

    ``role`` fixes how the tensor is held and initialised: ``matrix`` (2-D weight,
    model precision), ``vector`` (bias or gain), ``table`` (integer table, int32).
    ``init`` names the random-weights recipe: ``normal``, ``bias``, ``gain`` (around 1)
    or ``shift`` (around 0).
    """

    shape: Tuple[int, ...]
    role: str = "matrix"
    init: str = "normal"


@dataclass(frozen=True)
class NormSpec:
    kind: str
    dim: int
    eps: float
    bias: bool = True


@dataclass(frozen=True)
class PositionSpec:
    """Position encoding applied inside a mixer. ``kind`` ``none`` encodes nothing."""

    kind: str
    rotary_dim: int = 0
    theta: float = 0.0
    max_positions: int = 0


@dataclass(frozen=True)
class CacheSpec:
    """What an attention mixer keeps per token: keys and values of ``n_kv_heads`` x ``head_dim``.

    ``window`` = number of most recent positions a query reads (``None``: all), which
    lets the cache manager give back pages that have fallen out of it.

    The cache manager asks a specification three things and nothing else, so a mixer that keeps
    something other than keys and values per token (one latent, another layout) brings a
    specification class of its own with the same three: ``window``; ``page_tensors(page_size)``,
    the tensors of one page by name with their shapes (the manager allocates each as
    ``[runs of layers, pages, *shape]`` and hands a layer its slice as ``LayerCache.tensors[name]``);
    and ``group_key``, equal for layers that can share a block table and a pool of pages.
    """

    n_kv_heads: int
    head_dim: int
    window: Optional[int] = None

    def page_tensors(self, page_size: int) -> Dict[str, Tuple[int, ...]]:
        # values are kept transposed inside a page: eight consecutive keys of one channel are 16
        # bytes, which is what the MFMA attention kernels load at a time
        return {"k": (self.n_kv_heads, page_size, self.head_dim), "v": (self.n_kv_heads, self.head_dim, page_size)}

    @property
    def group_key(self) -> Tuple:
        return ("kv", self.n_kv_heads, self.head_dim, self.window)


@dataclass(frozen=True)
class StateSpec:
    """Per-request state of fixed size (one slot per live request), zeroed at admission."""

    shape: Tuple[int, ...]
    dtype: str = "float32"


@dataclass(frozen=True)
class AttentionSpec:
    kind: str
    dim: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    position: PositionSpec
    bias: bool = True
    scale: Optional[float] = None  # None: head_dim ** -0.5
    window: Optional[int] = None


@dataclass(frozen=True)
class DenseFeedForwardSpec:
    kind: str
    dim: int
    hidden_dim: int
    activation: str = "gelu_tanh"
    bias: bool = True


@dataclass(frozen=True)
class LayerSpec:
    """One block: its parts, how they are arranged, and where their tensors are named.

    ``arrangement``: ``parallel`` = ``x + mixer(norm(x)) + ff(norm(x))`` (one norm);
    ``sequential`` = ``x += mixer(norm(x)); x += ff(norm2(x))``.
    ``names`` maps ``"<part>.<local tensor name>"`` (parts: ``norm``, ``norm2``, ``mixer``,
    ``feed_forward``) to the tensor's name in the checkpoint.
    """

    arrangement: str
    norm: object
    mixer: object
    feed_forward: object
    norm2: Optional[object] = None
    names: Mapping[str, str] = field(default_factory=dict)


@dataclass(frozen=True)
class ScheduleEntry:
    """One run of a layer. ``reads_cache_of``: index of an earlier schedule entry whose
    cache this run reads instead of keeping one of its own."""

    layer: int
    reads_cache_of: Optional[int] = None


@dataclass(frozen=True)
class ModelPlan:
    """Everything the generic decoder needs: parts layer by layer and their order."""

    architecture: str
    vocab_size: int
    dim: int
    max_positions: int
    layers: Tuple[LayerSpec, ...]
    schedule: Tuple[ScheduleEntry, ...]
    final_norm: object
    head_bias: bool
    tied_head: bool
    names: Mapping[str, str]  # "embedding", "final_norm.weight", "head.weight", ... -> tensor name
    eos_token_ids: Tuple[int, ...] = ()
    bos_token_id: Optional[int] = None
    # constants some architectures put around the stack (all neutral by default): a factor on the
    # looked-up embeddings, a factor on the logits, and a cap ``c`` that turns logits into c * tanh(logits / c)
    embedding_scale: float = 1.0
    logit_scale: float = 1.0
    logit_softcap: Optional[float] = None
    # a position encoding of the whole model (a specification whose part is registered as a position
    # encoding): its ``add_to_embeddings`` runs on the embedded tokens before the first block; its tensors
    # are named by ``names["position.<local name>"]``. ``None``: positions are the mixers' business.
    position: Optional[object] = None

    def describe(self) -> Dict[str, object]:
        return {"architecture": self.architecture, "layers": len(self.layers), "schedule": len(self.schedule),
                "dim": self.dim, "vocab_size": self.vocab_size}
