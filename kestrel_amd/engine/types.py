"""Requests and results of generation.

Reference: ``kestrel/scheduler/types.py:16-288`` (``GenerationRequest``, phases
``types.py:24-31``, ``SchedulerResult``), ``kestrel/engine/_types.py:35-56``
(``EngineMetrics``, ``EngineResult``).
"""

from __future__ import annotations

import enum
import time
from dataclasses import dataclass, field
from typing import Callable, List, Optional, Sequence, Tuple

import numpy as np
import torch


@dataclass(frozen=True)
class GeneratedPrefix:
    """Tokens a request has already generated (``kestrel/scheduler/types.py:16-21``): they are fed
    after the prompt, count against ``max_new_tokens`` and stand at the head of the result."""

    tokens: Tuple[int, ...] = ()
    logprobs: Optional[Tuple[float, ...]] = None


class RequestPhase(enum.Enum):
    WAITING = "waiting"
    PREFILLING = "prefilling"
    RUNNING = "running"
    COMPLETED = "completed"


@dataclass
class GenerationRequest:
    """One generation. The sequence is ``prefix_ids`` then ``prefix_embeds`` (given
    embeddings, e.g. an encoded image) then ``prompt_ids``. If ``prefix_embeds`` are given,
    ``prefix_ids`` and those embeddings form one block whose positions see each other both
    ways (the reference's BOS + image block, ``kestrel/models/moondream/runtime.py:1733-1743``).

    More than one block (the reference's mask is "dynamic in the number and position of image
    blocks", ``kestrel/models/moondream/text.py:146-157``, ``runtime.py:1711-1743``): ``prompt_ids`` may hold
    ``-1`` at places whose embeddings are the rows of ``prompt_embeds``, in order, and ``blocks`` names the
    position ranges ``[lo, hi)`` of the whole sequence whose tokens see each other both ways (``None``:
    the one block described above, if there is one; ``()``: none at all)."""

    request_id: int
    prompt_ids: Sequence[int]
    max_new_tokens: int
    temperature: float = 0.0
    top_p: float = 1.0
    prefix_embeds: Optional[torch.Tensor] = None
    prefix_ids: Sequence[int] = ()
    stop_ids: Optional[Tuple[int, ...]] = None      # None: the model's end-of-sequence ids
    seed: Optional[int] = None                      # None: the request id
    on_token: Optional[Callable[[int, int], None]] = None   # (token, index) as they are committed
    # masks before sampling and scores after it (``kestrel/scheduler/scheduler.py:2563-2604,3019-3042``)
    return_logprobs: bool = False                   # the chosen tokens' log-probabilities come back too
    suppress_next_token_ids: Sequence[int] = ()     # not to be the first generated token
    suppressed_token_ids: Sequence[int] = ()        # never to be generated
    allowed_token_ids: Optional[Sequence[int]] = None   # if given, the only tokens that may be generated
    generated_prefix: GeneratedPrefix = field(default_factory=GeneratedPrefix)
    prompt_embeds: Optional[torch.Tensor] = None    # rows for the places of ``prompt_ids`` that hold -1
    blocks: Optional[Sequence[Tuple[int, int]]] = None

    def __post_init__(self) -> None:
        # what a resumed request brings must be consistent (``kestrel/scheduler/types.py:215-237``)
        prefix = self.generated_prefix
        if prefix.logprobs is not None and len(prefix.logprobs) != len(prefix.tokens):
            raise ValueError(f"a resumed request brings {len(prefix.tokens)} tokens but {len(prefix.logprobs)} "
                             f"log-probabilities: one per token, or none")
        if prefix.tokens and len(prefix.tokens) >= self.max_new_tokens:
            raise ValueError(f"a resumed request brings {len(prefix.tokens)} tokens, which leaves nothing to generate "
                             f"within max_new_tokens={self.max_new_tokens}")
        if prefix.tokens and self.return_logprobs and prefix.logprobs is None:
            raise ValueError("a resumed request that wants log-probabilities back must bring those of the tokens "
                             "it generated before")
        self._ids: Optional[np.ndarray] = None
        self._given_before: Optional[np.ndarray] = None

    @property
    def _n_prefix_embeds(self) -> int:
        return 0 if self.prefix_embeds is None else int(self.prefix_embeds.shape[0])

    @property
    def prompt_length(self) -> int:
        return len(self.prefix_ids) + self._n_prefix_embeds + len(self.prompt_ids)

    @property
    def block_ranges(self) -> Tuple[Tuple[int, int], ...]:
        """The bidirectional blocks as sorted position ranges ``[lo, hi)``."""
        if self.blocks is not None:
            return tuple(sorted((int(lo), int(hi)) for lo, hi in self.blocks))
        n = self._n_prefix_embeds
        return ((0, n + len(self.prefix_ids)),) if n else ()

    @property
    def longest_block(self) -> int:
        return max((hi - lo for lo, hi in self.block_ranges), default=0)

    def check_blocks(self) -> None:
        """Blocks lie inside the prompt, hold at least one position and do not overlap."""
        at = 0
        for lo, hi in self.block_ranges:
            if not (at <= lo < hi <= self.prompt_length):
                raise ValueError(f"the bidirectional block [{lo}, {hi}) must hold at least one position, lie inside the "
                                 f"prompt of {self.prompt_length} positions and not overlap the block before it")
            at = hi

    def places(self, lo: int, hi: int):
        """The places ``[lo, hi)`` of what is fed before the first token is sampled: ``(ids, embeds)``, ids with
        -1 where an embedding is given, embeds the rows for those places (or ``None``)."""
        if self._ids is None:
            ids = np.concatenate([np.asarray(self.prefix_ids, dtype=np.int64).reshape(-1),
                                  np.full(self._n_prefix_embeds, -1, dtype=np.int64),
                                  np.asarray(self.prompt_ids, dtype=np.int64).reshape(-1),
                                  np.asarray(self.generated_prefix.tokens, dtype=np.int64).reshape(-1)])
            self._given_before = np.concatenate([[0], np.cumsum(ids == -1)])
            self._ids = ids
        ids = self._ids[lo:hi]
        a, b = int(self._given_before[lo]), int(self._given_before[hi])
        if a == b:
            return ids, None
        n_first = self._n_prefix_embeds                # rows come from the prefix first, then from prompt_embeds
        rows = []
        if a < n_first:
            rows.append(self.prefix_embeds[a:min(b, n_first)])
        if b > n_first:
            rows.append(self.prompt_embeds[max(a, n_first) - n_first:b - n_first])
        return ids, rows[0] if len(rows) == 1 else torch.cat([r.to(rows[0].device, rows[0].dtype) for r in rows])

    @property
    def generated_prefix_length(self) -> int:
        return len(self.generated_prefix.tokens)

    @property
    def prefill_length(self) -> int:
        """Places that are fed before the first token is sampled: the prompt, then what the
        request had generated before (``types.py:260-262``)."""
        return self.prompt_length + len(self.generated_prefix.tokens)


@dataclass
class RequestMetrics:
    prompt_tokens: int = 0
    decode_tokens: int = 0
    prefill_time_ms: float = 0.0
    ttft_ms: float = 0.0
    decode_time_ms: float = 0.0


@dataclass
class SchedulerResult:
    request_id: int
    tokens: List[int]
    finish_reason: str              # "stop", "length" or "error"
    metrics: RequestMetrics
    error: Optional[str] = None
    logprobs: Optional[List[float]] = None          # one per token, if the request asked for them


@dataclass
class Sequence_:
    """A request's life inside the scheduler."""

    request: GenerationRequest
    phase: RequestPhase = RequestPhase.WAITING
    slot: Optional[int] = None
    fed: int = 0                                     # prompt places already run
    tokens: List[int] = field(default_factory=list)  # generated so far, as the host has read them
    logprobs: List[float] = field(default_factory=list)
    launched: int = 0                                # tokens sampled on the device (>= len(tokens))
    inflight: int = 0                                # steps launched whose token the host has not read
    finish_reason: Optional[str] = None
    submitted_at: float = field(default_factory=time.perf_counter)
    first_token_at: Optional[float] = None
    prefill_started_at: Optional[float] = None
    finished_at: Optional[float] = None

    def __post_init__(self) -> None:
        # generated before: already part of the result, and of the count (``types.py:67-70``)
        prefix = self.request.generated_prefix
        self.tokens.extend(int(t) for t in prefix.tokens)
        self.launched = len(prefix.tokens)
        if self.request.return_logprobs and prefix.logprobs is not None:
            self.logprobs.extend(float(v) for v in prefix.logprobs)

    @property
    def total_length(self) -> int:
        return self.request.prompt_length + len(self.tokens)
