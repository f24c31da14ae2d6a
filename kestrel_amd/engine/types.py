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

import torch


class RequestPhase(enum.Enum):
    WAITING = "waiting"
    PREFILLING = "prefilling"
    RUNNING = "running"
    COMPLETED = "completed"


@dataclass
class GenerationRequest:
    """One generation. The sequence is ``prefix_ids`` then ``prefix_embeds`` (given
    embeddings, e.g. an encoded image) then ``prompt_ids``. If embeddings are given,
    ``prefix_ids`` and the embeddings form one block whose positions see each other both
    ways (the reference's BOS + image block, ``kestrel/models/moondream/runtime.py:1733-1743``)."""

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

    @property
    def block_length(self) -> int:
        n = 0 if self.prefix_embeds is None else int(self.prefix_embeds.shape[0])
        return n + len(self.prefix_ids) if n else 0

    @property
    def prompt_length(self) -> int:
        n = 0 if self.prefix_embeds is None else int(self.prefix_embeds.shape[0])
        return len(self.prefix_ids) + n + len(self.prompt_ids)


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

    @property
    def total_length(self) -> int:
        return self.request.prompt_length + len(self.tokens)
