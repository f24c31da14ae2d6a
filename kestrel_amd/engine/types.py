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
    generated_prefix: GeneratedPrefix = field(default_factory=GeneratedPrefix)

    def __post_init__(self) -> None:
        # the checks of ``kestrel/scheduler/types.py:215-237``
        prefix = self.generated_prefix
        if prefix.logprobs is not None and len(prefix.logprobs) != len(prefix.tokens):
            raise ValueError("generated_prefix.logprobs must have the same length as generated_prefix.tokens")
        if prefix.tokens and len(prefix.tokens) >= self.max_new_tokens:
            raise ValueError("generated_prefix.tokens must be shorter than max_new_tokens")
        if prefix.tokens and self.return_logprobs and prefix.logprobs is None:
            raise ValueError("generated_prefix.logprobs is required when return_logprobs is true")

    @property
    def block_length(self) -> int:
        n = 0 if self.prefix_embeds is None else int(self.prefix_embeds.shape[0])
        return n + len(self.prefix_ids) if n else 0

    @property
    def prompt_length(self) -> int:
        n = 0 if self.prefix_embeds is None else int(self.prefix_embeds.shape[0])
        return len(self.prefix_ids) + n + len(self.prompt_ids)

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
