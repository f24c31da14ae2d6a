"""The scheduler: admits requests, cuts prompts into portions, decodes, finishes, frees.

Every ``advance()`` builds one step for the step function: one token for every running
request (up to ``max_batch_size`` of them, oldest first) and, with the token budget that
is left, portions of the prompts that are being fed or can be admitted. A portion never
splits a bidirectional block. The logits of decoded tokens and of portions that end a
prompt are sampled, the tokens committed, finished requests released.

What happens when pages run out: a request is promised the pages for its whole length
(prompt + ``max_new_tokens``) when it is admitted, so a running request can never run out.
A waiting request that does not fit stays in the queue (later ones that fit may pass it)
until pages come back; if nothing is live any more and it still does not fit, it can
never fit and fails alone with "Insufficient KV cache capacity for request N (needs T
tokens)." — as the reference decides (``kestrel/scheduler/scheduler.py:550-568,1650-1652``).

Reference: queues and phases ``scheduler.py:285-286``, ``types.py:24-31``; admission test
``scheduler.py:1615-1665`` (pages for ``prompt + max_new`` reserved at admission,
``kestrel/models/moondream/runtime.py:1885-1913``); token budget 2048
(``scheduler.py:54,171-268``); decode cohort = first ``max_batch_size`` running
(``scheduler.py:2219-2240``); finishing ``scheduler.py:3058-3108``. The reference runs
either prompts or decodes in a forward and never cuts a prompt; mixing both in one
step and cutting prompts is this engine's own design.

Pipelining (``pipeline_depth`` 2, ``scheduler.py:459-548``, ``pipeline.py:49-65``): a step is
launched before the tokens of the step before it have reached the host. A request enters
``running`` as soon as its first token is sampled on the device; its next step names that
token as ``PENDING_TOKEN`` and the embedding kernel takes it from the device table that the
sampling kernel filled. The host reads a step's tokens one step late, so its work between
two steps overlaps the GPU's. A request that turns out to have stopped has then already
been launched once more: that step's token is thrown away, and the slot and pages are given
back when it has been read ("zombie" steps, ``scheduler.py:2482-2527``). Limits of length
are known without the token, so no step is launched beyond them.
"""

from __future__ import annotations

import logging
import time
from collections import deque
from dataclasses import dataclass, field
from typing import Deque, Dict, List, Optional, Tuple

import numpy as np
import torch

from .step import PENDING_TOKEN, StepEntry, StepRefused
from .types import GenerationRequest, RequestMetrics, RequestPhase, SchedulerResult, Sequence_

_LOGGER = logging.getLogger(__name__)


@dataclass
class PlannedRow:
    seq: Sequence_
    entry: StepEntry
    samples: bool            # its last place's logits are sampled
    kind: str                # "decode" or "prefill"


@dataclass
class StepPlan:
    rows: List[PlannedRow] = field(default_factory=list)

    @property
    def n_tokens(self) -> int:
        return sum(len(r.entry.tokens) for r in self.rows)


@dataclass
class LaunchedStep:
    """A step whose forward and sampling are queued on the GPU and whose tokens are on
    their way to ``ids`` (pinned host memory; ``event`` tells when they are there)."""

    rows: List[PlannedRow]
    ids: Optional[torch.Tensor]
    event: Optional["torch.cuda.Event"]
    logprobs: Optional[torch.Tensor] = None


class GenerationScheduler:
    HOST_RING = 8

    def __init__(self, runner, sampler, max_batch_size: int, max_num_batched_tokens: int,
                 eos_token_ids: Tuple[int, ...] = (), max_positions: Optional[int] = None,
                 pipeline_depth: int = 1) -> None:
        if pipeline_depth not in (1, 2):
            raise ValueError("pipeline_depth must be 1 (every step read before the next) or 2")
        self.runner, self.sampler = runner, sampler
        self.pipeline_depth = pipeline_depth
        self._inflight: Deque[LaunchedStep] = deque()
        self._host_ids: List[Optional[torch.Tensor]] = [None] * self.HOST_RING
        self._host_next = 0
        self.max_batch_size = max_batch_size
        self.max_num_batched_tokens = max_num_batched_tokens
        self.eos_token_ids = tuple(eos_token_ids)
        self.max_positions = max_positions if max_positions is not None else runner.model.plan.max_positions
        self.waiting: Deque[Sequence_] = deque()
        self.prefilling: List[Sequence_] = []
        self.running: List[Sequence_] = []
        self.completed: List[SchedulerResult] = []
        self.steps = 0
        self.failed_steps = 0

    # ------------------------------------------------------------------ intake
    def enqueue_request(self, request: GenerationRequest) -> None:
        if request.max_new_tokens <= 0:
            raise ValueError("max_new_tokens must be positive")
        if request.temperature < 0:
            raise ValueError("temperature must be non-negative")
        if not 0 < request.top_p <= 1:
            raise ValueError("top_p must be in (0, 1]")
        if request.allowed_token_ids is not None and len(request.allowed_token_ids) == 0:
            raise ValueError("an allow-list needs at least one token")
        if request.prompt_length == 0:
            raise ValueError("a request needs at least one prompt token or embedding")
        if request.prefill_length >= self.max_positions:
            raise ValueError(f"prompt of {request.prefill_length} tokens leaves no room in a context of {self.max_positions}")
        self._check_contents(request)
        if request.longest_block > self.max_num_batched_tokens:
            raise ValueError(f"the bidirectional block of {request.longest_block} positions does not fit in one step "
                             f"of {self.max_num_batched_tokens} tokens")
        self.waiting.append(Sequence_(request))

    def _check_contents(self, request: GenerationRequest) -> None:
        """What a request brings must be what the step function takes, so that it is refused here,
        alone, and not in the middle of a step that others share."""
        plan = self.runner.model.plan
        vocab = plan.vocab_size
        for name, ids in (("prompt_ids", request.prompt_ids), ("prefix_ids", request.prefix_ids),
                          ("generated_prefix.tokens", request.generated_prefix.tokens),
                          ("suppress_next_token_ids", request.suppress_next_token_ids),
                          ("suppressed_token_ids", request.suppressed_token_ids),
                          ("allowed_token_ids", request.allowed_token_ids or ()),
                          ("stop_ids", request.stop_ids or ())):
            if len(ids) == 0:
                continue
            values = np.asarray(ids)
            if values.ndim != 1 or values.dtype.kind not in "iu":
                raise ValueError(f"{name} must be a flat sequence of integer token ids")
            if name == "prompt_ids" and request.prompt_embeds is not None:
                values = values[values != -1]             # places whose embeddings are given
                if values.size == 0:
                    continue
            low, high = int(values.min()), int(values.max())
            if low < 0 or high >= vocab:
                bad = low if low < 0 else high
                raise ValueError(f"{name}: token id {bad} outside the vocabulary of {vocab}")
        dim = getattr(plan, "dim", None)
        for name, embeds in (("prefix_embeds", request.prefix_embeds), ("prompt_embeds", request.prompt_embeds)):
            if embeds is None:
                continue
            if not isinstance(embeds, torch.Tensor) or embeds.dim() != 2 or not embeds.is_floating_point() \
                    or (dim is not None and embeds.shape[1] != dim):
                shape = tuple(embeds.shape) if isinstance(embeds, torch.Tensor) else type(embeds).__name__
                raise ValueError(f"{name} must be a floating-point tensor [rows, {dim}], got {shape}")
        if request.prompt_embeds is not None:
            n_places = int((np.asarray(request.prompt_ids) == -1).sum()) if len(request.prompt_ids) else 0
            if n_places != int(request.prompt_embeds.shape[0]):
                raise ValueError(f"prompt_embeds has {int(request.prompt_embeds.shape[0])} rows for {n_places} places of "
                                 f"prompt_ids that hold -1")
        request.check_blocks()

    def has_pending_work(self) -> bool:
        return bool(self.waiting or self.prefilling or self.running or self._inflight)

    def pop_completed(self) -> List[SchedulerResult]:
        out, self.completed = self.completed, []
        return out

    # ------------------------------------------------------------------ planning
    def _target_length(self, request: GenerationRequest) -> int:
        return min(request.prompt_length + request.max_new_tokens, self.max_positions)

    def _portion(self, seq: Sequence_, budget: int) -> int:
        """Places of the prompt to feed next within ``budget`` (0: does not fit now). A portion that
        does not end the prompt ends on a page boundary where it can, and never inside a
        bidirectional block: it is cut back to the block's start, and a block that starts the
        portion goes in whole or not at all."""
        request = seq.request
        left = request.prefill_length - seq.fed
        end = seq.fed + min(left, budget)
        blocks = request.block_ranges

        def inside_a_block(place: int) -> Optional[Tuple[int, int]]:
            return next(((lo, hi) for lo, hi in blocks if lo < place < hi), None)

        split = inside_a_block(end)
        if split is not None:
            end = split[0]                # the block waits for a portion that holds all of it
        if seq.fed < end < request.prefill_length:
            # cut on a page boundary where that is possible, so that the next portion starts on one
            page = self.runner.cache.page_size
            aligned = end // page * page
            if aligned > seq.fed and inside_a_block(aligned) is None:
                end = aligned
        return max(0, end - seq.fed)

    def _prompt_slice(self, seq: Sequence_, take: int) -> StepEntry:
        request = seq.request
        lo, hi = seq.fed, seq.fed + take
        ids, embeds = request.places(lo, hi)
        tokens = ids.tolist() if take <= 64 else ids
        bidirectional = [block for block in request.block_ranges if lo <= block[0] and block[1] <= hi]
        ends_prompt = hi == request.prefill_length
        return StepEntry(seq.slot, tokens, want=[take - 1] if ends_prompt else [], embeds=embeds,
                         bidirectional=bidirectional, start=lo)

    def plan_step(self) -> StepPlan:
        plan = StepPlan()
        budget = self.max_num_batched_tokens
        # 1. one token for every running request (stable cohort: the oldest first)
        for seq in self.running[: self.max_batch_size]:
            request = seq.request
            if seq.launched >= request.max_new_tokens or request.prompt_length + seq.launched >= self.max_positions:
                continue                  # its last token is on its way: it ends when that is read
            token = seq.tokens[-1] if len(seq.tokens) == seq.launched else PENDING_TOKEN
            entry = StepEntry(seq.slot, [token], want=[0], start=request.prompt_length + seq.launched - 1)
            plan.rows.append(PlannedRow(seq, entry, True, "decode"))
            budget -= 1
        # 2. prompts already being fed, in order of admission
        for seq in self.prefilling:
            if budget <= 0:
                break
            take = self._portion(seq, budget)
            if take:
                entry = self._prompt_slice(seq, take)
                plan.rows.append(PlannedRow(seq, entry, bool(entry.want), "prefill"))
                budget -= take
        # 3. admit waiting requests while slots, pages and budget allow
        admitted = []
        for seq in list(self.waiting):
            live = len(self.running) + len(self.prefilling) + len(admitted)
            if budget <= 0 or live >= self.max_batch_size:
                break
            target = self._target_length(seq.request)
            if not self.runner.cache.can_admit(target, self.max_num_batched_tokens):
                continue                  # waits for pages; a later, smaller request may pass
            take = self._portion(seq, budget)
            if not take:
                continue
            seq.slot = self.runner.admit(target, self.max_num_batched_tokens)
            seq.phase = RequestPhase.PREFILLING
            seq.prefill_started_at = time.perf_counter()
            admitted.append(seq)
            entry = self._prompt_slice(seq, take)
            plan.rows.append(PlannedRow(seq, entry, bool(entry.want), "prefill"))
            budget -= take
        for seq in admitted:
            self.waiting.remove(seq)
            self.prefilling.append(seq)
        # prompt portions first in the packed batch: a portion that starts on a page boundary then
        # also starts on a multiple of 16 tokens, which is what lets the cache write store whole
        # pages of values at once
        plan.rows.sort(key=lambda row: row.kind != "prefill")
        return plan

    # ------------------------------------------------------------------ running
    def advance(self) -> bool:
        """Launch the next step, then read the oldest one that may no longer wait. Returns
        whether anything was done."""
        plan = self.plan_step()
        did = False
        if plan.rows:
            self._launch(plan)
            did = True
        keep = self.pipeline_depth - 1 if plan.rows else 0
        while len(self._inflight) > keep:
            self._commit_step(self._inflight.popleft())
            did = True
        return did or self._fail_unfittable()

    def drain(self) -> None:
        """Read every step that is still in flight (``kestrel/engine/core.py:1556-1569``: what a pause
        does before it reports). Nothing is launched; requests keep their pages."""
        while self._inflight:
            self._commit_step(self._inflight.popleft())

    def _sample(self, plan: StepPlan, logits: torch.Tensor):
        """Queue the sampling of the rows that end a prompt or decode, and the copy of their
        tokens to the host. Returns ``(ids, event, logprobs)``."""
        sampled_rows = [row for row in plan.rows if row.samples]
        ids = event = logprobs = None
        if sampled_rows:
            requests = [row.seq.request for row in sampled_rows]
            temps = [r.temperature for r in requests]
            tops = [r.top_p for r in requests]
            seeds = [r.seed if r.seed is not None else r.request_id for r in requests]
            indices = [row.seq.launched for row in sampled_rows]
            # masks: what a request never wants, and what it does not want as its first new token
            suppress = [(i, int(t)) for i, r in enumerate(requests) for t in r.suppressed_token_ids]
            suppress += [(i, int(t)) for i, (row, r) in enumerate(zip(sampled_rows, requests))
                         if row.seq.launched == r.generated_prefix_length for t in r.suppress_next_token_ids]
            allowed = [r.allowed_token_ids for r in requests]
            extras = {}
            if suppress:
                extras["suppress"] = suppress
            if any(a for a in allowed):
                extras["allowed"] = allowed
            if any(r.return_logprobs for r in requests):
                extras["logprobs"] = True
            if self.pipeline_depth > 1:
                # the step function has left every logits row's slot on the device
                on_device = getattr(self.runner, "logit_slots", None)
                if on_device is not None and on_device.numel() == len(sampled_rows) == logits.shape[0]:
                    extras["slots"] = on_device
                else:
                    extras["slots"] = [row.seq.slot for row in sampled_rows]
            if logits.is_cuda and "logprobs" not in extras:
                # the sampling kernel writes the ids into pinned host memory itself: no copy behind it
                # (the kernel of the log-probabilities reads them on the device)
                extras["out"] = self._host_buffer(len(sampled_rows), torch.int32)
            if extras.keys() - {"slots", "out"}:
                ids, logprobs = self.sampler.sample_step(logits, temps, tops, seeds, indices, **extras)
            else:
                ids = self.sampler.sample(logits, temps, tops, seeds, indices, **extras)
            if logits.is_cuda:
                if ids.is_cuda:                       # (a sampler that brought its own output)
                    ids, event = self._to_host(ids)
                if logprobs is not None:
                    logprobs, event = self._to_host(logprobs)
                else:
                    event = torch.cuda.Event()
                    event.record()
        return ids, event, logprobs

    def _launch(self, plan: StepPlan) -> None:
        self.steps += 1
        try:
            logits = self.runner.step([row.entry for row in plan.rows])
            ids, event, logprobs = self._sample(plan, logits)
        except Exception as exc:
            self._fail_rows(plan, exc)
            return
        for row in plan.rows:
            seq = row.seq
            if row.kind == "prefill":
                seq.fed += len(row.entry.tokens)
            if not row.samples:
                continue
            seq.launched += 1
            seq.inflight += 1
            if row.kind == "prefill":       # its first token exists on the device: it decodes from the next step on
                self.prefilling.remove(seq)
                self.running.append(seq)
                seq.phase = RequestPhase.RUNNING
        self._inflight.append(LaunchedStep(plan.rows, ids, event, logprobs))

    def _fail_rows(self, plan: StepPlan, exc: Exception) -> None:
        """The step function raised. If it refused one entry (``StepRefused``: found before anything
        ran or changed), that request fails alone and the others are planned again. Anything else
        may have happened half-way through the step: every request of the step fails, the ones in
        other queues go on (``kestrel/scheduler/scheduler.py:1576-1613,1696-1763``). Slots and pages
        come back at once, or when a step of the request that is still in flight has been read."""
        now = time.perf_counter()
        if isinstance(exc, StepRefused) and 0 <= exc.entry_index < len(plan.rows):
            rows = [plan.rows[exc.entry_index]]
        else:
            rows = list(plan.rows)
        _LOGGER.error("step %d failed (%s: %s): %d of its %d requests fail: %s", self.steps, type(exc).__name__, exc,
                      len(rows), len(plan.rows), [row.seq.request.request_id for row in rows])
        for row in rows:
            if row.seq.finish_reason is None:
                self._finish(row.seq, "error", now, f"{type(exc).__name__}: {exc}")
        self.failed_steps += 1

    def _host_buffer(self, n: int, dtype) -> torch.Tensor:
        """Pinned memory for a step's tokens or log-probabilities, from a ring with more buffers than
        steps in flight."""
        index = self._host_next
        self._host_next = (index + 1) % self.HOST_RING
        buf = self._host_ids[index]
        if buf is None or buf.numel() < n:
            buf = self._host_ids[index] = torch.empty(max(n, 256), dtype=torch.int32, pin_memory=True)
        return buf[:n].view(dtype)                            # int32 or float32: four bytes either way

    def _to_host(self, values: torch.Tensor):
        """Start the copy of a step's tokens (or their log-probabilities) into pinned memory; the
        event tells when it is done."""
        host = self._host_buffer(values.numel(), values.dtype)
        host.copy_(values, non_blocking=True)
        event = torch.cuda.Event()
        event.record()
        return host, event

    def _commit_step(self, step: LaunchedStep) -> None:
        if step.event is not None:
            step.event.synchronize()
        ids = step.ids.tolist() if step.ids is not None else []
        logprobs = step.logprobs.tolist() if step.logprobs is not None else None
        now = time.perf_counter()
        at = 0
        for row in step.rows:
            if not row.samples:
                continue
            seq = row.seq
            token = int(ids[at])
            logprob = logprobs[at] if logprobs is not None else None
            at += 1
            seq.inflight -= 1
            if seq.finish_reason is not None:      # it stopped a step ago: this token is not part of it
                if seq.inflight == 0:
                    self._release(seq)
                continue
            if row.kind == "prefill":
                seq.first_token_at = now
            if seq.request.return_logprobs and logprob is not None:
                seq.logprobs.append(float(logprob))
            self._commit(seq, token, now)

    def _commit(self, seq: Sequence_, token: int, now: float) -> None:
        seq.tokens.append(token)
        request = seq.request
        if request.on_token is not None:
            request.on_token(token, len(seq.tokens) - 1)
        stop_ids = request.stop_ids if request.stop_ids is not None else self.eos_token_ids
        reason = None
        if token in stop_ids:
            reason = "stop"
        elif len(seq.tokens) >= request.max_new_tokens or seq.total_length >= self.max_positions:
            reason = "length"
        if reason is not None:
            self._finish(seq, reason, now)

    def _finish(self, seq: Sequence_, reason: str, now: float, error: Optional[str] = None) -> None:
        seq.finish_reason, seq.finished_at, seq.phase = reason, now, RequestPhase.COMPLETED
        if seq in self.running:
            self.running.remove(seq)
        if seq in self.prefilling:
            self.prefilling.remove(seq)
        if seq.inflight == 0:
            self._release(seq)             # else: when the step that is still in flight has been read
        started = seq.prefill_started_at if seq.prefill_started_at is not None else seq.submitted_at
        first = seq.first_token_at if seq.first_token_at is not None else now
        metrics = RequestMetrics(
            prompt_tokens=seq.request.prompt_length,
            decode_tokens=max(0, len(seq.tokens) - seq.request.generated_prefix_length),
            prefill_time_ms=(first - started) * 1e3, ttft_ms=(first - seq.submitted_at) * 1e3,
            decode_time_ms=(now - first) * 1e3)
        self.completed.append(SchedulerResult(seq.request.request_id, list(seq.tokens), reason, metrics, error,
                                              list(seq.logprobs) if seq.request.return_logprobs else None))

    def _release(self, seq: Sequence_) -> None:
        if seq.slot is not None:
            self.runner.release(seq.slot)
            seq.slot = None

    def _fail_unfittable(self) -> bool:
        """Nothing could be planned. If nothing is live either, the first waiting request can
        never be served: fail it alone and go on."""
        if self.running or self.prefilling or self._inflight or not self.waiting:
            return False
        seq = self.waiting.popleft()
        needed = self._target_length(seq.request)
        message = f"Insufficient KV cache capacity for request {seq.request.request_id} (needs {needed} tokens)."
        _LOGGER.warning("%s", message)
        self._finish(seq, "error", time.perf_counter(), message)
        return True

    def run_until_done(self) -> List[SchedulerResult]:
        results: List[SchedulerResult] = []
        while self.has_pending_work():
            if not self.advance() and not self.completed:
                raise RuntimeError("the scheduler made no progress")
            results.extend(self.pop_completed())
        results.extend(self.pop_completed())
        return results
