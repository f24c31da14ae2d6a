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
"""

from __future__ import annotations

import time
from collections import deque
from dataclasses import dataclass, field
from typing import Deque, Dict, List, Optional, Tuple

import torch

from .step import StepEntry
from .types import GenerationRequest, RequestMetrics, RequestPhase, SchedulerResult, Sequence_


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


class GenerationScheduler:
    def __init__(self, runner, sampler, max_batch_size: int, max_num_batched_tokens: int,
                 eos_token_ids: Tuple[int, ...] = (), max_positions: Optional[int] = None) -> None:
        self.runner, self.sampler = runner, sampler
        self.max_batch_size = max_batch_size
        self.max_num_batched_tokens = max_num_batched_tokens
        self.eos_token_ids = tuple(eos_token_ids)
        self.max_positions = max_positions if max_positions is not None else runner.model.plan.max_positions
        self.waiting: Deque[Sequence_] = deque()
        self.prefilling: List[Sequence_] = []
        self.running: List[Sequence_] = []
        self.completed: List[SchedulerResult] = []
        self.steps = 0

    # ------------------------------------------------------------------ intake
    def enqueue_request(self, request: GenerationRequest) -> None:
        if request.max_new_tokens <= 0:
            raise ValueError("max_new_tokens must be positive")
        if request.temperature < 0:
            raise ValueError("temperature must be non-negative")
        if not 0 < request.top_p <= 1:
            raise ValueError("top_p must be in (0, 1]")
        if request.prompt_length == 0:
            raise ValueError("a request needs at least one prompt token or embedding")
        if request.prompt_length >= self.max_positions:
            raise ValueError(f"prompt of {request.prompt_length} tokens leaves no room in a context of {self.max_positions}")
        if request.block_length > self.max_num_batched_tokens:
            raise ValueError(f"the bidirectional block of {request.block_length} positions does not fit in one step "
                             f"of {self.max_num_batched_tokens} tokens")
        self.waiting.append(Sequence_(request))

    def has_pending_work(self) -> bool:
        return bool(self.waiting or self.prefilling or self.running)

    def pop_completed(self) -> List[SchedulerResult]:
        out, self.completed = self.completed, []
        return out

    # ------------------------------------------------------------------ planning
    def _target_length(self, request: GenerationRequest) -> int:
        return min(request.prompt_length + request.max_new_tokens, self.max_positions)

    def _portion(self, seq: Sequence_, budget: int) -> int:
        """Places of the prompt to feed next within ``budget`` (0: does not fit now)."""
        request = seq.request
        left = request.prompt_length - seq.fed
        take = min(left, budget)
        block = request.block_length
        if seq.fed < block and seq.fed + take < block:
            return 0                      # the block must go in whole
        return take

    def _prompt_slice(self, seq: Sequence_, take: int) -> StepEntry:
        request = seq.request
        lo, hi = seq.fed, seq.fed + take
        n_ids = len(request.prefix_ids)
        n_emb = 0 if request.prefix_embeds is None else int(request.prefix_embeds.shape[0])
        tokens: List[int] = []
        embeds = None
        for p in range(lo, min(hi, n_ids)):
            tokens.append(int(request.prefix_ids[p]))
        if hi > n_ids and lo < n_ids + n_emb:
            a, b = max(lo, n_ids) - n_ids, min(hi, n_ids + n_emb) - n_ids
            tokens.extend([-1] * (b - a))
            embeds = request.prefix_embeds[a:b]
        for p in range(max(lo, n_ids + n_emb), hi):
            tokens.append(int(request.prompt_ids[p - n_ids - n_emb]))
        block = request.block_length
        bidirectional = [(0, block)] if block and lo == 0 else []
        ends_prompt = hi == request.prompt_length
        return StepEntry(seq.slot, tokens, want=[take - 1] if ends_prompt else [], embeds=embeds,
                         bidirectional=bidirectional, start=lo)

    def plan_step(self) -> StepPlan:
        plan = StepPlan()
        budget = self.max_num_batched_tokens
        # 1. one token for every running request (stable cohort: the oldest first)
        for seq in self.running[: self.max_batch_size]:
            entry = StepEntry(seq.slot, [seq.tokens[-1]], want=[0], start=seq.total_length - 1)
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
        return plan

    # ------------------------------------------------------------------ running
    def advance(self) -> bool:
        """Plan and run one step. Returns whether anything was done."""
        plan = self.plan_step()
        if not plan.rows:
            return self._fail_unfittable()
        self.steps += 1
        logits = self.runner.step([row.entry for row in plan.rows])
        sampled_rows = [row for row in plan.rows if row.samples]
        if sampled_rows:
            temps = [row.seq.request.temperature for row in sampled_rows]
            tops = [row.seq.request.top_p for row in sampled_rows]
            seeds = [row.seq.request.seed if row.seq.request.seed is not None else row.seq.request.request_id
                     for row in sampled_rows]
            indices = [len(row.seq.tokens) for row in sampled_rows]
            ids = self.sampler.sample(logits, temps, tops, seeds, indices).tolist()
        else:
            ids = []
        now = time.perf_counter()
        at = 0
        for row in plan.rows:
            seq = row.seq
            if row.kind == "prefill":
                seq.fed += len(row.entry.tokens)
            if not row.samples:
                continue
            token = int(ids[at])
            at += 1
            if row.kind == "prefill":
                self.prefilling.remove(seq)
                self.running.append(seq)
                seq.phase = RequestPhase.RUNNING
                seq.first_token_at = now
            self._commit(seq, token, now)
        return True

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
        if seq.slot is not None:
            self.runner.release(seq.slot)
            seq.slot = None
        started = seq.prefill_started_at if seq.prefill_started_at is not None else seq.submitted_at
        first = seq.first_token_at if seq.first_token_at is not None else now
        metrics = RequestMetrics(
            prompt_tokens=seq.request.prompt_length, decode_tokens=len(seq.tokens),
            prefill_time_ms=(first - started) * 1e3, ttft_ms=(first - seq.submitted_at) * 1e3,
            decode_time_ms=(now - first) * 1e3)
        self.completed.append(SchedulerResult(seq.request.request_id, list(seq.tokens), reason, metrics, error))

    def _fail_unfittable(self) -> bool:
        """Nothing could be planned. If nothing is live either, the first waiting request can
        never be served: fail it alone and go on."""
        if self.running or self.prefilling or not self.waiting:
            return False
        seq = self.waiting.popleft()
        needed = self._target_length(seq.request)
        message = f"Insufficient KV cache capacity for request {seq.request.request_id} (needs {needed} tokens)."
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
