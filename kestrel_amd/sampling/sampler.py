"""Greedy and temperature / top-p selection of the next token on the GPU.

Reference: ``kestrel/scheduler/scheduler.py:2929-2993``: all rows greedy -> argmax;
otherwise per-row temperature and top-p, rows with temperature <= 1e-6 greedy
(``scheduler.py:55``). Before that, tokens a request suppresses get -inf and a request with an
allow-list keeps only the tokens on it (``scheduler.py:2563-2604,2854-2927``); after it, the
log-probability of the chosen token can be had (``scheduler.py:3019-3042``). The reference draws from one device generator seeded from
``torch.seed()`` (``scheduler.py:404-405``) and is not reproducible; here every draw comes
from a counter-based generator keyed by (engine seed, request seed, index of the token),
so a request's tokens do not depend on what else is in the batch.
"""

from __future__ import annotations

from typing import List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..ops import core

GREEDY_EPS = 1e-6
_MASK64 = (1 << 64) - 1


def mix_key(engine_seed: int, request_seed: int) -> int:
    """64-bit key of a request's random stream (splitmix64 of the two seeds)."""
    z = (engine_seed * 0x9E3779B97F4A7C15 + request_seed + 0x632BE59BD9B4E019) & _MASK64
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK64
    return z ^ (z >> 31)


def _signed(value: int) -> int:
    return value - (1 << 64) if value >= (1 << 63) else value


class Sampler:
    """``pending`` (optional) is the step function's device table of the requests' latest tokens:
    with ``slots`` given to a call, row ``r``'s token is also stored at ``pending[slots[r]]``, where
    the next step's embedding can read it before the host has seen it."""

    STAGING_RING = 4

    def __init__(self, device: torch.device, seed: int = 0, pending: Optional[torch.Tensor] = None) -> None:
        self.device, self.seed, self.pending = device, seed, pending
        self._staging: List[Optional[torch.Tensor]] = [None] * self.STAGING_RING
        self._events: List[Optional[torch.cuda.Event]] = [None] * self.STAGING_RING
        self._device_args: List[Optional[torch.Tensor]] = [None] * self.STAGING_RING
        self._next = 0

    def reserve(self, rows: int) -> None:
        """Argument buffers for steps of up to ``rows`` rows, made now (all of the ring) instead of at
        the first steps that fill them."""
        words = max(1024, 32 * rows)
        for index in range(self.STAGING_RING):
            if self._staging[index] is None or self._staging[index].numel() < words:
                self._staging[index] = torch.empty(words, dtype=torch.int32, pin_memory=True)
                self._device_args[index] = torch.empty(words, dtype=torch.int32, device=self.device)

    def _upload(self, columns: Sequence[np.ndarray]) -> List[torch.Tensor]:
        """Small arguments (4- or 8-byte columns of any length) to the device with one copy out of
        pinned memory."""
        words = [len(c) * (c.dtype.itemsize // 4) for c in columns]
        padded = [(w + 3) & ~3 for w in words]                   # every column starts on 16 bytes
        total = sum(padded)
        index = self._next
        self._next = (index + 1) % self.STAGING_RING
        if self._events[index] is not None:
            self._events[index].synchronize()
        if self._staging[index] is None or self._staging[index].numel() < total:
            self._staging[index] = torch.empty(max(total, 1024), dtype=torch.int32, pin_memory=True)
            self._device_args[index] = torch.empty(max(total, 1024), dtype=torch.int32, device=self.device)
        host, dev = self._staging[index], self._device_args[index]
        raw = host.numpy()
        views: List[torch.Tensor] = []
        at = 0
        for column, n, n_padded in zip(columns, words, padded):
            raw[at:at + n] = column.view(np.int32)
            kind = {np.dtype(np.float32): torch.float32, np.dtype(np.int64): torch.int64,
                    np.dtype(np.int32): torch.int32}[column.dtype]
            views.append(dev[at:at + n].view(kind))
            at += n_padded
        dev[:total].copy_(host[:total], non_blocking=True)
        event = self._events[index] or torch.cuda.Event()
        event.record()
        self._events[index] = event
        return views

    def sample(self, logits: torch.Tensor, temperatures: Sequence[float], top_ps: Sequence[float],
               request_seeds: Sequence[int], token_indices: Sequence[int],
               slots=None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """One token id per row of fp32 ``logits``; int32 on the device (or in ``out``)."""
        return self.sample_step(logits, temperatures, top_ps, request_seeds, token_indices, slots=slots, out=out)[0]

    def sample_step(self, logits: torch.Tensor, temperatures: Sequence[float], top_ps: Sequence[float],
                    request_seeds: Sequence[int], token_indices: Sequence[int],
                    slots=None,
                    suppress: Sequence[Tuple[int, int]] = (),
                    allowed: Optional[Sequence[Optional[Sequence[int]]]] = None,
                    logprobs: bool = False,
                    out: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
        """Masks, then one token id per row, then (if asked) the chosen tokens' log-probabilities.

        ``slots``: per row the place in the table of latest tokens (``pending``) that also receives
        the row's token: a list, or an int32 tensor that is on the device already (the step
        function leaves one there: ``ModelRunner.logit_slots``).
        ``out``: where the ids go, int32 ``[rows]``, on the device or in pinned host memory (the
        kernel then writes them there itself and the host only waits for its end).
        ``suppress``: pairs (row, token) whose logit becomes -inf. ``allowed``: per row ``None`` or
        the only tokens the row may choose. Both change ``logits`` in place. Returns int32 ids and
        fp32 log-probabilities (or ``None``), both on the device.
        """
        rows = logits.shape[0]
        if not (len(temperatures) == len(top_ps) == len(request_seeds) == len(token_indices) == rows):
            raise ValueError("sampling parameters must have one entry per row of logits")
        slots_on_device = None
        if isinstance(slots, torch.Tensor):
            slots_on_device, slots = self._device_slots(slots, rows), None
        if slots is not None and (self.pending is None or len(slots) != rows):
            raise ValueError("slots need a pending table and one entry per row of logits")
        if allowed is not None and len(allowed) != rows:
            raise ValueError("allowed needs one entry per row of logits")
        if out is None:
            out = torch.empty(rows, dtype=torch.int32, device=self.device)
        elif out.dtype != torch.int32 or out.numel() != rows or not out.is_contiguous():
            raise ValueError("out must be contiguous int32, one entry per row of logits")
        if rows == 0:
            return out, (torch.empty(0, dtype=torch.float32, device=self.device) if logprobs else None)
        greedy = all(t <= GREEDY_EPS for t in temperatures)
        restrict = allowed is not None and any(a for a in allowed)
        columns: List[np.ndarray] = []
        names: List[str] = []

        def column(name: str, values, dtype) -> None:
            names.append(name)
            columns.append(np.asarray(values, dtype=dtype))

        if slots is not None:
            column("slots", slots, np.int32)
        if suppress:
            column("suppress_rows", [r for r, _ in suppress], np.int32)
            column("suppress_tokens", [t for _, t in suppress], np.int32)
        if restrict:
            starts, flat = [0], []
            for a in allowed:
                flat.extend(sorted(set(int(t) for t in a)) if a else [])
                starts.append(len(flat))
            column("allow_starts", starts, np.int32)
            column("allow_tokens", flat, np.int32)
        if not greedy or logprobs:
            column("temps", temperatures, np.float32)
        if not greedy:
            column("tops", top_ps, np.float32)
            column("keys", [_signed(mix_key(self.seed, s)) for s in request_seeds], np.int64)
            column("counters", token_indices, np.int32)
        arg = dict(zip(names, self._upload(columns))) if columns else {}
        if suppress:
            core.suppress_tokens(logits, arg["suppress_rows"], arg["suppress_tokens"])
        if restrict:
            core.allow_tokens(logits, arg["allow_starts"], arg["allow_tokens"])
        places = slots_on_device if slots_on_device is not None else arg.get("slots")
        pending = self.pending if places is not None else None
        if greedy:
            core.argmax(logits, out, pending, places)
        else:
            core.sample(logits, arg["temps"], arg["tops"], arg["keys"], arg["counters"], out, pending, places)
        chosen = None
        if logprobs:
            chosen = torch.empty(rows, dtype=torch.float32, device=self.device)
            core.token_logprobs(logits, out, arg["temps"], chosen)
        return out, chosen

    def greedy(self, logits: torch.Tensor, out: Optional[torch.Tensor] = None,
               slots: Optional[Sequence[int]] = None) -> torch.Tensor:
        if out is None:
            out = torch.empty(logits.shape[0], dtype=torch.int32, device=self.device)
        if slots is None:
            core.argmax(logits, out)
        elif isinstance(slots, torch.Tensor):
            core.argmax(logits, out, self.pending, self._device_slots(slots, logits.shape[0]))
        else:
            (pending_at,) = self._upload([np.asarray(slots, dtype=np.int32)])
            core.argmax(logits, out, self.pending, pending_at)
        return out

    def _device_slots(self, slots: torch.Tensor, rows: int) -> torch.Tensor:
        here = torch.device(self.device)
        same = slots.device.type == here.type and (here.index is None or slots.device.index == here.index)
        if slots.dtype != torch.int32 or not same or slots.numel() != rows or not slots.is_contiguous():
            raise ValueError("slots on the device must be contiguous int32, one per row of logits")
        if self.pending is None:
            raise ValueError("slots need a pending table")
        return slots
