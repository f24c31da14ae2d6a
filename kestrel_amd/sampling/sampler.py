"""Greedy and temperature / top-p selection of the next token on the GPU.

Reference: ``kestrel/scheduler/scheduler.py:2929-2993``: all rows greedy -> argmax;
otherwise per-row temperature and top-p, rows with temperature <= 1e-6 greedy
(``scheduler.py:55``). The reference draws from one device generator seeded from
``torch.seed()`` (``scheduler.py:404-405``) and is not reproducible; here every draw comes
from a counter-based generator keyed by (engine seed, request seed, index of the token),
so a request's tokens do not depend on what else is in the batch.
"""

from __future__ import annotations

from typing import List, Optional, Sequence

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
    def __init__(self, device: torch.device, seed: int = 0) -> None:
        self.device, self.seed = device, seed

    def sample(self, logits: torch.Tensor, temperatures: Sequence[float], top_ps: Sequence[float],
               request_seeds: Sequence[int], token_indices: Sequence[int]) -> torch.Tensor:
        """One token id per row of fp32 ``logits``; int32 on the device."""
        rows = logits.shape[0]
        if not (len(temperatures) == len(top_ps) == len(request_seeds) == len(token_indices) == rows):
            raise ValueError("sampling parameters must have one entry per row of logits")
        out = torch.empty(rows, dtype=torch.int32, device=self.device)
        if rows == 0:
            return out
        if all(t <= GREEDY_EPS for t in temperatures):
            core.argmax(logits, out)
            return out
        temps = torch.tensor(list(temperatures), dtype=torch.float32).to(self.device)
        tops = torch.tensor(list(top_ps), dtype=torch.float32).to(self.device)
        keys = torch.tensor([_signed(mix_key(self.seed, s)) for s in request_seeds], dtype=torch.int64).to(self.device)
        counters = torch.tensor(list(token_indices), dtype=torch.int32).to(self.device)
        core.sample(logits, temps, tops, keys, counters, out)
        return out

    def greedy(self, logits: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        if out is None:
            out = torch.empty(logits.shape[0], dtype=torch.int32, device=self.device)
        core.argmax(logits, out)
        return out
