"""Rotary position encoding on the first ``rotary_dim`` channels of each head."""

from __future__ import annotations

from typing import Optional

import torch

from .base import PositionEncoding, Rotation, register_position
from .specs import PositionSpec


class NeoxRotary(PositionEncoding):
    """Non-interleaved rotation: channel ``i`` pairs with ``i + rotary_dim / 2``.

    Table row ``p`` = ``[cos(p f_0), .., cos(p f_{R/2-1}), sin(p f_0), ..]`` with
    ``f_i = theta ** (-2 i / R)``, all in fp32
    (``kestrel/models/moondream/rope.py:6-32``; applied at ``text.py:123-125``).
    """

    replays_every_step = True

    def __init__(self, spec: PositionSpec) -> None:
        super().__init__(spec)
        if spec.rotary_dim % 2:
            raise ValueError(f"rotary_dim {spec.rotary_dim} must be even")
        if spec.rotary_dim and spec.max_positions <= 0:
            raise ValueError("a rotary encoding needs max_positions")
        self._table: Optional[torch.Tensor] = None

    def rotation(self, device: torch.device) -> Optional[Rotation]:
        table = self.table(device)
        return None if table is None else Rotation(table, "halves")

    def table(self, device: torch.device) -> Optional[torch.Tensor]:
        spec = self.spec
        if spec.rotary_dim == 0:
            return None
        if self._table is None or self._table.device != device:
            exponents = torch.arange(0, spec.rotary_dim, 2, dtype=torch.float32) / float(spec.rotary_dim)
            inv_freq = 1.0 / (float(spec.theta) ** exponents)
            angles = torch.arange(spec.max_positions, dtype=torch.float32).unsqueeze(1) * inv_freq.unsqueeze(0)
            self._table = torch.cat([torch.cos(angles), torch.sin(angles)], dim=-1).contiguous().to(device)
        return self._table


class NoPosition(PositionEncoding):
    """Encodes nothing (a mixer whose order comes from elsewhere)."""

    replays_every_step = True


register_position("rotary_neox", NeoxRotary)
register_position("none", NoPosition)
