"""LayerNorm with gain and optional shift; statistics in fp32."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..ops import core
from .base import Norm, register_norm
from .specs import NormSpec, ParamSpec


class LayerNorm(Norm):
    """``(x - mean) / sqrt(var + eps) * weight + bias`` over the last axis (biased variance).

    Reference: ``kestrel/models/moondream/layers.py:40-44`` (the kernel is called without
    eps; the modules are ``nn.LayerNorm(dim)``, ``text.py:311,359``).
    """

    replays_every_step = True

    def __init__(self, spec: NormSpec) -> None:
        super().__init__(spec)
        self.weight: Optional[torch.Tensor] = None
        self.bias: Optional[torch.Tensor] = None

    def params(self) -> Dict[str, ParamSpec]:
        out = {"weight": ParamSpec((self.spec.dim,), "vector", "gain")}
        if self.spec.bias:
            out["bias"] = ParamSpec((self.spec.dim,), "vector", "shift")
        return out

    def bind(self, tensors, dtype, device) -> None:
        # Gains and shifts are read as fp32 by the kernel whatever they are stored in.
        self.weight = tensors["weight"].to(device=device, dtype=torch.float32).contiguous()
        self.bias = tensors["bias"].to(device=device, dtype=torch.float32).contiguous() if self.spec.bias else None

    def forward(self, x, out, rows=None) -> None:
        core.layernorm(x, self.weight, self.bias, self.spec.eps, out, rows)

    def layernorm_operands(self):
        return self.weight, self.bias, float(self.spec.eps)


register_norm("layernorm", LayerNorm)
