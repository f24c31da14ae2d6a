"""Dense feed-forward: two linears around an activation."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..ops.linear import activation_code, linear
from .base import FeedForward, register_feed_forward
from .specs import DenseFeedForwardSpec, ParamSpec


class DenseFeedForward(FeedForward):
    """``fc2(act(fc1(h)))`` with biases; the activation runs in the first linear's epilogue.

    Reference: ``kestrel/models/moondream/layers.py:64-121`` (``fc1``, ``F.gelu`` with the
    tanh approximation ``layers.py:30-31``, ``fc2``).
    """

    replays_every_step = True

    def __init__(self, spec: DenseFeedForwardSpec) -> None:
        super().__init__(spec)
        self.act = activation_code(spec.activation)
        self.fc1_weight = self.fc1_bias = self.fc2_weight = self.fc2_bias = None
        self.dtype: Optional[torch.dtype] = None

    def params(self) -> Dict[str, ParamSpec]:
        spec = self.spec
        out = {"fc1.weight": ParamSpec((spec.hidden_dim, spec.dim)), "fc2.weight": ParamSpec((spec.dim, spec.hidden_dim))}
        if spec.bias:
            out["fc1.bias"] = ParamSpec((spec.hidden_dim,), "vector", "bias")
            out["fc2.bias"] = ParamSpec((spec.dim,), "vector", "bias")
        return out

    def bind(self, tensors, dtype, device) -> None:
        self.dtype = dtype
        self.fc1_weight = tensors["fc1.weight"].to(device).contiguous()
        self.fc2_weight = tensors["fc2.weight"].to(device).contiguous()
        if self.spec.bias:
            self.fc1_bias = tensors["fc1.bias"].to(device=device, dtype=torch.float32).contiguous()
            self.fc2_bias = tensors["fc2.bias"].to(device=device, dtype=torch.float32).contiguous()

    def input_projection(self):
        return self.fc1_weight, self.fc1_bias, self.spec.hidden_dim, self.act

    def output_projection(self):
        return self.fc2_weight, self.fc2_bias

    def forward(self, h, batch, residual) -> None:
        hidden = batch.workspace.get("ff.hidden", (h.shape[0], self.spec.hidden_dim), self.dtype)
        linear(h, self.fc1_weight, self.fc1_bias, hidden, act=self.act)
        linear(hidden, self.fc2_weight, self.fc2_bias, residual, accumulate=True)


register_feed_forward("dense", DenseFeedForward)
