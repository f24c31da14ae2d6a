"""Linear layers: chooses the kernel by operand types and by the number of rows."""

from __future__ import annotations

from typing import Optional

import torch

from . import core

# The codes of ``KaAct`` in csrc/ka_common.h, which is where a further activation is added (every
# linear kernel applies them through the same two functions there).
ACT_NONE, ACT_GELU_TANH, ACT_RELU, ACT_SILU = 0, 1, 2, 3
_ACTIVATIONS = {None: ACT_NONE, "none": ACT_NONE, "gelu_tanh": ACT_GELU_TANH, "relu": ACT_RELU, "silu": ACT_SILU}

# Rows up to which the weight-streaming kernel is used instead of the tiled MFMA one.
SKINNY_MAX_ROWS = 64


def activation_code(name: Optional[str]) -> int:
    if name not in _ACTIVATIONS:
        raise ValueError(f"unknown activation {name!r}; known: {', '.join(sorted(k for k in _ACTIVATIONS if k))}")
    return _ACTIVATIONS[name]


def linear(a: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
           act: int = ACT_NONE, accumulate: bool = False) -> None:
    """``out = act(a @ weight.T + bias)``, or ``out += a @ weight.T + bias`` into fp32 ``out``.

    bf16 x bf16 goes to the MFMA kernels (a weight-streaming one for few rows, a tiled
    one otherwise); every other mix of types, fp32 above all, to the plain fp32 FMA kernel.
    """
    if a.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16:
        from . import fast
        if fast.linear_bf16(a, weight, bias, out, act, accumulate):
            return
    core.linear_generic(a, weight, bias, out, act, accumulate)
