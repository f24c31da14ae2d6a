"""Linear layers: chooses the kernel by operand types and by the number of rows."""

from __future__ import annotations

from typing import Optional

import torch

from . import core

# The codes of ``KaAct`` in csrc/ka_common.h, which is where a further activation is added (every
# linear kernel applies them through the same two functions there).
ACT_NONE, ACT_GELU_TANH, ACT_RELU, ACT_SILU = 0, 1, 2, 3
_ACTIVATIONS = {None: ACT_NONE, "none": ACT_NONE, "gelu_tanh": ACT_GELU_TANH, "relu": ACT_RELU, "silu": ACT_SILU}

# Added to an activation's code: the linear is gated (``KA_ACT_GATED`` in csrc/ka_common.h): weight rows
# 2j and 2j + 1 are the gate's and the value's of output j, and ``out[:, j] = act(gate sum) * value sum``.
ACT_GATED = 0x100

# Rows up to which the weight-streaming kernel is used instead of the tiled MFMA one.
SKINNY_MAX_ROWS = 64


def activation_code(name: Optional[str]) -> int:
    if name not in _ACTIVATIONS:
        raise ValueError(f"unknown activation {name!r}; known: {', '.join(sorted(k for k in _ACTIVATIONS if k))}")
    return _ACTIVATIONS[name]


def outputs_of(n: int, act: int) -> int:
    """Columns that a linear of ``n`` weight rows writes: half of them if it is gated."""
    return n // 2 if act & ACT_GATED else n


def pair_rows(gate: torch.Tensor, value: torch.Tensor) -> torch.Tensor:
    """The weights (or biases) of a gated linear as its kernels take them: row ``2j`` is the gate's row
    ``j``, row ``2j + 1`` the value's. Done once, when the weights are bound."""
    if gate.shape != value.shape:
        raise ValueError(f"gate {tuple(gate.shape)} and value {tuple(value.shape)} must have one shape")
    return torch.stack([gate, value], dim=1).reshape(2 * gate.shape[0], *gate.shape[1:]).contiguous()


def linear_gated(a: torch.Tensor, weight_pairs: torch.Tensor, bias_pairs: Optional[torch.Tensor], out: torch.Tensor,
                 act: int) -> None:
    """``out = act(a @ gate.T + gate_bias) * (a @ value.T + value_bias)`` in one pass over ``a``, the product of
    the pair taken in the epilogue of the linear's kernel: ``weight_pairs`` ``[2 n, k]`` and ``bias_pairs`` ``[2 n]``
    are ``pair_rows(gate, value)``, ``out`` is ``[m, n]``. ``act``: an activation's code."""
    linear(a, weight_pairs, bias_pairs, out, act=act | ACT_GATED)


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
