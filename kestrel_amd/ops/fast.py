"""Python faces of the bf16 MFMA kernels (library ``fast``).

Each function returns ``False`` when the kernels do not cover the operands (the
caller then takes the generic kernel) and raises when they do but the call fails.
"""

from __future__ import annotations

from typing import Optional

import torch


def linear_bf16(a, weight, bias, out, act, accumulate) -> bool:
    return False


def attention_bf16(q, k_cache, v_cache, block_table, token_row, kv_lo, kv_hi, out, scale, n_heads, n_kv_heads,
                   head_dim, batch) -> bool:
    return False
