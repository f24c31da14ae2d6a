"""Paged attention: chooses between the MFMA kernels and the generic one."""

from __future__ import annotations

from typing import Optional

import torch

from . import core


def paged_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
                    token_row: torch.Tensor, kv_lo: Optional[torch.Tensor], kv_hi: torch.Tensor, out: torch.Tensor,
                    scale: float, n_heads: int, n_kv_heads: int, head_dim: int, batch=None) -> None:
    """Attention of the packed tokens over their rows' cached keys ``[kv_lo, kv_hi)``."""
    if q.dtype == torch.bfloat16:
        from . import fast
        if fast.attention_bf16(q, k_cache, v_cache, block_table, token_row, kv_lo, kv_hi, out, scale, n_heads,
                               n_kv_heads, head_dim, batch):
            return
    core.attention_generic(q, k_cache, v_cache, block_table, token_row, kv_lo, kv_hi, out, scale, n_heads,
                           n_kv_heads, head_dim)
