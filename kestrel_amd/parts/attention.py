"""Attention over the paged cache with a fused q|k|v projection."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..ops import core
from ..ops.attention import paged_attention
from ..ops.linear import linear
from .base import LayerCache, Mixer, build_part, register_mixer
from .specs import AttentionSpec, CacheSpec, ParamSpec


class PagedAttention(Mixer):
    """``proj(softmax(q k^T scale + mask) v)`` with grouped kv heads.

    One linear gives ``[q (H hd) | k (Hkv hd) | v (Hkv hd)]`` per token
    (``kestrel/models/moondream/text.py:101-121``); the position encoding is applied to
    q and k, k and v go into the paged cache first and attention then reads the cache
    (``text.py:123-135``); query head ``h`` reads kv head ``h // (H / Hkv)``; the scale is
    ``hd ** -0.5`` unless given (``text.py:158-185``); the output projection adds into the
    residual (``text.py:187-193``). Which keys a token sees comes with the batch
    (``kv_hi``, and the group's ``kv_lo`` for a window).

    Positions: the part built from ``spec.position`` is asked for a ``Rotation`` (a cos|sin table
    and the pairing of channels); ``None`` means q and k go into attention as they are. Nothing
    else is understood here: an encoding that needs more (several axes, a learned table added to
    the input) is refused when the weights are bound, not silently turned the rotary way.
    """

    replays_every_step = True

    def __init__(self, spec: AttentionSpec) -> None:
        super().__init__(spec)
        if spec.n_heads % spec.n_kv_heads:
            raise ValueError(f"{spec.n_heads} query heads cannot share {spec.n_kv_heads} kv heads")
        self.position = build_part("position", spec.position)
        self.scale = float(spec.scale) if spec.scale is not None else float(spec.head_dim) ** -0.5
        self.q_dim = spec.n_heads * spec.head_dim
        self.kv_dim = spec.n_kv_heads * spec.head_dim
        self.qkv_dim = self.q_dim + 2 * self.kv_dim
        self.qkv_weight = self.qkv_bias = self.proj_weight = self.proj_bias = None
        self.dtype: Optional[torch.dtype] = None
        self._table = None
        self._pairing = "halves"

    def params(self) -> Dict[str, ParamSpec]:
        spec = self.spec
        out = {"qkv.weight": ParamSpec((self.qkv_dim, spec.dim)), "proj.weight": ParamSpec((spec.dim, self.q_dim))}
        if spec.bias:
            out["qkv.bias"] = ParamSpec((self.qkv_dim,), "vector", "bias")
            out["proj.bias"] = ParamSpec((spec.dim,), "vector", "bias")
        return out

    def cache_spec(self) -> CacheSpec:
        return CacheSpec(self.spec.n_kv_heads, self.spec.head_dim, self.spec.window)

    def bind(self, tensors, dtype, device) -> None:
        spec = self.spec
        self.dtype = dtype
        self.qkv_weight = tensors["qkv.weight"].to(device).contiguous()
        self.proj_weight = tensors["proj.weight"].to(device).contiguous()
        if self.spec.bias:
            self.qkv_bias = tensors["qkv.bias"].to(device=device, dtype=torch.float32).contiguous()
            self.proj_bias = tensors["proj.bias"].to(device=device, dtype=torch.float32).contiguous()
        if int(getattr(self.position, "axes", 1)) != 1:
            raise ValueError(f"attention rotates by a token's place in the sequence; the position encoding "
                             f"{getattr(spec.position, 'kind', '?')!r} takes {self.position.axes} numbers per token")
        rotation = self.position.rotation(device)
        if rotation is None and callable(getattr(self.position, "table", None)) and self.position.table(device) is not None:
            raise ValueError(f"the position encoding {getattr(spec.position, 'kind', '?')!r} holds a table but offers no "
                             f"rotation(): attention would not know which channels to pair")
        if rotation is not None:
            table = rotation.table
            if rotation.pairing not in core.ROTARY_PAIRINGS:
                raise ValueError(f"attention cannot apply a rotation with pairing {rotation.pairing!r}; known: "
                                 f"{', '.join(sorted(core.ROTARY_PAIRINGS))}")
            if table.dtype != torch.float32 or table.dim() != 2 or table.shape[1] % 2 or table.shape[1] > self.spec.head_dim:
                raise ValueError(f"a rotation's table must be fp32 [positions, R] with R even and at most the head size "
                                 f"{self.spec.head_dim}, got {tuple(table.shape)} {table.dtype}")
            self._table, self._pairing = table.to(device).contiguous(), rotation.pairing
        else:
            self._table, self._pairing = None, "halves"

    def query_tile(self) -> Optional[int]:
        if self.dtype != torch.bfloat16:
            return None                     # the generic kernel takes tokens one by one
        from ..ops import fast
        return fast.prefill_query_block(self.spec.head_dim)

    # The three stages are also offered one by one, so that a block may fuse the first with its
    # norm and the last with its feed-forward (see ``Mixer.input_projection``).
    def input_projection(self):
        return self.qkv_weight, self.qkv_bias, self.qkv_dim

    def output_projection(self):
        return self.proj_weight, self.proj_bias

    def _decodes_fused(self, batch, cache: LayerCache) -> bool:
        """One token per row in bf16 with a rotation by halves: the decode kernel then rotates q and
        k and stores k and v itself."""
        return self.dtype == torch.bfloat16 and batch.decode_only and cache.writes and self._table is not None \
            and self._pairing == "halves"          # the MFMA-path kernels turn halves; the generic one any pairing

    def takes_beside(self, job, batch, cache: LayerCache) -> bool:
        if not self._decodes_fused(batch, cache):
            return False
        from ..ops import fast
        return fast.attention_decode_takes(job, job.a.shape[0], self.spec.n_heads, self.spec.head_dim, cache.k.shape[2],
                                           batch.max_kv)

    def attend(self, qkv, batch, cache: LayerCache, beside=None):
        """Position encoding, cache write and attention on the projected input ``[n, q|k|v]``."""
        spec = self.spec
        n = qkv.shape[0]
        group = batch.groups[cache.group]
        out = batch.workspace.get("attn.out", (n, self.q_dim), self.dtype)
        halves = self._pairing == "halves"
        if qkv.dtype == torch.bfloat16 and self._decodes_fused(batch, cache):
            from ..ops import fast
            k_new = qkv[:, self.q_dim:self.q_dim + self.kv_dim]
            v_new = qkv[:, self.q_dim + self.kv_dim:]
            operands = (qkv, cache.k, cache.v, group.block_table, batch.token_row, group.kv_lo, batch.kv_hi, out,
                        self.scale, spec.n_heads, spec.n_kv_heads, spec.head_dim, batch)
            fuse = (k_new, v_new, self._table, group.slots)
            if beside is not None and fast.attention_decode_bf16(*operands, fuse=fuse, beside=beside):
                return out
            if beside is not None:
                self._alone(beside)
                beside = None
            if fast.attention_decode_bf16(*operands, fuse=fuse):
                return out
        if beside is not None:
            self._alone(beside)
        slots = group.slots if cache.writes else None
        done = False
        if qkv.dtype == torch.bfloat16 and halves:
            from ..ops import fast
            done = fast.rope_cache_bf16(qkv, batch.positions, slots, self._table, cache.k, cache.v, spec.n_heads,
                                        spec.n_kv_heads, spec.head_dim, group.page_size,
                                        runs=getattr(batch, "page_runs", None))
        if not done:
            core.rope_cache(qkv, batch.positions, slots, self._table, cache.k, cache.v, spec.n_heads, spec.n_kv_heads,
                            spec.head_dim, group.page_size, self._pairing)
        paged_attention(qkv, cache.k, cache.v, group.block_table, batch.token_row, group.kv_lo, batch.kv_hi, out,
                        self.scale, spec.n_heads, spec.n_kv_heads, spec.head_dim, batch)
        return out

    @staticmethod
    def _alone(job) -> None:
        """A job that was promised a place in the attention launch and did not get one after all."""
        linear(job.a, job.weight, job.bias, job.out, act=job.act)

    def forward(self, h, batch, cache: LayerCache, residual) -> None:
        qkv = batch.workspace.get("attn.qkv", (h.shape[0], self.qkv_dim), self.dtype)
        linear(h, self.qkv_weight, self.qkv_bias, qkv)
        out = self.attend(qkv, batch, cache)
        linear(out, self.proj_weight, self.proj_bias, residual, accumulate=True)


register_mixer("attention", PagedAttention)
