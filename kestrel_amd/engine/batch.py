"""The packed batch of one step as the parts see it, and the scratch memory they share."""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Optional, Tuple

import torch


class Workspace:
    """Named scratch tensors that live as long as the engine.

    ``get(name, shape, dtype)`` returns a view of a persistent buffer, grown on demand;
    the same name gives the same memory in every step, so a captured HIP graph can be
    replayed. ``freeze()`` forbids further growth (addresses must not change any more).
    """

    def __init__(self, device: torch.device) -> None:
        self.device = device
        self._buffers: Dict[Tuple[str, torch.dtype], torch.Tensor] = {}
        self._frozen = False

    def freeze(self) -> None:
        self._frozen = True

    def get(self, name: str, shape: Tuple[int, ...], dtype: torch.dtype) -> torch.Tensor:
        count = 1
        for s in shape:
            count *= int(s)
        key = (name, dtype)
        buf = self._buffers.get(key)
        if buf is None or buf.numel() < count:
            if self._frozen:
                raise RuntimeError(f"workspace {name!r} would have to grow to {count} elements after freeze()")
            buf = torch.empty(max(count, 1), dtype=dtype, device=self.device)
            self._buffers[key] = buf
        return buf[:count].view(*shape)

    def bytes(self) -> int:
        return sum(b.numel() * b.element_size() for b in self._buffers.values())


@dataclass
class GroupBatch:
    """Per cache group: where this step's tokens live and what they may read."""

    block_table: torch.Tensor           # int32 [rows, max_pages]
    slots: torch.Tensor                 # int32 [tokens]: page * page_size + offset
    kv_lo: Optional[torch.Tensor]       # int32 [tokens] first visible key, or None for 0
    page_size: int = 0


@dataclass
class StepBatch:
    """One step: ``n_tokens`` packed tokens of ``n_rows`` requests, on the device.

    Token ``t`` belongs to row ``token_row[t]``, stands at ``positions[t]`` and sees the
    keys ``[kv_lo[t], kv_hi[t])`` of its row. ``row_slot[r]`` is the request's slot in the
    per-request state tensors. ``logit_rows`` names the tokens whose logits are wanted.
    """

    n_tokens: int
    n_rows: int
    token_ids: torch.Tensor             # int32 [tokens], -1 where an embedding is given
    positions: torch.Tensor             # int32 [tokens]: the token's place in its sequence (and in the cache)
    token_row: torch.Tensor             # int32 [tokens]
    kv_hi: torch.Tensor                 # int32 [tokens]
    row_slot: torch.Tensor              # int32 [rows]
    cu_q: torch.Tensor                  # int32 [rows + 1]
    kv_len: torch.Tensor                # int32 [rows]: keys held after this step
    logit_rows: torch.Tensor            # int32 [wanted]
    logit_slot: torch.Tensor            # int32 [wanted]: the slot of the request a row of logits belongs to (-1: a padding row)
    groups: Dict[int, GroupBatch]
    workspace: Workspace
    # per size of block that a mixer's kernel asked for: (int32 [blocks] row of each block of that
    # many queries of one row, int32 [blocks] its first token), the blocks that see the most keys first
    query_blocks: Dict[int, Tuple[torch.Tensor, torch.Tensor]] = field(default_factory=dict)
    # (int32 [runs] first token, int32 [runs] count): the tokens cut into runs that fill one page of their row in
    # order, and runs of up to a page's worth of other tokens (for the kernels that write the cache by pages)
    page_runs: Optional[Tuple[torch.Tensor, torch.Tensor]] = None
    # int32 [tokens, axes] where a position encoding of the model takes more than one number per token
    position_axes: Optional[torch.Tensor] = None
    pending: Optional[torch.Tensor] = None        # int32 device table: an id <= -2 stands for pending[-2 - id]
    given_embeds: Optional[torch.Tensor] = None   # [m, dim]
    given_rows: Optional[torch.Tensor] = None     # int32 [m] token indices they go to
    # facts known on the host, for choosing kernels
    max_q: int = 1
    max_kv: int = 1
    decode_only: bool = False
    causal_only: bool = True            # no token sees past its own position
    wants_every_token: bool = False     # ``logit_rows`` is 0, 1, ..., n_tokens - 1: every token's logits, in order
    host: dict = field(default_factory=dict)
