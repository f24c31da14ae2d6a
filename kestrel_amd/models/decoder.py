"""The generic decoder: embedding, the scheduled blocks, final norm and head.

It is put together from a ``ModelPlan`` alone and knows no architecture. The order of
execution is the plan's ``schedule``: a list of runs, each naming a layer (a layer may be
named twice and then shares its weights) and optionally an earlier run whose cache it
reads instead of keeping one.
"""

from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..ops import core
from ..ops.linear import linear
from ..parts.base import LayerCache, build_part
from ..parts.block import Block
from ..parts.specs import ModelPlan, ParamSpec


class DecoderModel:
    def __init__(self, plan: ModelPlan) -> None:
        self.plan = plan
        self.blocks: List[Block] = [Block(layer) for layer in plan.layers]
        self.final_norm = build_part("norm", plan.final_norm)
        self.position = build_part("position", plan.position) if plan.position is not None else None
        for index, entry in enumerate(plan.schedule):
            if not 0 <= entry.layer < len(self.blocks):
                raise ValueError(f"schedule entry {index} names layer {entry.layer}, the plan has {len(self.blocks)}")
            if entry.reads_cache_of is not None:
                if not 0 <= entry.reads_cache_of < index:
                    raise ValueError(f"schedule entry {index} must read the cache of an earlier entry")
                if plan.schedule[entry.reads_cache_of].reads_cache_of is not None:
                    raise ValueError(f"schedule entry {index} reads the cache of an entry that keeps none")
        self.embedding: Optional[torch.Tensor] = None
        self.head_weight: Optional[torch.Tensor] = None
        self.head_bias: Optional[torch.Tensor] = None
        self.dtype: Optional[torch.dtype] = None
        self.device: Optional[torch.device] = None

    # ------------------------------------------------------------------ tensors
    def params(self) -> Dict[str, ParamSpec]:
        """Checkpoint tensor name -> shape and role of every tensor the model owns."""
        plan = self.plan
        out = {plan.names["embedding"]: ParamSpec((plan.vocab_size, plan.dim), "matrix", "normal")}
        for block in self.blocks:
            out.update(block.params())
        for local, pspec in self.final_norm.params().items():
            out[plan.names[f"final_norm.{local}"]] = pspec
        if self.position is not None:
            for local, pspec in self.position.params().items():
                out[plan.names[f"position.{local}"]] = pspec
        if not plan.tied_head:
            out[plan.names["head.weight"]] = ParamSpec((plan.vocab_size, plan.dim), "matrix", "normal")
        if plan.head_bias:
            out[plan.names["head.bias"]] = ParamSpec((plan.vocab_size,), "vector", "bias")
        return out

    def bind(self, tensors: Dict[str, torch.Tensor], dtype: torch.dtype, device: torch.device) -> None:
        plan = self.plan
        self.dtype, self.device = dtype, device
        self.embedding = tensors[plan.names["embedding"]].to(device).contiguous()
        for block in self.blocks:
            block.bind(tensors, dtype, device)
        self.final_norm.bind({k: tensors[plan.names[f"final_norm.{k}"]] for k in self.final_norm.params()}, dtype,
                             device)
        if self.position is not None:
            self.position.bind({k: tensors[plan.names[f"position.{k}"]] for k in self.position.params()}, dtype, device)
        self.head_weight = self.embedding if plan.tied_head else tensors[plan.names["head.weight"]].to(device).contiguous()
        if plan.head_bias:
            self.head_bias = tensors[plan.names["head.bias"]].to(device=device, dtype=torch.float32).contiguous()

    # ------------------------------------------------------------------ cache needs
    def cache_needs(self):
        """Per schedule entry: ``(cache_spec or None, state_spec or None, reads_cache_of)``."""
        needs = []
        for entry in self.plan.schedule:
            mixer = self.blocks[entry.layer].mixer
            needs.append((mixer.cache_spec(), mixer.state_spec(), entry.reads_cache_of))
        return needs

    def position_axes(self) -> int:
        """The most numbers any position encoding of the model (its own, or a mixer's) needs per token."""
        parts = [self.position] + [getattr(block.mixer, "position", None) for block in self.blocks]
        return max([1] + [int(getattr(part, "axes", 1)) for part in parts if part is not None])

    def replays_every_step(self) -> bool:
        """Whether steps of every shape may be captured and replayed: every part of the model says so
        (``Part.replays_every_step``)."""
        parts = [self.final_norm, self.position]
        for block in self.blocks:
            parts += list(block.parts().values()) + [getattr(block.mixer, "position", None)]
        return all(bool(getattr(part, "replays_every_step", False)) for part in parts if part is not None)

    def query_tiles(self):
        """Sizes of blocks of queries that the mixers' kernels want listed with a step."""
        return {tile for tile in (block.mixer.query_tile() for block in self.blocks) if tile}

    def _head_with_norm(self, x, batch, logits) -> bool:
        """A few decoded rows, every one of them wanted, in order: the head's launch normalises them itself
        (one launch less a step)."""
        ln = self.final_norm.layernorm_operands()
        if self.dtype != torch.bfloat16 or not batch.decode_only or not getattr(batch, "wants_every_token", False) or ln is None:
            return False
        from ..ops import fast
        return fast.layernorm_linear(x, *ln, self.head_weight, self.head_bias, logits, 0)

    # ------------------------------------------------------------------ forward
    def forward(self, batch, caches: List[LayerCache]) -> torch.Tensor:
        """Run the packed tokens of ``batch``; returns fp32 logits ``[wanted, vocab]``."""
        plan = self.plan
        ws = batch.workspace
        x = ws.get("model.x", (batch.n_tokens, plan.dim), torch.float32)
        core.embed(self.embedding, batch.token_ids, x, batch.pending, plan.embedding_scale)
        if batch.given_embeds is not None:
            core.scatter_rows(batch.given_embeds, batch.given_rows, x)
        if self.position is not None:
            self.position.add_to_embeddings(x, batch)
        handed = None      # the next block's first norm of x, where a block's last launch has computed it
        for index, entry in enumerate(plan.schedule):
            after = plan.schedule[index + 1] if index + 1 < len(plan.schedule) else None
            then = self.blocks[after.layer].norm if after is not None else None
            handed = self.blocks[entry.layer].forward(x, batch, caches[index], normed=handed, then=then)
        wanted = int(batch.logit_rows.numel())
        logits = ws.get("model.logits", (wanted, plan.vocab_size), torch.float32)
        if wanted:
            if not self._head_with_norm(x, batch, logits):
                normed = ws.get("model.head_in", (wanted, plan.dim), self.dtype)
                self.final_norm.forward(x, normed, rows=batch.logit_rows)
                linear(normed, self.head_weight, self.head_bias, logits)
            if plan.logit_scale != 1.0 or plan.logit_softcap is not None:
                core.adjust_logits(logits, plan.logit_scale, plan.logit_softcap)
        return logits
