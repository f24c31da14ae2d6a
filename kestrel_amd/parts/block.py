"""A block: a mixer, a feed-forward and their norm(s) in one of the known arrangements."""

from __future__ import annotations

from typing import Callable, Dict, Optional

import torch

from .base import LayerCache, Part, SideLinear, build_part
from .specs import LayerSpec, ParamSpec


def _parallel_few_rows(block: "Block", x, batch, cache, normed, then, handed) -> bool:
    """The parallel block for a few bf16 rows in three launches: norm + both first linears, the
    mixer's core, both last linears + residual. Needs a mixer and a feed-forward that offer their
    stages (``input_projection`` / ``output_projection``); returns ``False`` otherwise.
    ``normed``: the block's norm of ``x``, where the block before has computed it; ``then``: the norm
    the next block starts with, which the last launch computes as well where it pays (``handed``, a
    list, then gets the normalised rows)."""
    from ..ops import fast
    from ..ops.linear import linear

    n = x.shape[0]
    if block.dtype != torch.bfloat16 or n > fast.SKINNY_MAX_ROWS:
        return False
    m_in, f_in = block.mixer.input_projection(), block.feed_forward.input_projection()
    m_out, f_out = block.mixer.output_projection(), block.feed_forward.output_projection()
    if m_in is None or f_in is None or m_out is None or f_out is None:
        return False
    ws = batch.workspace
    projected = ws.get("block.mixer_in", (n, m_in[2]), block.dtype)
    hidden = ws.get("block.ff_hidden", (n, f_in[2]), block.dtype)
    norm = block.norm
    fused = False
    beside = None
    if normed is not None:
        fused = fast.linear_two_outputs(normed, m_in[0], m_in[1], projected, 0, f_in[0], f_in[1], hidden, f_in[3])
    ln = norm.layernorm_operands()            # (a norm of another form is run through its own forward below)
    if not fused and fast.FUSE_LAYERNORM_PROLOGUE and ln is not None:
        # the feed-forward's first linear goes into the mixer's launch where the mixer takes it (the
        # launch of the mixer's first linear then leaves the normalised rows for it), else into the
        # launch of the mixer's first linear
        h = ws.get("block.h", tuple(x.shape), block.dtype)
        job = SideLinear(h, f_in[0], f_in[1], hidden, f_in[3])
        if block.mixer.takes_beside(job, batch, cache) and \
                fast.layernorm_linear(x, *ln, m_in[0], m_in[1], projected, 0, store=h):
            fused, beside = True, job
        else:
            fused = fast.layernorm_linear(x, *ln, m_in[0], m_in[1], projected, 0, f_in[0], f_in[1], hidden, f_in[3])
    if not fused:
        h = ws.get("block.h", tuple(x.shape), block.dtype)
        norm.forward(x, h)
        if not fast.linear_two_outputs(h, m_in[0], m_in[1], projected, 0, f_in[0], f_in[1], hidden, f_in[3]):
            linear(h, m_in[0], m_in[1], projected)
            linear(h, f_in[0], f_in[1], hidden, act=f_in[3])
    mixed = block.mixer.attend(projected, batch, cache, beside) if beside is not None \
        else block.mixer.attend(projected, batch, cache)
    # More rows than the next block's first launch normalises by itself, or a last launch of this block that
    # ends in a kernel that finishes whole rows anyway: the next block's norm is computed here, by that
    # kernel, instead of in a launch or a prologue of its own (9 to 16 rows of 2048: 1 to 2 % of a step;
    # rows of 2560, which leave the prologue's kernel no registers for a third strip of weights in flight, from
    # 5 rows on: 3 to 4 %).
    handing = n > fast.SKINNY_LN_MAX_ROWS or fast.pair_finishes_rows(n, x.shape[1])
    then_ln = then.layernorm_operands() if then is not None and handing else None
    if then_ln is not None:
        rows = ws.get("block.handed", tuple(x.shape), block.dtype)
        if fast.linear_pair_accumulate(mixed, m_out[0], m_out[1], hidden, f_out[0], f_out[1], x,
                                       then_norm=(*then_ln, rows)):
            handed.append(rows)
            return True
    if not fast.linear_pair_accumulate(mixed, m_out[0], m_out[1], hidden, f_out[0], f_out[1], x):
        linear(mixed, m_out[0], m_out[1], x, accumulate=True)
        linear(hidden, f_out[0], f_out[1], x, accumulate=True)
    return True


def _parallel(block: "Block", x, batch, cache, normed=None, then=None):
    """``x + mixer(norm(x)) + ff(norm(x))``: both branches read the same normalised input.

    Reference: ``kestrel/models/moondream/text.py:222-275``.
    """
    handed = []
    if _parallel_few_rows(block, x, batch, cache, normed, then, handed):
        return handed[0] if handed else None
    h = normed
    if h is None:
        h = batch.workspace.get("block.h", tuple(x.shape), block.dtype)
        block.norm.forward(x, h)
    block.mixer.forward(h, batch, cache, x)
    block.feed_forward.forward(h, batch, x)
    return None


_parallel.hands_over = True


def _sequential(block: "Block", x, batch, cache) -> None:
    """``x += mixer(norm(x)); x += ff(norm2(x))``."""
    h = batch.workspace.get("block.h", tuple(x.shape), block.dtype)
    block.norm.forward(x, h)
    block.mixer.forward(h, batch, cache, x)
    block.norm2.forward(x, h)
    block.feed_forward.forward(h, batch, x)


ARRANGEMENTS: Dict[str, Callable] = {"parallel": _parallel, "sequential": _sequential}


def register_arrangement(name: str, fn: Callable) -> None:
    """``fn(block, x, batch, cache)`` updates the fp32 residual ``x`` in place. A function with the
    attribute ``hands_over = True`` is called as ``fn(block, x, batch, cache, normed=, then=)``:
    ``normed`` is ``block.norm`` of ``x`` if the block before has computed it (else ``None``), ``then``
    the first norm of the block that follows (or ``None``); it may return that norm of its result, or
    ``None``."""
    ARRANGEMENTS[name] = fn


class Block:
    """Parts of one layer, built from its specification through the registries."""

    def __init__(self, spec: LayerSpec) -> None:
        if spec.arrangement not in ARRANGEMENTS:
            raise ValueError(f"unknown arrangement {spec.arrangement!r}; known: {', '.join(sorted(ARRANGEMENTS))}")
        self.spec = spec
        self.norm = build_part("norm", spec.norm)
        self.norm2 = build_part("norm", spec.norm2) if spec.norm2 is not None else None
        if spec.arrangement == "sequential" and self.norm2 is None:
            raise ValueError("the sequential arrangement needs norm2")
        self.mixer = build_part("mixer", spec.mixer)
        self.feed_forward = build_part("feed_forward", spec.feed_forward)
        self.dtype: Optional[torch.dtype] = None
        self._run = ARRANGEMENTS[spec.arrangement]

    def parts(self) -> Dict[str, Part]:
        out = {"norm": self.norm, "mixer": self.mixer, "feed_forward": self.feed_forward}
        if self.norm2 is not None:
            out["norm2"] = self.norm2
        return out

    def params(self) -> Dict[str, ParamSpec]:
        """Checkpoint tensor name -> spec, for every tensor of this layer."""
        out = {}
        for part_name, part in self.parts().items():
            for local, pspec in part.params().items():
                key = f"{part_name}.{local}"
                if key not in self.spec.names:
                    raise ValueError(f"the architecture names no tensor for {key!r}")
                out[self.spec.names[key]] = pspec
        return out

    def bind(self, tensors: Dict[str, torch.Tensor], dtype, device) -> None:
        self.dtype = dtype
        for part_name, part in self.parts().items():
            local = {name: tensors[self.spec.names[f"{part_name}.{name}"]] for name in part.params()}
            part.bind(local, dtype, device)

    def forward(self, x: torch.Tensor, batch, cache: LayerCache, normed: Optional[torch.Tensor] = None,
                then: Optional[Part] = None) -> Optional[torch.Tensor]:
        """Updates the fp32 residual ``x`` in place. ``normed``: this block's first norm of ``x``, if the
        block before has computed it; ``then``: the first norm of the block that follows. Returns that
        norm of the result where the block's last launch computed it, else ``None``."""
        if getattr(self._run, "hands_over", False):
            return self._run(self, x, batch, cache, normed=normed, then=then)
        self._run(self, x, batch, cache)
        return None
