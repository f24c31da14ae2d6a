"""A block: a mixer, a feed-forward and their norm(s) in one of the known arrangements."""

from __future__ import annotations

from typing import Callable, Dict, Optional

import torch

from .base import LayerCache, Part, build_part
from .specs import LayerSpec, ParamSpec


def _parallel(block: "Block", x, batch, cache) -> None:
    """``x + mixer(norm(x)) + ff(norm(x))``: both branches read the same normalised input.

    Reference: ``kestrel/models/moondream/text.py:222-275``.
    """
    h = batch.workspace.get("block.h", tuple(x.shape), block.dtype)
    block.norm.forward(x, h)
    block.mixer.forward(h, batch, cache, x)
    block.feed_forward.forward(h, batch, x)


def _sequential(block: "Block", x, batch, cache) -> None:
    """``x += mixer(norm(x)); x += ff(norm2(x))``."""
    h = batch.workspace.get("block.h", tuple(x.shape), block.dtype)
    block.norm.forward(x, h)
    block.mixer.forward(h, batch, cache, x)
    block.norm2.forward(x, h)
    block.feed_forward.forward(h, batch, x)


ARRANGEMENTS: Dict[str, Callable] = {"parallel": _parallel, "sequential": _sequential}


def register_arrangement(name: str, fn: Callable) -> None:
    """``fn(block, x, batch, cache)`` updates the fp32 residual ``x`` in place."""
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

    def forward(self, x: torch.Tensor, batch, cache: LayerCache) -> None:
        self._run(self, x, batch, cache)
