"""Seeded random weights: a model folder (config.json, model.safetensors) from a configuration.

Every tensor is drawn from a generator seeded by (seed, tensor name), so its values do
not depend on the other tensors or on their order, and a float32 run and a bfloat16
run of the same folder start from the same stored values.
"""

from __future__ import annotations

import hashlib
import json
from dataclasses import dataclass
from pathlib import Path
from typing import Any, Dict, Optional

import torch
from safetensors.torch import save_file

from ..config.registry import resolve
from ..parts.specs import ParamSpec

_STORE = {"bfloat16": torch.bfloat16, "float32": torch.float32}


@dataclass(frozen=True)
class InitRecipe:
    """Standard deviations: ``std`` of matrices, ``bias_std`` of biases (``None``: ``std``),
    ``gain_std`` of norm gains around 1, ``shift_std`` of norm shifts around 0."""

    std: float = 0.02
    bias_std: Optional[float] = None
    gain_std: float = 0.0
    shift_std: float = 0.0


def _seed_of(seed: int, name: str) -> int:
    digest = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return int.from_bytes(digest[:8], "little") & (2 ** 63 - 1)


def random_tensor(name: str, spec: ParamSpec, seed: int, recipe: InitRecipe, device="cpu") -> torch.Tensor:
    """One tensor of the recipe, in float32."""
    gen = torch.Generator(device=device)
    gen.manual_seed(_seed_of(seed, name))
    if spec.role == "table":
        raise ValueError(f"{name}: no random recipe for integer tables")
    noise = torch.randn(tuple(spec.shape), generator=gen, dtype=torch.float32, device=device)
    if spec.init == "normal":
        return noise * recipe.std
    if spec.init == "bias":
        return noise * (recipe.std if recipe.bias_std is None else recipe.bias_std)
    if spec.init == "gain":
        return 1.0 + noise * recipe.gain_std
    if spec.init == "shift":
        return noise * recipe.shift_std
    raise ValueError(f"{name}: unknown init {spec.init!r}")


def random_tensors(expected: Dict[str, ParamSpec], seed: int, recipe: InitRecipe = InitRecipe(),
                   store_dtype: torch.dtype = torch.bfloat16, device="cpu") -> Dict[str, torch.Tensor]:
    return {name: random_tensor(name, spec, seed, recipe, device).to(store_dtype) for name, spec in expected.items()}


def write_random_model(folder, config: Dict[str, Any], seed: int, recipe: InitRecipe = InitRecipe(),
                       store_dtype: str = "bfloat16", model: Optional[str] = None) -> Path:
    """Write ``config.json`` and ``model.safetensors`` for ``config`` into ``folder``."""
    from ..models.decoder import DecoderModel

    if store_dtype not in _STORE:
        raise ValueError(f"store_dtype must be one of {sorted(_STORE)}")
    spec = resolve(config, model)
    typed = spec.read_config(config)
    plan = spec.build_plan(typed)
    expected = DecoderModel(plan).params()
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    tensors = random_tensors(expected, seed, recipe, _STORE[store_dtype])
    prefix = spec.tensor_prefixes[-1] if spec.extras.get("write_prefixed") else ""
    save_file({prefix + k: v.contiguous() for k, v in tensors.items()}, str(folder / spec.filename))
    written = typed.to_dict() if hasattr(typed, "to_dict") else dict(config)
    written.setdefault("model", spec.name)
    with open(folder / "config.json", "w") as handle:
        json.dump(written, handle, indent=2)
    return folder
