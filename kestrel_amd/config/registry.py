"""One registry from an architecture's name to everything the engine needs of it.

An architecture registers a ``ModelSpec``: how to read its ``config.json`` keys into
a typed configuration, and how to turn that into a ``ModelPlan`` (parts, order,
tensor names). The engine, the weight loader, the random-weights writer and the
replay program all go through ``resolve`` and never name an architecture.

Reference: ``kestrel/models/registry.py:23-91`` (``ModelSpec``, ``register``, ``get_spec``,
``known_models``; families register themselves on import,
``kestrel/models/moondream/__init__.py:26-37``).
"""

from __future__ import annotations

import json
from dataclasses import dataclass, field
from pathlib import Path
from typing import Any, Callable, Dict, List, Optional, Tuple


@dataclass(frozen=True)
class ModelSpec:
    """Bootstrap facts of one architecture.

    ``read_config(config_dict) -> typed config``; ``build_plan(typed config) -> ModelPlan``;
    ``aliases``: other names ``config.json`` may use for it (``model_type``,
    ``architectures``); ``claims(config_dict)``: says whether a ``config.json`` without any
    name is this architecture's; ``tensor_prefixes``: prefixes that may stand before the
    plan's tensor names in a checkpoint; ``foreign_prefixes``: tensors of a checkpoint
    that belong to parts outside the text decoder and are passed over.
    """

    name: str
    read_config: Callable[[Dict[str, Any]], Any]
    build_plan: Callable[[Any], Any]
    aliases: Tuple[str, ...] = ()
    claims: Optional[Callable[[Dict[str, Any]], bool]] = None
    filename: str = "model.safetensors"
    tensor_prefixes: Tuple[str, ...] = ("",)
    foreign_prefixes: Tuple[str, ...] = ()
    default_config: Optional[Callable[[], Dict[str, Any]]] = None
    extras: Dict[str, Any] = field(default_factory=dict)


_REGISTRY: Dict[str, ModelSpec] = {}
_ALIASES: Dict[str, str] = {}


def register(spec: ModelSpec) -> None:
    _REGISTRY[spec.name] = spec
    for alias in spec.aliases:
        _ALIASES[alias.lower()] = spec.name


def known_models() -> List[str]:
    _ensure_builtin()
    return sorted(_REGISTRY)


def get_spec(name: str) -> ModelSpec:
    _ensure_builtin()
    key = name if name in _REGISTRY else _ALIASES.get(str(name).lower())
    if key is None or key not in _REGISTRY:
        known = ", ".join(sorted(_REGISTRY))
        raise ValueError(f"Unknown model {name!r}. Known models: {known}")
    return _REGISTRY[key]


def _ensure_builtin() -> None:
    from .. import models  # noqa: F401  (architectures register themselves on import)


def name_in_config(config: Dict[str, Any]) -> Optional[str]:
    """The architecture name a ``config.json`` carries, if any."""
    for key in ("model", "model_type", "architecture"):
        value = config.get(key)
        if isinstance(value, str) and value:
            return value
    archs = config.get("architectures")
    if isinstance(archs, (list, tuple)) and archs and isinstance(archs[0], str):
        return archs[0]
    return None


def resolve(config: Dict[str, Any], model: Optional[str] = None) -> ModelSpec:
    """The architecture of a ``config.json``: by the given name, by the name the file
    carries, or by the one registered architecture that claims its keys."""
    _ensure_builtin()
    if model:
        return get_spec(model)
    named = name_in_config(config)
    if named is not None:
        return get_spec(named)
    claimants = [s for s in _REGISTRY.values() if s.claims is not None and s.claims(config)]
    if len(claimants) == 1:
        return claimants[0]
    known = ", ".join(sorted(_REGISTRY))
    raise ValueError("config.json names no architecture (keys model / model_type / architectures) and "
                     f"{'several' if claimants else 'no'} registered architectures match its keys. Known models: {known}")


def read_model_dir(folder, model: Optional[str] = None):
    """``(spec, typed config, plan)`` of a model folder with a ``config.json``."""
    folder = Path(folder)
    path = folder / "config.json"
    if not path.exists():
        raise FileNotFoundError(f"{path} not found: a model folder holds config.json and model.safetensors")
    with open(path) as handle:
        config = json.load(handle)
    if not isinstance(config, dict):
        raise ValueError(f"{path} must hold a JSON object")
    spec = resolve(config, model)
    typed = spec.read_config(config)
    return spec, typed, spec.build_plan(typed)
