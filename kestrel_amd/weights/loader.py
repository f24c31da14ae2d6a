"""Reads a model's tensors from a safetensors file (or a ``.pt`` checkpoint of tensors) by name
and checks them against the plan.

Tensors are matched by name (an architecture may allow a prefix such as ``model.``),
never by order. Floating tensors stored in 16 bits are held in bfloat16; a tensor
stored in 32 bits stays in 32 bits; integer tables become int32. In a float32 run
every floating tensor is held in float32. Everything that is wrong with a file is
reported at once, in one error.

Reference: ``kestrel/models/moondream/weights.py:48-58`` (safetensors by name),
``:80-110`` (Moondream 2 names, used as stored: fused qkv, ``[out, in]`` linears),
``:545,566`` (``._orig_mod`` stripped from keys), ``:560-566`` (``.pt`` files through
``torch.load(map_location="cpu", weights_only=True, mmap=True)``: nothing in the file is run).
"""

from __future__ import annotations

from pathlib import Path
from typing import Dict, Iterable, List, Optional, Tuple

import torch
from safetensors import safe_open

from ..parts.specs import ParamSpec


class WeightsError(ValueError):
    """The file does not hold the tensors the model needs.

    ``missing``, ``unexpected`` and ``mismatched`` list every offending tensor.
    """

    def __init__(self, path, missing: List[str], unexpected: List[str], mismatched: List[str]) -> None:
        self.missing, self.unexpected, self.mismatched = missing, unexpected, mismatched
        lines = [f"{path}: the tensors do not fit the model"]
        if missing:
            lines.append(f"  missing ({len(missing)}): " + ", ".join(missing))
        if unexpected:
            lines.append(f"  unexpected ({len(unexpected)}): " + ", ".join(unexpected))
        if mismatched:
            lines.append(f"  wrong shape or type ({len(mismatched)}): " + "; ".join(mismatched))
        super().__init__("\n".join(lines))


def held_dtype(stored: torch.dtype, role: str, run_dtype: torch.dtype) -> torch.dtype:
    """The type a tensor is held in, given how it is stored and the precision of the run."""
    if role == "table" or not stored.is_floating_point:
        return torch.int32
    if run_dtype == torch.float32:
        return torch.float32
    if stored in (torch.float32, torch.float64):
        return torch.float32
    return torch.bfloat16


def _canonical(key: str, prefixes: Iterable[str], expected: Dict[str, ParamSpec]) -> Optional[str]:
    key = key.replace("._orig_mod", "")
    for prefix in sorted(prefixes, key=len, reverse=True):
        if key.startswith(prefix) and key[len(prefix):] in expected:
            return key[len(prefix):]
    return None


class _SafetensorsFile:
    def __init__(self, path: Path) -> None:
        self._handle = safe_open(str(path), framework="pt")
        self._handle.__enter__()

    def keys(self) -> List[str]:
        return list(self._handle.keys())

    def shape(self, key: str) -> Tuple[int, ...]:
        return tuple(self._handle.get_slice(key).get_shape())

    def tensor(self, key: str) -> torch.Tensor:
        return self._handle.get_tensor(key)

    def close(self) -> None:
        self._handle.__exit__(None, None, None)


class _TorchFile:
    """A ``.pt`` / ``.pth`` / ``.bin`` checkpoint: a mapping from names to tensors, read with the
    loader that runs nothing from the file, memory-mapped (``weights.py:560-566``)."""

    def __init__(self, path: Path) -> None:
        try:
            loaded = torch.load(str(path), map_location="cpu", weights_only=True, mmap=True)
        except Exception as exc:
            raise ValueError(f"{path}: not a checkpoint that the weights-only loader reads ({exc})") from exc
        if isinstance(loaded, dict) and isinstance(loaded.get("state_dict"), dict):
            loaded = loaded["state_dict"]
        if not isinstance(loaded, dict) or not all(isinstance(k, str) and isinstance(v, torch.Tensor)
                                                   for k, v in loaded.items()):
            raise ValueError(f"{path}: a checkpoint must be a mapping from tensor names to tensors")
        self._tensors: Dict[str, torch.Tensor] = loaded

    def keys(self) -> List[str]:
        return list(self._tensors)

    def shape(self, key: str) -> Tuple[int, ...]:
        return tuple(self._tensors[key].shape)

    def tensor(self, key: str) -> torch.Tensor:
        return self._tensors[key]

    def close(self) -> None:
        self._tensors = {}


TORCH_SUFFIXES = (".pt", ".pth", ".bin")


def find_weights(folder, filename: str) -> Path:
    """The weights file of a model folder: ``filename``, or the same name as a ``.pt`` checkpoint."""
    folder = Path(folder)
    candidates = [folder / filename] + [(folder / filename).with_suffix(suffix) for suffix in TORCH_SUFFIXES]
    for path in candidates:
        if path.exists():
            return path
    raise FileNotFoundError(f"{folder} holds no weights: looked for {', '.join(c.name for c in candidates)}")


def load_tensors(path, expected: Dict[str, ParamSpec], run_dtype: torch.dtype, device="cpu",
                 prefixes: Tuple[str, ...] = ("",), foreign_prefixes: Tuple[str, ...] = ()) -> Dict[str, torch.Tensor]:
    """All tensors of ``expected`` from the file at ``path`` (safetensors, or a ``.pt`` checkpoint
    by its suffix), on ``device``."""
    path = Path(path)
    if not path.exists():
        raise FileNotFoundError(f"{path} not found")
    missing, unexpected, mismatched = [], [], []
    out: Dict[str, torch.Tensor] = {}
    handle = _TorchFile(path) if path.suffix in TORCH_SUFFIXES else _SafetensorsFile(path)
    try:
        found: Dict[str, str] = {}
        for key in handle.keys():
            name = _canonical(key, prefixes, expected)
            if name is None:
                if not any(key.replace("._orig_mod", "").startswith(p) for p in foreign_prefixes):
                    unexpected.append(key)
            elif name in found:
                mismatched.append(f"{name}: stored twice ({found[name]} and {key})")
            else:
                found[name] = key
        for name, spec in expected.items():
            key = found.get(name)
            if key is None:
                missing.append(name)
                continue
            shape = handle.shape(key)
            if shape != tuple(spec.shape):
                mismatched.append(f"{name}: stored {list(shape)}, the model needs {list(spec.shape)}")
        if missing or unexpected or mismatched:
            raise WeightsError(path, sorted(missing), sorted(unexpected), mismatched)
        for name, spec in expected.items():
            tensor = handle.tensor(found[name])
            if spec.role != "table" and not tensor.dtype.is_floating_point:
                mismatched.append(f"{name}: stored as {tensor.dtype}, a floating type is needed")
                continue
            out[name] = tensor.to(device=device, dtype=held_dtype(tensor.dtype, spec.role, run_dtype))
    finally:
        handle.close()
    if mismatched:
        raise WeightsError(path, [], [], mismatched)
    return out
