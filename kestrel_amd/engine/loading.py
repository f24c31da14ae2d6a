"""From a model folder to a bound model, a cache and a runner."""

from __future__ import annotations

from pathlib import Path
from typing import Optional

import torch

from ..cache.manager import CacheManager
from ..config.registry import read_model_dir
from ..models.decoder import DecoderModel
from ..weights.loader import find_weights, load_tensors
from .step import ModelRunner


def require_gpu(device: torch.device) -> None:
    if not torch.cuda.is_available():
        raise RuntimeError("no GPU is visible: kestrel_amd runs on an AMD GPU only, there is no CPU path")
    if device.type != "cuda":
        raise RuntimeError(f"device {device} is no GPU")


def load_model(model_dir, dtype: torch.dtype, device: torch.device, model: Optional[str] = None) -> DecoderModel:
    """The model of ``model_dir`` (class chosen by its config.json) with its weights bound.
    ``model_dir`` is a folder with ``config.json`` and the weights, or the weights file itself
    (safetensors or a ``.pt`` checkpoint) with ``config.json`` beside it."""
    require_gpu(device)
    model_dir = Path(model_dir)
    weights_file = None
    if model_dir.is_file():
        weights_file, model_dir = model_dir, model_dir.parent
    spec, _typed, plan = read_model_dir(model_dir, model)
    net = DecoderModel(plan)
    tensors = load_tensors(weights_file or find_weights(model_dir, spec.filename), net.params(), dtype, device=device,
                           prefixes=spec.tensor_prefixes, foreign_prefixes=spec.foreign_prefixes)
    net.bind(tensors, dtype, device)
    return net


def make_runner(net: DecoderModel, page_size: int, n_pages: int, max_requests: int,
                max_tokens_per_step: int = 4096, enable_graphs: bool = False) -> ModelRunner:
    cache = CacheManager(net.cache_needs(), page_size, n_pages, max_requests, dtype=net.dtype, device=net.device)
    return ModelRunner(net, cache, net.device, max_tokens_per_step, enable_graphs=enable_graphs)
