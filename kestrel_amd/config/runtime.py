"""Knobs of the engine, as one typed object.

Reference: ``kestrel/config.py:155-202`` (``RuntimeConfig``: ``model_path``, ``device``,
``dtype``, ``max_batch_size``, ``page_size``, ``kv_cache_pages``, ``enable_cuda_graphs``,
``model``) with its checks (``:181-197``); names are kept where the meaning is the same.
"""

from __future__ import annotations

from dataclasses import dataclass
from pathlib import Path
from typing import Optional, Union

import torch

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32,
           "float": torch.float32}


def parse_dtype(value) -> torch.dtype:
    if isinstance(value, torch.dtype):
        if value not in (torch.bfloat16, torch.float32):
            raise ValueError(f"dtype must be bfloat16 or float32, got {value}")
        return value
    try:
        return _DTYPES[str(value).lower()]
    except KeyError:
        raise ValueError(f"dtype must be bfloat16 or float32, got {value!r}") from None


@dataclass
class RuntimeConfig:
    """``model_path``: folder with ``config.json`` and ``model.safetensors``.

    ``model``: architecture name; ``None`` takes it from ``config.json``.
    ``max_batch_size``: most requests decoded together. ``page_size``: tokens per cache
    page. The pool is sized by one of ``kv_cache_pages``, ``kv_cache_bytes`` (a byte budget as the
    reference's ``KVMemoryPool`` takes, ``kestrel/kv_cache.py:52-86``) or ``kv_cache_tokens``; with
    none of them, for ``max_batch_size`` full contexts. A pool that does not fit in the device's
    free memory is refused at start with a ``MemoryError``.
    ``max_num_batched_tokens``: token budget of one step (prompt portions are cut to it).
    ``enable_graphs``: replay decode-only steps, and every other step of up to 2,048 tokens, as captured HIP graphs.
    ``pipeline_depth``: 2 launches a step before the tokens of the one before have reached
    the host (``kestrel/scheduler/pipeline.py:49-65``); 1 reads every step first.
    ``seed``: base of the sampling generator.
    ``warmup``: make everything at start that steps would otherwise make when they first need it (the
    graph of every bucket of decode rows and of tokens, scratch buffers, the plans of the prompt's linears), as
    the reference does before ``create`` returns (``kestrel/engine/core.py:458-484``).
    ``tune_linears``: with ``warmup``, the linears of prompt steps that go through the vendor library time the
    algorithms it offers (that many products each) once per bucket of rows and keep the fastest; 0: the first
    the library names. Which algorithm wins can differ from start to start, and with it the last bits of a result.
    """

    model_path: Union[str, Path, None] = None
    device: str = "cuda"
    dtype: Union[torch.dtype, str] = torch.bfloat16
    max_batch_size: int = 4
    page_size: int = 16
    kv_cache_pages: Optional[int] = None
    kv_cache_tokens: Optional[int] = None
    kv_cache_bytes: Optional[int] = None
    max_num_batched_tokens: int = 2048
    enable_graphs: bool = True
    pipeline_depth: int = 2
    model: Optional[str] = None
    seed: int = 0
    max_seq_len: Optional[int] = None
    warmup: bool = True
    tune_linears: int = 0

    def __post_init__(self) -> None:
        self.dtype = parse_dtype(self.dtype)
        if self.max_batch_size <= 0:
            raise ValueError("max_batch_size must be a positive integer")
        if self.page_size <= 0:
            raise ValueError("page_size must be a positive integer")
        if self.kv_cache_pages is not None and self.kv_cache_pages <= 0:
            raise ValueError("kv_cache_pages must be a positive integer")
        if self.kv_cache_tokens is not None and self.kv_cache_tokens <= 0:
            raise ValueError("kv_cache_tokens must be a positive integer")
        if self.kv_cache_bytes is not None and self.kv_cache_bytes <= 0:
            raise ValueError("kv_cache_bytes must be a positive integer")
        if sum(v is not None for v in (self.kv_cache_pages, self.kv_cache_tokens, self.kv_cache_bytes)) > 1:
            raise ValueError("give one of kv_cache_pages, kv_cache_tokens and kv_cache_bytes")
        if self.max_num_batched_tokens <= 0:
            raise ValueError("max_num_batched_tokens must be a positive integer")
        if self.tune_linears < 0:
            raise ValueError("tune_linears must be zero or a positive number of timed products")
        if self.pipeline_depth not in (1, 2):
            raise ValueError("pipeline_depth must be 1 or 2")
        if self.max_seq_len is not None and self.max_seq_len <= 0:
            raise ValueError("max_seq_len must be a positive integer")
        device = torch.device(self.device)
        if device.type != "cuda":
            raise ValueError(f"device must be a GPU ('cuda' or 'cuda:N'), got {self.device!r}: there is no CPU path")

    def resolved_device(self) -> torch.device:
        device = torch.device(self.device)
        return torch.device("cuda", device.index if device.index is not None else 0)
