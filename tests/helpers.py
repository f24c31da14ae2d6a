"""Tiny configurations, random model folders and runner helpers shared by the tests."""

from __future__ import annotations

import functools
import tempfile
from typing import Dict, List, Optional, Sequence

import torch

from kestrel_amd.weights import InitRecipe, write_random_model

# Two tiny configurations that differ in every size and option, and a third with an
# explicit head size that is no power of two, grouped kv heads and an odd vocabulary.
TINY_A = {"text": {"dim": 64, "ff_dim": 256, "n_layers": 2, "vocab_size": 512, "max_context": 128, "n_heads": 4,
                   "n_kv_heads": 4, "rope_theta": 10000.0, "prefix_attn": 0, "layer_norm_eps": 1e-5}}
TINY_B = {"text": {"dim": 96, "ff_dim": 320, "n_layers": 3, "vocab_size": 1000, "max_context": 256, "n_heads": 3,
                   "n_kv_heads": 1, "rope_theta": 5000.0, "prefix_attn": 17, "layer_norm_eps": 1e-6}}
TINY_C = {"text": {"dim": 120, "ff_dim": 200, "n_layers": 2, "vocab_size": 777, "max_context": 320, "n_heads": 6,
                   "n_kv_heads": 2, "head_dim": 48, "rotary_dim": 12, "rope_theta": 1234.5, "prefix_attn": 5,
                   "layer_norm_eps": 3e-5}}
RECIPES = {
    "A": InitRecipe(std=0.02),
    "B": InitRecipe(std=0.03, gain_std=0.02, shift_std=0.02),
    "C": InitRecipe(std=0.05, bias_std=0.1, gain_std=0.1, shift_std=0.05),
}
CONFIGS = {"A": TINY_A, "B": TINY_B, "C": TINY_C}
SEEDS = {"A": 0, "B": 1, "C": 2}


@functools.lru_cache(maxsize=None)
def model_dir(name: str, store_dtype: str = "bfloat16") -> str:
    """A temporary model folder for one of the tiny configurations (made once per process)."""
    folder = tempfile.mkdtemp(prefix=f"kestrel_amd_tiny{name}_")
    write_random_model(folder, CONFIGS[name], SEEDS[name], RECIPES[name], store_dtype=store_dtype)
    return folder


def flat_config(name: str) -> dict:
    return dict(CONFIGS[name]["text"])


def stored_weights(folder: str) -> Dict[str, torch.Tensor]:
    from safetensors.torch import load_file

    return load_file(folder + "/model.safetensors")


def random_ids(seed: int, count: int, vocab: int) -> List[int]:
    gen = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (count,), generator=gen).tolist()


def tolerance(dtype: torch.dtype):
    """(atol, rtol) for logits of the tiny models against the float64 plain implementation."""
    if dtype == torch.float32:
        return 2e-5, 2e-5
    return 3e-2, 3e-2


def assert_close(actual: torch.Tensor, expected: torch.Tensor, dtype: torch.dtype, what: str = "") -> None:
    atol, rtol = tolerance(dtype)
    actual = actual.detach().cpu().double()
    expected = expected.detach().cpu().double()
    assert actual.shape == expected.shape, f"{what}: shape {tuple(actual.shape)} vs {tuple(expected.shape)}"
    err = (actual - expected).abs()
    bound = atol + rtol * expected.abs()
    if not bool((err <= bound).all()):
        worst = int(torch.argmax(err - bound))
        idx = tuple(int(i) for i in torch.unravel_index(torch.tensor(worst), err.shape))
        raise AssertionError(f"{what}: worst at {idx}: got {actual[idx]:.6g}, expected {expected[idx]:.6g}, "
                             f"error {err[idx]:.3g} > {bound[idx]:.3g}; max error {err.max():.3g}")
