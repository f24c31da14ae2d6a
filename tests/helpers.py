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
# Head sizes the MFMA kernels take (64 with one shared kv head, 128 with as many kv heads as heads),
# widths that are no multiple of 64: what serving runs, at toy size.
TINY_D = {"text": {"dim": 128, "ff_dim": 136, "n_layers": 2, "vocab_size": 300, "max_context": 256, "n_heads": 2,
                   "n_kv_heads": 1, "rope_theta": 10000.0, "prefix_attn": 9, "layer_norm_eps": 1e-5}}
TINY_E = {"text": {"dim": 256, "ff_dim": 264, "n_layers": 2, "vocab_size": 411, "max_context": 192, "n_heads": 2,
                   "n_kv_heads": 2, "rope_theta": 2500.0, "rotary_dim": 32, "prefix_attn": 6, "layer_norm_eps": 2e-6}}
# A head size that is no power of two on the MFMA kernels (80, as in Phi-2: ten 16-byte chunks a key row, two
# and a half blocks of 32 output channels), grouped kv heads, a rotary part of 32 channels.
TINY_F = {"text": {"dim": 160, "ff_dim": 168, "n_layers": 2, "vocab_size": 333, "max_context": 256, "n_heads": 4,
                   "n_kv_heads": 2, "head_dim": 80, "rotary_dim": 32, "rope_theta": 10000.0, "prefix_attn": 7,
                   "layer_norm_eps": 1e-5}}
# A long context (rows of more than 4096 keys are cut into parts by the decode attention kernel), one layer.
TINY_G = {"text": {"dim": 64, "ff_dim": 72, "n_layers": 1, "vocab_size": 211, "max_context": 6144, "n_heads": 2,
                   "n_kv_heads": 1, "rope_theta": 50000.0, "prefix_attn": 0, "layer_norm_eps": 1e-5}}
RECIPES = {
    "A": InitRecipe(std=0.02),
    "B": InitRecipe(std=0.03, gain_std=0.02, shift_std=0.02),
    "C": InitRecipe(std=0.05, bias_std=0.1, gain_std=0.1, shift_std=0.05),
    "D": InitRecipe(std=0.04, gain_std=0.05, shift_std=0.05),
    "E": InitRecipe(std=0.03, bias_std=0.05, gain_std=0.05, shift_std=0.02),
    "F": InitRecipe(std=0.04, bias_std=0.03, gain_std=0.05, shift_std=0.03),
    "G": InitRecipe(std=0.08, bias_std=0.05, gain_std=0.05, shift_std=0.03),
}
CONFIGS = {"A": TINY_A, "B": TINY_B, "C": TINY_C, "D": TINY_D, "E": TINY_E, "F": TINY_F, "G": TINY_G}
SEEDS = {"A": 0, "B": 1, "C": 2, "D": 3, "E": 4, "F": 5, "G": 6}


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
    """(atol, rtol, spread) for logits against the float64 plain implementation: an error may be
    ``atol + rtol * |expected| + spread * std(expected row)``. float32: absolute and relative 2e-5.
    bfloat16: what eight bits of mantissa leave after a few layers is a share of the spread of a
    row's logits (measured on the tiny configurations: at most 1.8 % of it), so the bound is 3 % of
    that spread plus 1 % of the value, whatever the scale of the weights."""
    if dtype == torch.float32:
        return 2e-5, 2e-5, 0.0
    return 0.0, 1e-2, 3e-2


def assert_close(actual: torch.Tensor, expected: torch.Tensor, dtype: torch.dtype, what: str = "") -> None:
    atol, rtol, spread = tolerance(dtype)
    actual = actual.detach().cpu().double()
    expected = expected.detach().cpu().double()
    assert actual.shape == expected.shape, f"{what}: shape {tuple(actual.shape)} vs {tuple(expected.shape)}"
    err = (actual - expected).abs()
    bound = atol + rtol * expected.abs()
    if spread:
        rows = expected.reshape(-1, expected.shape[-1])
        bound = bound + spread * rows.std(dim=1, unbiased=False).reshape(*expected.shape[:-1], 1)
    if not bool((err <= bound).all()):
        worst = int(torch.argmax(err - bound))
        idx = tuple(int(i) for i in torch.unravel_index(torch.tensor(worst), err.shape))
        raise AssertionError(f"{what}: worst at {idx}: got {actual[idx]:.6g}, expected {expected[idx]:.6g}, "
                             f"error {err[idx]:.3g} > {bound[idx]:.3g}; max error {err.max():.3g}")


def assert_greedy_follows(cfg: dict, weights, prompt: Sequence[int], tokens: Sequence[int], slack: float, what: str,
                          prefix_embeds: Optional[torch.Tensor] = None) -> None:
    """Every generated token must be the plain implementation's choice *after the engine's own
    earlier tokens*: the plain model is run once over prompt + tokens and, at each place, the
    engine's token may lie at most ``slack`` below the best logit. A near tie thus excuses one token
    only and every later one is still checked."""
    from tests.plain import moondream_plain as plain

    tokens = list(tokens)
    logits = plain.forward(cfg, weights, list(prompt) + tokens[:-1], prefix_embeds)
    n_prefix = 0 if prefix_embeds is None else prefix_embeds.shape[0]
    first = n_prefix + len(prompt) - 1
    for i, token in enumerate(tokens):
        row = logits[first + i]
        gap = float(row.max() - row[token])
        assert gap <= slack, (f"{what}: token {i} is {token}, the plain implementation gives {int(row.argmax())} "
                              f"after the same tokens ({gap:.3g} better)")


# ----------------------------------------------------------------------------
# replaying requests through a runner in a given way of cutting
# ----------------------------------------------------------------------------

class Request:
    """A test request: optional prefix embeddings (one bidirectional block) and token ids."""

    def __init__(self, name: str, ids: Sequence[int], prefix: Optional[torch.Tensor] = None) -> None:
        self.name, self.ids, self.prefix = name, list(ids), prefix
        self.n_prefix = 0 if prefix is None else prefix.shape[0]
        self.length = self.n_prefix + len(self.ids)
        self.done = 0            # tokens fed so far
        self.slot = None

    def take(self, count: int):
        """The next ``count`` places as (tokens, embeds, bidirectional)."""
        lo, hi = self.done, min(self.done + count, self.length)
        tokens, embeds = [], None
        if lo < self.n_prefix:
            if hi < self.n_prefix:
                raise AssertionError("test bug: a portion splits the prefix block")
            tokens += [-1] * (self.n_prefix - lo)
            embeds = self.prefix[lo:self.n_prefix]
        tokens += self.ids[max(lo, self.n_prefix) - self.n_prefix:hi - self.n_prefix]
        bidir = [(0, self.n_prefix)] if lo == 0 and self.n_prefix else []
        self.done = hi
        return tokens, embeds, bidir, lo


def replay(runner, requests: Dict[str, "Request"], steps, poison: bool = False) -> Dict[str, torch.Tensor]:
    """Run ``steps`` = list of lists of (request name, number of tokens); every fed place is
    wanted. Returns the logits per request in position order, ``[fed, vocab]``. A request is
    admitted at its first portion and released after its last. With ``poison`` the pages a
    request gives back are filled with NaN, so that a later read of them shows."""
    from kestrel_amd.engine.step import StepEntry

    rows: Dict[str, List[torch.Tensor]] = {name: [] for name in requests}
    for step in steps:
        entries, order = [], []
        for name, count in step:
            req = requests[name]
            if req.slot is None:
                req.slot = runner.admit()
            tokens, embeds, bidir, _lo = req.take(count)
            entries.append(StepEntry(req.slot, tokens, want=list(range(len(tokens))), embeds=embeds,
                                     bidirectional=bidir))
            order.append((name, len(tokens)))
        logits = runner.step(entries).clone()
        at = 0
        for name, count in order:
            rows[name].append(logits[at:at + count])
            at += count
        for name, _ in order:
            req = requests[name]
            if req.done == req.length:
                pages = [[p for p in runner.cache.block_table(g, req.slot) if p >= 0]
                         for g in range(len(runner.cache.groups))]
                runner.release(req.slot)
                req.slot = None
                if poison:
                    for g, group in enumerate(runner.cache.groups):
                        if pages[g]:
                            for tensor in group.tensors.values():
                                tensor[:, torch.tensor(pages[g], device=tensor.device)] = float("nan")
        runner.cache.check()
    return {name: torch.cat(chunks, dim=0) for name, chunks in rows.items() if chunks}


def poison_cache(runner) -> None:
    for group in runner.cache.groups:
        for tensor in group.tensors.values():
            tensor.fill_(float("nan"))
