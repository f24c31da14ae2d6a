"""Moondream 2 text decoder: its configuration keys, its plan and its tensor names.

A Phi-1.5-style dense decoder: every block is ``x + attn(ln(x)) + mlp(ln(x))`` from one
biased LayerNorm, a fused biased q|k|v projection, non-interleaved rotary on the first
``head_dim / 2`` channels, a biased GELU-tanh MLP; the stack ends in a LayerNorm and an
untied biased head (``kestrel/models/moondream/text.py:197-377``).

Configuration keys are those of the reference's ``TextConfig``
(``kestrel/models/moondream/config.py:23-36``), nested under ``"text"`` as in its
configuration dicts (``config.py:259-273``) or flat. Three values the reference fixes in
code may also be given: ``layer_norm_eps`` (``nn.LayerNorm`` default, ``text.py:311``),
``rotary_dim`` (``dim // (2 n_heads)``, ``text.py:365-366``) and ``head_dim``
(``dim // n_heads``, ``text.py:92``). The sizes of the released model live in
``presets/moondream2.json`` and are used only when ``config.json`` has no text section.
"""

from __future__ import annotations

import json
from dataclasses import dataclass
from pathlib import Path
from typing import Any, Dict, Optional, Tuple

from ..config.registry import ModelSpec, register
from ..parts.specs import (AttentionSpec, DenseFeedForwardSpec, LayerSpec, ModelPlan, NormSpec, PositionSpec,
                           ScheduleEntry)

_PRESET = Path(__file__).resolve().parent / "presets" / "moondream2.json"
_REQUIRED = ("dim", "ff_dim", "n_layers", "vocab_size", "max_context", "n_heads", "n_kv_heads", "rope_theta")
_OPTIONAL = ("prefix_attn", "group_size", "moe", "tau_attn", "head_dim", "rotary_dim", "layer_norm_eps")
# Other spellings of the three values that the reference fixes in code and of its rotary base.
_ALIASES = {"layer_norm_eps": ("layernorm_eps", "ln_eps", "norm_eps", "eps", "layer_norm_epsilon"),
            "rotary_dim": ("rot_dim", "rope_dim", "rotary_ndims"),
            "rope_theta": ("theta", "rotary_theta", "rope_base")}


def _preset() -> Dict[str, Any]:
    with open(_PRESET) as handle:
        return json.load(handle)


@dataclass(frozen=True)
class MoondreamTextConfig:
    dim: int
    ff_dim: int
    n_layers: int
    vocab_size: int
    max_context: int
    n_heads: int
    n_kv_heads: int
    rope_theta: float
    head_dim: int
    rotary_dim: int
    layer_norm_eps: float
    prefix_attn: int = 0        # declared by the reference and never read there (``config.py:32,268``): the mask follows
                                # the block a request brings; kept as the length measurements and tests give that block
    bos_id: int = 0
    eos_id: int = 0

    @classmethod
    def from_dict(cls, config: Dict[str, Any]) -> "MoondreamTextConfig":
        preset = _preset()
        text = config.get("text")
        if text is None:
            spellings = _REQUIRED + _OPTIONAL + tuple(o for others in _ALIASES.values() for o in others)
            flat = {k: config[k] for k in spellings if k in config}
            text = flat if flat else preset["text"]
        if not isinstance(text, dict):
            raise ValueError("config.json: 'text' must be an object")
        text = dict(text)
        for key, others in _ALIASES.items():
            given = [o for o in others if o in text]
            if given and (key in text or len(given) > 1):
                raise ValueError(f"config.json: {[key] * (key in text) + given} name the same value")
            if given:
                text[key] = text.pop(given[0])
        unknown = sorted(set(text) - set(_REQUIRED) - set(_OPTIONAL))
        if unknown:
            raise ValueError(f"config.json: unknown text keys {unknown}; known: {sorted(_REQUIRED + _OPTIONAL)}")
        missing = [k for k in _REQUIRED if k not in text]
        if missing:
            raise ValueError(f"config.json: text keys missing: {missing}")
        if text.get("moe") is not None:
            raise ValueError("config.json: 'moe' is set; this engine builds the dense Moondream 2 decoder only")
        if text.get("tau_attn"):
            raise ValueError("config.json: 'tau_attn' is set; Moondream 2 has no tau attention")
        if text.get("group_size") is not None:
            raise NotImplementedError("Quantized linear layers are not supported")
        ints = {k: _positive_int(text, k) for k in ("dim", "ff_dim", "n_layers", "vocab_size", "max_context",
                                                    "n_heads", "n_kv_heads")}
        if ints["n_heads"] % ints["n_kv_heads"]:
            raise ValueError(f"config.json: n_heads {ints['n_heads']} is no multiple of n_kv_heads {ints['n_kv_heads']}")
        if text.get("head_dim") is not None:
            head_dim = _positive_int(text, "head_dim")
        else:
            if ints["dim"] % ints["n_heads"]:
                raise ValueError(f"config.json: dim {ints['dim']} is no multiple of n_heads {ints['n_heads']}")
            head_dim = ints["dim"] // ints["n_heads"]
        rotary_dim = int(text["rotary_dim"]) if text.get("rotary_dim") is not None else head_dim // 2
        if rotary_dim < 0 or rotary_dim > head_dim or rotary_dim % 2:
            raise ValueError(f"config.json: rotary_dim {rotary_dim} must be even and within head_dim {head_dim}")
        eps = float(text["layer_norm_eps"]) if text.get("layer_norm_eps") is not None \
            else float(preset["fixed"]["layer_norm_eps"])
        if not eps > 0:
            raise ValueError("config.json: layer_norm_eps must be positive")
        theta = float(text["rope_theta"])
        if not theta > 0:
            raise ValueError("config.json: rope_theta must be positive")
        prefix = int(text.get("prefix_attn") or 0)
        if prefix < 0 or prefix > ints["max_context"]:
            raise ValueError(f"config.json: prefix_attn {prefix} out of range")
        tokenizer = config.get("tokenizer") or preset["tokenizer"]
        return cls(rope_theta=theta, head_dim=head_dim, rotary_dim=rotary_dim, layer_norm_eps=eps,
                   prefix_attn=prefix, bos_id=int(tokenizer.get("bos_id", 0)), eos_id=int(tokenizer.get("eos_id", 0)),
                   **ints)

    def to_dict(self) -> Dict[str, Any]:
        text = {k: getattr(self, k) for k in _REQUIRED}
        text.update(head_dim=self.head_dim, rotary_dim=self.rotary_dim, layer_norm_eps=self.layer_norm_eps,
                    prefix_attn=self.prefix_attn, group_size=None, moe=None, tau_attn=False)
        return {"model": "moondream2", "text": text, "tokenizer": {"bos_id": self.bos_id, "eos_id": self.eos_id}}


def _positive_int(text: Dict[str, Any], key: str) -> int:
    value = text[key]
    if isinstance(value, bool) or not isinstance(value, int) or value <= 0:
        raise ValueError(f"config.json: {key} must be a positive integer, got {value!r}")
    return value


def build_plan(cfg: MoondreamTextConfig) -> ModelPlan:
    """Layer ``i`` takes the tensors ``text.blocks.{i}.*`` (``weights.py:80-107``)."""
    position = PositionSpec("rotary_neox", cfg.rotary_dim, cfg.rope_theta, cfg.max_context)
    layers = []
    for i in range(cfg.n_layers):
        p = f"text.blocks.{i}."
        names = {
            "norm.weight": p + "ln.weight", "norm.bias": p + "ln.bias",
            "mixer.qkv.weight": p + "attn.qkv.weight", "mixer.qkv.bias": p + "attn.qkv.bias",
            "mixer.proj.weight": p + "attn.proj.weight", "mixer.proj.bias": p + "attn.proj.bias",
            "feed_forward.fc1.weight": p + "mlp.fc1.weight", "feed_forward.fc1.bias": p + "mlp.fc1.bias",
            "feed_forward.fc2.weight": p + "mlp.fc2.weight", "feed_forward.fc2.bias": p + "mlp.fc2.bias",
        }
        layers.append(LayerSpec(
            arrangement="parallel",
            norm=NormSpec("layernorm", cfg.dim, cfg.layer_norm_eps, bias=True),
            mixer=AttentionSpec("attention", cfg.dim, cfg.n_heads, cfg.n_kv_heads, cfg.head_dim, position, bias=True),
            feed_forward=DenseFeedForwardSpec("dense", cfg.dim, cfg.ff_dim, "gelu_tanh", bias=True),
            names=names,
        ))
    return ModelPlan(
        architecture="moondream2", vocab_size=cfg.vocab_size, dim=cfg.dim, max_positions=cfg.max_context,
        layers=tuple(layers), schedule=tuple(ScheduleEntry(i) for i in range(cfg.n_layers)),
        final_norm=NormSpec("layernorm", cfg.dim, cfg.layer_norm_eps, bias=True), head_bias=True, tied_head=False,
        names={"embedding": "text.wte", "final_norm.weight": "text.post_ln.weight",
               "final_norm.bias": "text.post_ln.bias", "head.weight": "text.lm_head.weight",
               "head.bias": "text.lm_head.bias"},
        eos_token_ids=(cfg.eos_id,), bos_token_id=cfg.bos_id,
    )


def _claims(config: Dict[str, Any]) -> bool:
    text = config.get("text", config)
    return isinstance(text, dict) and all(k in text for k in ("dim", "ff_dim", "n_layers", "n_heads")) \
        and any(k in text for k in ("rope_theta",) + _ALIASES["rope_theta"])


register(ModelSpec(
    name="moondream2",
    read_config=MoondreamTextConfig.from_dict,
    build_plan=build_plan,
    aliases=("moondream", "moondream1", "HfMoondream", "moondream-2", "vikhyatk/moondream2"),
    claims=_claims,
    filename="model.safetensors",
    tensor_prefixes=("", "model."),
    foreign_prefixes=("vision.", "region.", "model.vision.", "model.region."),
    default_config=_preset,
))
