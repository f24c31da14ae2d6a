"""Plain, slow implementation of the Moondream 2 text decoder.

Whole sequences, no cache, one function per part, dense masks. Written from the
formulas of the reference (cited per function as ``file:line`` relative to the
reference tree) and sharing no code with ``kestrel_amd``. Everything runs on the
CPU in one floating type (``float64`` by default), so that its error is far below
that of the engine it judges.

The configuration is a plain ``dict`` with the reference's ``TextConfig`` keys
(``kestrel/models/moondream/config.py:23-36``) plus the three that the reference
fixes in code: ``layer_norm_eps`` (``nn.LayerNorm`` default, ``text.py:311``),
``rotary_dim`` (``head_dim // 2``, ``text.py:365-366``) and ``head_dim``
(``dim // n_heads``, ``text.py:92``).
"""

from __future__ import annotations

import math
from typing import Dict, Optional, Sequence

import torch

Tensor = torch.Tensor


# ----------------------------------------------------------------------------
# configuration helpers
# ----------------------------------------------------------------------------

def head_dim_of(cfg: dict) -> int:
    """``head_dim = d_model // n_heads`` (``text.py:92``) unless given."""
    return int(cfg.get("head_dim") or cfg["dim"] // cfg["n_heads"])


def rotary_dim_of(cfg: dict) -> int:
    """Rotated channels per head: ``dim // (2 * n_heads)`` (``text.py:365-366``)."""
    value = cfg.get("rotary_dim")
    return int(value) if value is not None else head_dim_of(cfg) // 2


def eps_of(cfg: dict) -> float:
    """LayerNorm eps: ``nn.LayerNorm(dim)`` default 1e-5 (``text.py:311,359``)."""
    return float(cfg.get("layer_norm_eps", 1e-5))


# ----------------------------------------------------------------------------
# parts
# ----------------------------------------------------------------------------

def embedding(ids: Tensor, wte: Tensor) -> Tensor:
    """``x[t] = wte[id[t]]``, no scale and no positional add (``text.py:39-40``)."""
    return wte[ids.long()]


def layer_norm(x: Tensor, weight: Tensor, bias: Tensor, eps: float) -> Tensor:
    """LayerNorm over the last axis with affine (``layers.py:40-44``; biased variance)."""
    mean = x.mean(dim=-1, keepdim=True)
    centred = x - mean
    var = (centred * centred).mean(dim=-1, keepdim=True)
    return centred / torch.sqrt(var + eps) * weight + bias


def linear(x: Tensor, weight: Tensor, bias: Optional[Tensor]) -> Tensor:
    """``x @ W.T + b`` with ``W`` stored ``[out, in]`` (``layers.py:53-54``)."""
    y = x @ weight.transpose(-1, -2)
    return y if bias is None else y + bias


def gelu_tanh(x: Tensor) -> Tensor:
    """``F.gelu(approximate="tanh")`` written out (``layers.py:30-31``)."""
    inner = math.sqrt(2.0 / math.pi) * (x + 0.044715 * x * x * x)
    return 0.5 * x * (1.0 + torch.tanh(inner))


def rotary_table(rot_dim: int, n_positions: int, theta: float, dtype=torch.float64) -> Tensor:
    """Row ``p`` is ``cat(cos(p*f), sin(p*f))``, ``f_i = theta**(-2i/rot_dim)`` (``rope.py:6-32``)."""
    if rot_dim % 2:
        raise ValueError("rot_dim must be even")
    exponents = torch.arange(0, rot_dim, 2, dtype=dtype) / float(rot_dim)
    inv_freq = 1.0 / (theta ** exponents)
    angles = torch.arange(n_positions, dtype=dtype).unsqueeze(1) * inv_freq.unsqueeze(0)
    return torch.cat([torch.cos(angles), torch.sin(angles)], dim=-1)


def apply_rotary(x: Tensor, positions: Tensor, table: Tensor) -> Tensor:
    """Non-interleaved (NeoX) rotation of the first ``R`` channels of every head.

    ``x``: ``[T, heads, head_dim]``; ``table``: ``[P, R]``. With ``a = x[..., :R/2]`` and
    ``b = x[..., R/2:R]``: ``a' = a cos - b sin``, ``b' = b cos + a sin``; channels from
    ``R`` on pass through (``text.py:123-125``; rotate-half stated at ``ops/rotary.py:58-72``).
    """
    rot = table.shape[1]
    half = rot // 2
    rows = table[positions.long()]
    cos = rows[:, :half].unsqueeze(1)
    sin = rows[:, half:].unsqueeze(1)
    a = x[..., :half]
    b = x[..., half:rot]
    out = x.clone()
    out[..., :half] = a * cos - b * sin
    out[..., half:rot] = b * cos + a * sin
    return out


def visibility(positions: Tensor, block_ids: Optional[Tensor]) -> Tensor:
    """``allowed[q, k]``: causal, or both tokens in the same block with id >= 0.

    (``text.py:146-157``; block ids ``runtime.py:1733-1743``: image rows and BOS share a
    block id >= 0, text tokens carry -1.)
    """
    allowed = positions.unsqueeze(0) <= positions.unsqueeze(1)
    if block_ids is not None:
        same = (block_ids.unsqueeze(0) == block_ids.unsqueeze(1)) & (block_ids.unsqueeze(1) >= 0)
        allowed = allowed | same
    return allowed


def attention_core(q: Tensor, k: Tensor, v: Tensor, allowed: Tensor, scale: float) -> Tensor:
    """``softmax(q k^T * scale + mask) v`` per head; kv head of query head ``h`` is ``h // G``.

    ``q``: ``[T, H, hd]``; ``k, v``: ``[T, Hkv, hd]``; scale is the flash default
    ``hd**-0.5`` because the reference passes none (``text.py:158-185``).
    """
    n_heads, n_kv = q.shape[1], k.shape[1]
    group = n_heads // n_kv
    out = torch.empty_like(q)
    for h in range(n_heads):
        kh = k[:, h // group, :]
        vh = v[:, h // group, :]
        scores = (q[:, h, :] @ kh.transpose(0, 1)) * scale
        scores = scores.masked_fill(~allowed, float("-inf"))
        scores = scores - scores.max(dim=-1, keepdim=True).values
        weights = torch.exp(scores)
        weights = weights / weights.sum(dim=-1, keepdim=True)
        out[:, h, :] = weights @ vh
    return out


def attention(x_norm: Tensor, w: Dict[str, Tensor], prefix: str, cfg: dict,
              positions: Tensor, allowed: Tensor, table: Tensor) -> Tensor:
    """Fused QKV, split q|k|v, rotary on q and k, masked softmax, output projection.

    (``text.py:101-121`` projection and split order, ``:123-125`` rotary, ``:134-185``
    attention, ``:187-193`` output projection.)
    """
    n_heads, n_kv, hd = cfg["n_heads"], cfg["n_kv_heads"], head_dim_of(cfg)
    qkv = linear(x_norm, w[prefix + "attn.qkv.weight"], w[prefix + "attn.qkv.bias"])
    q, k, v = qkv.split([n_heads * hd, n_kv * hd, n_kv * hd], dim=-1)
    tokens = x_norm.shape[0]
    q = apply_rotary(q.reshape(tokens, n_heads, hd), positions, table)
    k = apply_rotary(k.reshape(tokens, n_kv, hd), positions, table)
    v = v.reshape(tokens, n_kv, hd)
    out = attention_core(q, k, v, allowed, hd ** -0.5).reshape(tokens, n_heads * hd)
    return linear(out, w[prefix + "attn.proj.weight"], w[prefix + "attn.proj.bias"])


def mlp(x_norm: Tensor, w: Dict[str, Tensor], prefix: str) -> Tensor:
    """``fc2(gelu_tanh(fc1(x)))`` with biases (``layers.py:90,105-106``)."""
    hidden = gelu_tanh(linear(x_norm, w[prefix + "mlp.fc1.weight"], w[prefix + "mlp.fc1.bias"]))
    return linear(hidden, w[prefix + "mlp.fc2.weight"], w[prefix + "mlp.fc2.bias"])


def block(x: Tensor, w: Dict[str, Tensor], index: int, cfg: dict,
          positions: Tensor, allowed: Tensor, table: Tensor) -> Tensor:
    """``x + attn(ln(x)) + mlp(ln(x))``: one norm feeds both branches (``text.py:222-275``)."""
    prefix = f"text.blocks.{index}."
    x_norm = layer_norm(x, w[prefix + "ln.weight"], w[prefix + "ln.bias"], eps_of(cfg))
    return x + attention(x_norm, w, prefix, cfg, positions, allowed, table) + mlp(x_norm, w, prefix)


def head(x: Tensor, w: Dict[str, Tensor], cfg: dict) -> Tensor:
    """``lm_head(post_ln(x))``, untied, with bias (``text.py:283-295``)."""
    normed = layer_norm(x, w["text.post_ln.weight"], w["text.post_ln.bias"], eps_of(cfg))
    return linear(normed, w["text.lm_head.weight"], w["text.lm_head.bias"])


# ----------------------------------------------------------------------------
# whole model
# ----------------------------------------------------------------------------

def _as(w: Dict[str, Tensor], dtype) -> Dict[str, Tensor]:
    out = {}
    for name, tensor in w.items():
        if name.startswith("model."):
            name = name[len("model."):]
        out[name] = tensor.to(dtype)
    return out


def forward(cfg: dict, weights: Dict[str, Tensor], ids: Sequence[int],
            prefix_embeds: Optional[Tensor] = None, block_ids: Optional[Sequence[int]] = None,
            position_start: int = 0, dtype=torch.float64, rows: Optional[Sequence[int]] = None) -> Tensor:
    """Logits ``[T, V]`` at every position of one sequence, or ``[len(rows), V]`` at the positions
    ``rows`` (the rows are taken before the final norm and the head, ``runtime.py:2374-2379``).

    The sequence is ``prefix_embeds`` rows (given embeddings, used verbatim:
    ``runtime.py:2081-2115``) followed by the embeddings of ``ids``. ``block_ids`` has
    one entry per position (``-1`` = causal text); when omitted and a prefix is given,
    the prefix rows form block 0 (``runtime.py:1733-1735``). Positions count from
    ``position_start`` (``runtime.py:332-334``).
    """
    w = _as(weights, dtype)
    parts = []
    if prefix_embeds is not None and prefix_embeds.numel():
        parts.append(prefix_embeds.to(dtype))
    if len(ids):
        parts.append(embedding(torch.as_tensor(list(ids)), w["text.wte"]))
    x = torch.cat(parts, dim=0)
    total = x.shape[0]
    if block_ids is None and prefix_embeds is not None:
        n_prefix = prefix_embeds.shape[0]
        block_ids = [0] * n_prefix + [-1] * (total - n_prefix)
    positions = torch.arange(position_start, position_start + total)
    blocks = None if block_ids is None else torch.as_tensor(list(block_ids))
    allowed = visibility(positions, blocks)
    table = rotary_table(rotary_dim_of(cfg), position_start + total, float(cfg["rope_theta"]), dtype)
    for index in range(cfg["n_layers"]):
        x = block(x, w, index, cfg, positions, allowed, table)
    if rows is not None:
        x = x[torch.as_tensor(list(rows), dtype=torch.long)]
    return head(x, w, cfg)


def greedy_generate(cfg: dict, weights: Dict[str, Tensor], ids: Sequence[int], n_new: int,
                    prefix_embeds: Optional[Tensor] = None, dtype=torch.float64):
    """Greedy continuation by recomputing the whole sequence for every token.

    Returns ``(tokens, margins)`` where ``margins[i]`` is the gap between the best and
    the second best logit at step ``i`` (a test may skip exact comparison on near ties).
    """
    ids = list(ids)
    out, margins = [], []
    for _ in range(n_new):
        logits = forward(cfg, weights, ids, prefix_embeds, dtype=dtype)[-1]
        top = torch.topk(logits, 2)
        out.append(int(top.indices[0]))
        margins.append(float(top.values[0] - top.values[1]))
        ids.append(out[-1])
    return out, margins


# ----------------------------------------------------------------------------
# sampling
# ----------------------------------------------------------------------------

def nucleus_probs(logits: Tensor, temperature: float, top_p: float) -> Tensor:
    """Distribution sampled from: ``softmax(logits / T)`` restricted to the top-p nucleus.

    Tokens are taken in order of falling probability until their mass reaches ``top_p``
    (the token that crosses it is kept); the rest get zero; renormalised
    (``scheduler.py:2955-2993``; ``T <= 1e-6`` is greedy: ``scheduler.py:55,3019-3042``).
    """
    logits = logits.to(torch.float64)
    if temperature <= 1e-6:
        probs = torch.zeros_like(logits)
        probs[int(torch.argmax(logits))] = 1.0
        return probs
    probs = torch.softmax(logits / temperature, dim=-1)
    if top_p < 1.0:
        order = torch.argsort(probs, descending=True, stable=True)
        sorted_probs = probs[order]
        before = torch.cumsum(sorted_probs, dim=0) - sorted_probs
        keep = before < top_p
        kept = torch.zeros_like(probs)
        kept[order[keep]] = sorted_probs[keep]
        probs = kept / kept.sum()
    return probs
