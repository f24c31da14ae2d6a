"""Pins of the plain implementation: what fixes each formula beside the reference's text.

Each check is chosen so that a plausible mistake (a wrong sign or pairing, a norm in the
wrong place, the wrong GELU) fails it.
"""

import math

import pytest
import torch
import torch.nn.functional as F

from tests import helpers
from tests.plain import moondream_plain as plain

torch.manual_seed(0)
D = torch.float64


def test_layer_norm_equals_library_and_eps_matters():
    x = torch.randn(5, 96, dtype=D)
    w, b = torch.randn(96, dtype=D), torch.randn(96, dtype=D)
    for eps in (1e-5, 1e-6):
        torch.testing.assert_close(plain.layer_norm(x, w, b, eps), F.layer_norm(x, (96,), w, b, eps))
    tiny = 3.0 + 1e-3 * torch.randn(1, 96, dtype=D)   # variance ~1e-6: eps 1e-5 and 1e-6 must differ
    a = plain.layer_norm(tiny, torch.ones(96, dtype=D), torch.zeros(96, dtype=D), 1e-5)
    c = plain.layer_norm(tiny, torch.ones(96, dtype=D), torch.zeros(96, dtype=D), 1e-6)
    assert (a - c).abs().max() > 0.1
    y = plain.layer_norm(x, torch.ones(96, dtype=D), torch.zeros(96, dtype=D), 0.0)
    torch.testing.assert_close(y.mean(-1), torch.zeros(5, dtype=D), atol=1e-12, rtol=0)
    torch.testing.assert_close((y * y).mean(-1), torch.ones(5, dtype=D), atol=1e-9, rtol=0)


def test_linear():
    x, w, b = torch.randn(4, 7, dtype=D), torch.randn(3, 7, dtype=D), torch.randn(3, dtype=D)
    torch.testing.assert_close(plain.linear(x, w, b), F.linear(x, w, b))
    torch.testing.assert_close(plain.linear(x, torch.zeros_like(w), b), b.expand(4, 3))


def test_gelu_is_the_tanh_variant():
    x = torch.linspace(-6, 6, 241, dtype=D)
    torch.testing.assert_close(plain.gelu_tanh(x), F.gelu(x, approximate="tanh"))
    assert plain.gelu_tanh(torch.zeros(1, dtype=D)).item() == 0.0
    assert abs(plain.gelu_tanh(torch.tensor([10.0], dtype=D)).item() - 10.0) < 1e-9
    assert abs(plain.gelu_tanh(torch.tensor([-10.0], dtype=D)).item()) < 1e-9
    gap = (plain.gelu_tanh(x) - F.gelu(x)).abs().max().item()
    assert 1e-5 < gap < 2e-3          # close to, but not, the erf form


def test_rotary_table_is_cat_cos_sin():
    table = plain.rotary_table(8, 50, 10000.0)
    p, i = 37, 3
    f = 10000.0 ** (-2 * i / 8)
    assert abs(table[p, i].item() - math.cos(p * f)) < 1e-12
    assert abs(table[p, 4 + i].item() - math.sin(p * f)) < 1e-12
    assert table.shape == (50, 8)


def test_rotary_properties():
    hd, rot = 16, 8
    table = plain.rotary_table(rot, 64, 10000.0)
    x = torch.randn(3, 2, hd, dtype=D)
    pos = torch.tensor([0, 5, 9])
    y = plain.apply_rotary(x, pos, table)
    torch.testing.assert_close(y[0], x[0])                                 # position 0 is the identity
    torch.testing.assert_close(y[..., rot:], x[..., rot:])                 # channels >= R untouched
    half = rot // 2
    torch.testing.assert_close(y[..., :half] ** 2 + y[..., half:rot] ** 2,
                               x[..., :half] ** 2 + x[..., half:rot] ** 2)  # pairs (i, i + R/2) keep their norm
    # equals the rotate-half formula on the first R channels (ops/rotary.py:58-72)
    rows = table[pos]
    cos = torch.cat([rows[:, :half], rows[:, :half]], -1).unsqueeze(1)
    sin = torch.cat([rows[:, half:], rows[:, half:]], -1).unsqueeze(1)
    xr = x[..., :rot]
    rotated = torch.cat((-xr[..., half:], xr[..., :half]), dim=-1)
    torch.testing.assert_close(y[..., :rot], xr * cos + rotated * sin)
    # scores depend on the distance only
    q, k = torch.randn(1, 1, hd, dtype=D), torch.randn(1, 1, hd, dtype=D)

    def score(m, n):
        return (plain.apply_rotary(q, torch.tensor([m]), table) * plain.apply_rotary(k, torch.tensor([n]), table)).sum()

    assert abs(score(9, 4).item() - score(25, 20).item()) < 1e-9
    assert abs(score(9, 4).item() - score(4, 9).item()) > 1e-6           # the sign of the distance matters


def test_attention_reduces_to_library_causal():
    t, h, hd = 11, 4, 16
    q, k, v = (torch.randn(t, h, hd, dtype=D) for _ in range(3))
    allowed = plain.visibility(torch.arange(t), None)
    got = plain.attention_core(q, k, v, allowed, hd ** -0.5)
    want = F.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1), is_causal=True)
    torch.testing.assert_close(got, want.transpose(0, 1))


def test_attention_one_key_and_grouping():
    hd = 8
    q = torch.randn(1, 3, hd, dtype=D)
    k = torch.randn(1, 1, hd, dtype=D)
    v = torch.randn(1, 1, hd, dtype=D)
    out = plain.attention_core(q, k, v, torch.ones(1, 1, dtype=torch.bool), hd ** -0.5)
    torch.testing.assert_close(out, v.expand(1, 3, hd))                    # one key: the output is v
    # MQA equals MHA with the single kv head repeated; GQA maps head h to kv head h // G
    t = 6
    q = torch.randn(t, 4, hd, dtype=D)
    k2, v2 = torch.randn(t, 2, hd, dtype=D), torch.randn(t, 2, hd, dtype=D)
    allowed = plain.visibility(torch.arange(t), None)
    grouped = plain.attention_core(q, k2, v2, allowed, hd ** -0.5)
    repeated = plain.attention_core(q, k2.repeat_interleave(2, dim=1), v2.repeat_interleave(2, dim=1), allowed, hd ** -0.5)
    torch.testing.assert_close(grouped, repeated)


def test_visibility_of_blocks():
    pos = torch.arange(6)
    blocks = torch.tensor([0, 0, 0, -1, -1, -1])
    allowed = plain.visibility(pos, blocks)
    assert allowed[:3, :3].all()                 # the block sees itself both ways
    assert not allowed[0, 3] and not allowed[3, 4] and allowed[4, 3] and allowed[5, 0]
    assert torch.equal(plain.visibility(pos, None), torch.tril(torch.ones(6, 6, dtype=torch.bool)))


def _model(name):
    folder = helpers.model_dir(name)
    return helpers.flat_config(name), {k: v.double() for k, v in helpers.stored_weights(folder).items()}


def test_block_is_parallel_and_mlp_reads_the_normed_input():
    cfg, w = _model("A")
    t = 7
    x = torch.randn(t, cfg["dim"], dtype=D)
    pos = torch.arange(t)
    allowed = plain.visibility(pos, None)
    table = plain.rotary_table(plain.rotary_dim_of(cfg), t, cfg["rope_theta"])
    p = "text.blocks.0."
    xn = plain.layer_norm(x, w[p + "ln.weight"], w[p + "ln.bias"], plain.eps_of(cfg))
    full = plain.block(x, w, 0, cfg, pos, allowed, table)
    no_attn = dict(w)
    no_attn[p + "attn.proj.weight"] = torch.zeros_like(w[p + "attn.proj.weight"])
    no_attn[p + "attn.proj.bias"] = torch.zeros_like(w[p + "attn.proj.bias"])
    torch.testing.assert_close(plain.block(x, no_attn, 0, cfg, pos, allowed, table), x + plain.mlp(xn, w, p))
    no_mlp = dict(w)
    no_mlp[p + "mlp.fc2.weight"] = torch.zeros_like(w[p + "mlp.fc2.weight"])
    no_mlp[p + "mlp.fc2.bias"] = torch.zeros_like(w[p + "mlp.fc2.bias"])
    attn_only = plain.block(x, no_mlp, 0, cfg, pos, allowed, table)
    torch.testing.assert_close(full, attn_only + plain.mlp(xn, w, p))     # branches add, mlp sees ln(x) not x + attn


def test_qkv_split_order():
    cfg, w = _model("C")
    p = "text.blocks.0."
    hd, h, hkv = plain.head_dim_of(cfg), cfg["n_heads"], cfg["n_kv_heads"]
    t = 5
    xn = torch.randn(t, cfg["dim"], dtype=D)
    pos = torch.arange(t)
    allowed = plain.visibility(pos, None)
    table = plain.rotary_table(plain.rotary_dim_of(cfg), t, cfg["rope_theta"])
    base = plain.attention(xn, w, p, cfg, pos, allowed, table)
    # zeroing the v third (the last Hkv*hd rows of the fused weight and bias) leaves only the proj bias
    z = dict(w)
    z[p + "attn.qkv.weight"] = w[p + "attn.qkv.weight"].clone()
    z[p + "attn.qkv.bias"] = w[p + "attn.qkv.bias"].clone()
    z[p + "attn.qkv.weight"][(h + hkv) * hd:] = 0
    z[p + "attn.qkv.bias"][(h + hkv) * hd:] = 0
    out = plain.attention(xn, z, p, cfg, pos, allowed, table)
    torch.testing.assert_close(out, w[p + "attn.proj.bias"].expand(t, -1))
    assert (base - out).abs().max() > 1e-4


def test_whole_model_causality_and_prefix():
    cfg, w = _model("B")
    ids = helpers.random_ids(5, 12, cfg["vocab_size"])
    base = plain.forward(cfg, w, ids)
    changed = list(ids)
    changed[9] = (changed[9] + 1) % cfg["vocab_size"]
    other = plain.forward(cfg, w, changed)
    torch.testing.assert_close(other[:9], base[:9])                        # a later token never moves earlier logits
    assert (other[9:] - base[9:]).abs().max() > 1e-6
    prefix = torch.randn(6, cfg["dim"], dtype=D)
    with_prefix = plain.forward(cfg, w, ids, prefix)
    moved = prefix.clone()
    moved[5] += torch.randn(cfg["dim"], dtype=D)   # (a constant shift would vanish in the norm)
    again = plain.forward(cfg, w, ids, moved)
    assert (again[0] - with_prefix[0]).abs().max() > 1e-6                  # the block is bidirectional
    # a shift of all positions leaves causal logits unchanged: only distances count
    shifted = plain.forward(cfg, w, ids, position_start=40)
    torch.testing.assert_close(shifted, base, atol=1e-9, rtol=1e-9)


def test_head_is_untied():
    cfg, w = _model("A")
    ids = helpers.random_ids(6, 4, cfg["vocab_size"])
    base = plain.forward(cfg, w, ids)
    w2 = dict(w)
    w2["text.wte"] = w["text.wte"].clone()
    unused = [i for i in range(cfg["vocab_size"]) if i not in ids][0]
    w2["text.wte"][unused] += 1.0
    torch.testing.assert_close(plain.forward(cfg, w2, ids), base)          # wte moves logits only through inputs


def test_nucleus_probs():
    logits = torch.tensor([2.0, 1.0, 0.5, -1.0, -3.0])
    torch.testing.assert_close(plain.nucleus_probs(logits, 0.7, 1.0), torch.softmax(logits.double() / 0.7, -1))
    greedy = plain.nucleus_probs(logits, 0.0, 0.9)
    assert greedy[0] == 1.0 and greedy.sum() == 1.0
    p = torch.softmax(logits.double(), -1)
    kept = plain.nucleus_probs(logits, 1.0, float(p[0] + 0.5 * p[1]))
    assert (kept > 0).sum() == 2 and abs(kept.sum().item() - 1.0) < 1e-12   # the token that crosses top_p is kept
    torch.testing.assert_close(kept[:2], p[:2] / p[:2].sum())
