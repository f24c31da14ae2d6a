"""Each HIP kernel alone against a plain fp64 reference, at sizes other than the engine's."""

from types import SimpleNamespace

import pytest
import torch
import torch.nn.functional as F

from tests.plain import moondream_plain as plain

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _tol(dtype):
    return (1e-5, 1e-5) if dtype == torch.float32 else (2e-2, 2e-2)


def _close(actual, expected, dtype, scale=1.0):
    atol, rtol = _tol(dtype)
    torch.testing.assert_close(actual.double().cpu(), expected.double().cpu(), atol=atol * scale, rtol=rtol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embed_and_scatter(dtype):
    from kestrel_amd.ops import core

    torch.manual_seed(0)
    table = torch.randn(333, 100).to(dtype).to(DEV)
    ids = torch.tensor([5, -1, 332, 0, -1, 17], dtype=torch.int32, device=DEV)
    out = torch.full((6, 100), 7.0, device=DEV)
    core.embed(table, ids, out)
    keep = ids.cpu() >= 0
    _close(out.cpu()[keep], table.float().cpu()[ids.cpu()[keep].long()], torch.float32)
    assert bool((out.cpu()[~keep] == 7.0).all())                 # given places are left alone
    given = torch.randn(2, 100).to(dtype).to(DEV)
    core.scatter_rows(given, torch.tensor([1, 4], dtype=torch.int32, device=DEV), out)
    _close(out[[1, 4]], given.float(), torch.float32)


def test_tokens_kept_on_the_device_reach_the_embedding():
    """Sampling stores a row's token at a place of the pending table; an id <= -2 makes the
    embedding read that place. Rows whose place is negative are not stored."""
    from kestrel_amd.ops import core

    torch.manual_seed(3)
    table = torch.randn(50, 24).to(DEV)
    logits = torch.randn(4, 50).to(DEV)
    pending = torch.full((6,), 49, dtype=torch.int32, device=DEV)
    places = torch.tensor([4, -1, 0, 5], dtype=torch.int32, device=DEV)
    out = torch.empty(4, dtype=torch.int32, device=DEV)
    core.argmax(logits, out, pending, places)
    best = logits.argmax(dim=1).cpu()
    assert out.cpu().tolist() == best.tolist()
    assert pending.cpu().tolist() == [int(best[2]), 49, 49, 49, int(best[0]), int(best[3])]
    ids = torch.tensor([-2 - 4, 7, -1, -2 - 0, -2 - 1], dtype=torch.int32, device=DEV)
    x = torch.full((5, 24), 3.0, device=DEV)
    core.embed(table, ids, x, pending)
    want = table.cpu()[[int(best[0]), 7, 0, int(best[2]), 49]]
    want[2] = 3.0
    assert torch.equal(x.cpu(), want)
    # the sampling kernel stores the same way
    temps = torch.tensor([0.0, 0.7, 0.0, 1.1], device=DEV)
    keys = torch.tensor([1, 2, 3, 4], dtype=torch.int64, device=DEV)
    counters = torch.zeros(4, dtype=torch.int32, device=DEV)
    pending.fill_(49)
    core.sample(logits, temps, None, keys, counters, out, pending, places)
    got = out.cpu().tolist()
    assert pending.cpu().tolist() == [got[2], 49, 49, 49, got[0], got[3]]


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("dim", [100, 2048, 5000])
def test_layernorm(dim, out_dtype):
    from kestrel_amd.ops import core

    torch.manual_seed(1)
    x = (torch.randn(9, dim) * 3 + 1.5).to(DEV)
    gamma, beta = (1 + 0.1 * torch.randn(dim)).to(DEV), (0.1 * torch.randn(dim)).to(DEV)
    for eps in (1e-5, 1e-2):
        out = torch.empty(9, dim, dtype=out_dtype, device=DEV)
        core.layernorm(x, gamma, beta, eps, out)
        _close(out, F.layer_norm(x.double(), (dim,), gamma.double(), beta.double(), eps), out_dtype, scale=4)
    rows = torch.tensor([8, 0, 3], dtype=torch.int32, device=DEV)
    out = torch.empty(3, dim, dtype=out_dtype, device=DEV)
    core.layernorm(x, gamma, None, 1e-6, out, rows)
    _close(out, F.layer_norm(x.double()[[8, 0, 3]], (dim,), gamma.double(), None, 1e-6), out_dtype, scale=4)


_ACTIVATE = {0: lambda x: x, 1: plain.gelu_tanh, 2: F.relu, 3: F.silu}       # the codes of kestrel_amd.ops.linear


def _linear_case(fn, m, n, k, a_dtype, w_dtype, out_dtype, act, accumulate, seed=0, lda=None):
    torch.manual_seed(seed)
    lda = lda or k
    a_full = torch.randn(m, lda).to(a_dtype).to(DEV)
    a = a_full[:, :k]
    w = (torch.randn(n, k) / k ** 0.5).to(w_dtype).to(DEV)
    bias = torch.randn(n).to(DEV)
    start = torch.randn(m, n).to(out_dtype).to(DEV)
    out = start.clone()
    fn(a, w, bias, out, act=act, accumulate=accumulate)
    ref = a.double() @ w.double().T + bias.double()
    ref = _ACTIVATE[act](ref)
    if accumulate:
        ref = ref + start.double()
    worst = torch.float32 if (a_dtype == w_dtype == out_dtype == torch.float32) else torch.bfloat16
    _close(out, ref, worst, scale=2)


@pytest.mark.parametrize("shape", [(1, 37, 19), (65, 130, 200), (7, 64, 96), (130, 77, 333), (16, 51, 2048), (3, 1000, 260),
                                   (17, 40, 64), (300, 257, 1028), (129, 128, 12), (2048, 100, 520), (2050, 4100, 36)])
def test_linear_generic(shape):
    from kestrel_amd.ops import core

    m, n, k = shape
    f32, bf = torch.float32, torch.bfloat16
    for a_dtype, w_dtype, out_dtype in [(f32, f32, f32), (bf, bf, bf), (bf, bf, f32), (bf, f32, bf), (f32, bf, f32)]:
        for act, accumulate in [(0, False), (1, False), (0, True)]:
            if accumulate and out_dtype != f32:
                continue
            _linear_case(core.linear_generic, m, n, k, a_dtype, w_dtype, out_dtype, act, accumulate)
    _linear_case(core.linear_generic, m, n, k, f32, f32, f32, 0, False, lda=k + 5)      # strided rows


@pytest.mark.parametrize("name,code", [("gelu_tanh", 1), ("relu", 2), ("silu", 3)])
def test_every_activation_in_every_linear_kernel(name, code):
    """The activations come from one table that every kernel family applies in its epilogue: the
    plain fp32 kernel, the weight-streaming ones (persistent, split, wide, with the norm in front),
    the tiled one and the one that adds up parts of K."""
    from kestrel_amd.ops import core, fast
    from kestrel_amd.ops.linear import activation_code, linear

    assert activation_code(name) == code and activation_code(None) == 0
    with pytest.raises(ValueError, match="unknown activation"):
        activation_code("swish-ish")
    bf, f32 = torch.bfloat16, torch.float32
    _linear_case(core.linear_generic, 19, 77, 130, f32, f32, f32, code, False)
    _linear_case(core.linear_generic, 200, 136, 264, f32, f32, f32, code, False)       # the tiled fp32 form

    def through_dispatch(a, w, bias, out, act, accumulate):
        linear(a, w, bias, out, act=act, accumulate=accumulate)

    for library in (True, False):                            # many rows: the vendor library's epilogues, then this package's tiles
        fast.LIBRARY_LINEAR, was = library, fast.LIBRARY_LINEAR
        try:
            for m, n, k in ((8, 2048, 2048), (40, 4100, 2048), (200, 333, 520), (520, 2048, 8192), (2048, 512, 1024)):
                _linear_case(through_dispatch, m, n, k, bf, bf, bf, code, False)
        finally:
            fast.LIBRARY_LINEAR = was
    for mode in (0, 2):                                      # the split kernel, then the wide one wherever it can run
        fast.set_skinny_persistent(0 if mode == 0 else 1)
        fast.set_skinny_wide(mode)
        try:
            _linear_case(through_dispatch, 12, 515, 3000, bf, bf, bf, code, False)
        finally:
            fast.set_skinny_persistent(1)
            fast.set_skinny_wide(1)
    torch.manual_seed(6)
    x = (torch.randn(5, 264) * 2).to(DEV)
    gamma, beta = (1 + 0.1 * torch.randn(264)).to(DEV), (0.1 * torch.randn(264)).to(DEV)
    w = (torch.randn(72, 264) / 16).bfloat16().to(DEV)
    out = torch.empty(5, 72, dtype=bf, device=DEV)
    assert fast.layernorm_linear(x, gamma, beta, 1e-5, w, None, out, code)
    h = F.layer_norm(x.double(), (264,), gamma.double(), beta.double(), 1e-5).to(bf).double()
    _close(out, _ACTIVATE[code](h @ w.double().T), bf, scale=2)


def _gated_case(fn, m, n, k, a_dtype, w_dtype, out_dtype, code, seed=0):
    """``fn(a, weight_pairs, bias_pairs, out, act)`` against ``act(a Wg^T + bg) * (a Wu^T + bu)`` in float64; the
    output is poisoned first, so a column the kernel leaves out shows."""
    from kestrel_amd.ops.linear import pair_rows

    torch.manual_seed(seed)
    a = torch.randn(m, k).to(a_dtype).to(DEV)
    gate, value = ((torch.randn(n, k) / k ** 0.5).to(w_dtype).to(DEV) for _ in range(2))
    gate_bias, value_bias = torch.randn(n).to(DEV), torch.randn(n).to(DEV)
    out = torch.full((m, n), float("nan"), dtype=out_dtype, device=DEV)
    fn(a, pair_rows(gate, value), pair_rows(gate_bias, value_bias), out, code)
    ref = _ACTIVATE[code](a.double() @ gate.double().T + gate_bias.double()) * (a.double() @ value.double().T + value_bias.double())
    worst = torch.float32 if (a_dtype == w_dtype == out_dtype == torch.float32) else torch.bfloat16
    _close(out, ref, worst, scale=3)


@pytest.mark.parametrize("name,code", [("silu", 3), ("gelu_tanh", 1), ("none", 0)])
def test_a_gated_linear_in_every_kernel_family(name, code):
    """``out = act(gate) * value`` as an epilogue option of the linear kernels (weight rows in pairs): the plain
    fp32 kernels, the weight-streaming ones (persistent, split, wide, behind a LayerNorm prologue, as the second
    of two targets), the tiled one with and without the vendor library asked first (which has no such
    epilogue and declines)."""
    from kestrel_amd.ops import core, fast
    from kestrel_amd.ops.linear import ACT_GATED, linear_gated, pair_rows

    bf, f32 = torch.bfloat16, torch.float32
    for m, n, k in ((3, 37, 36), (19, 77, 130), (200, 136, 264), (130, 65, 333)):       # few rows, the tiled fp32 form, odd sizes
        _gated_case(linear_gated, m, n, k, f32, f32, f32, code)
    _gated_case(linear_gated, 9, 40, 64, bf, f32, bf, code)                            # mixed types: the plain kernel
    for library in (True, False):
        fast.LIBRARY_LINEAR, was = library, fast.LIBRARY_LINEAR
        try:
            for m, n, k in ((1, 24, 64), (8, 1024, 2048), (16, 515, 520), (40, 2050, 2048), (64, 512, 10240), (200, 333, 520),
                            (520, 1024, 2048), (2048, 512, 1024)):
                _gated_case(linear_gated, m, n, k, bf, bf, bf, code)
        finally:
            fast.LIBRARY_LINEAR = was
    for mode in (0, 2):                                      # the split kernel, then the wide one wherever it can run
        fast.set_skinny_persistent(0 if mode == 0 else 1)
        fast.set_skinny_wide(mode)
        try:
            _gated_case(linear_gated, 12, 258, 3000, bf, bf, bf, code)
            _gated_case(linear_gated, 40, 130, 1000, bf, bf, f32, code)
        finally:
            fast.set_skinny_persistent(1)
            fast.set_skinny_wide(1)
    # behind the LayerNorm prologue, as the second of two targets (the first plain): one launch
    torch.manual_seed(7)
    x = (torch.randn(5, 264) * 2).to(DEV)
    gamma, beta = (1 + 0.1 * torch.randn(264)).to(DEV), (0.1 * torch.randn(264)).to(DEV)
    w_plain = (torch.randn(72, 264) / 16).bfloat16().to(DEV)
    gate, value = ((torch.randn(40, 264) / 16).bfloat16().to(DEV) for _ in range(2))
    out_plain = torch.empty(5, 72, dtype=bf, device=DEV)
    out_gated = torch.full((5, 40), float("nan"), dtype=bf, device=DEV)
    assert fast.layernorm_linear(x, gamma, beta, 1e-5, w_plain, None, out_plain, 0, pair_rows(gate, value), None, out_gated,
                                 code | ACT_GATED)
    h = F.layer_norm(x.double(), (264,), gamma.double(), beta.double(), 1e-5).to(bf).double()
    _close(out_plain, h @ w_plain.double().T, bf, scale=2)
    _close(out_gated, _ACTIVATE[code](h @ gate.double().T) * (h @ value.double().T), bf, scale=3)
    # what cannot be: an odd number of weight rows, accumulation
    from kestrel_amd.ops.core import KernelError
    with pytest.raises((KernelError, ValueError), match="even"):
        linear_gated(torch.zeros(4, 64, device=DEV), torch.zeros(7, 64, device=DEV), None, torch.zeros(4, 3, device=DEV), code)
    with pytest.raises((KernelError, ValueError), match="accumulation"):
        core.linear_generic(torch.zeros(4, 64, device=DEV), torch.zeros(8, 64, device=DEV), None, torch.zeros(4, 4, device=DEV),
                            code | ACT_GATED, True)


@pytest.mark.parametrize("persistent,wide", [(1, 0), (0, 0), (1, 2)])
@pytest.mark.parametrize("shape", [(1, 48, 64), (8, 2048, 2048), (5, 100, 200), (16, 6144, 2048), (33, 77, 8192),
                                   (64, 51200, 512), (17, 2048, 8192), (3, 16, 8), (9, 20000, 1032), (40, 4100, 2048),
                                   (8, 1000, 4096), (12, 515, 3000), (64, 9000, 1024), (50, 333, 1000), (20, 1000, 200)])
def test_linear_skinny_bf16(shape, persistent, wide):
    """The weight-streaming MFMA kernels: the persistent one (activations in registers, workgroups
    walk over strips; a form of its own for at most 8 rows), the one with K-splits that takes
    the rest, which is tested on the same shapes with the persistent one switched off, and the
    wide one, which the engine uses where the others do badly and which mode 2 sends all of these
    shapes to."""
    from kestrel_amd.ops import fast

    m, n, k = shape
    fast.set_skinny_wide(wide)
    bf, f32 = torch.bfloat16, torch.float32

    def fn(a, w, bias, out, act, accumulate):
        assert fast.linear_bf16(a, w, bias, out, act, accumulate)

    fast.set_skinny_persistent(persistent)
    try:
        for out_dtype, act, accumulate in [(bf, 0, False), (bf, 1, False), (f32, 0, True), (f32, 0, False)]:
            _linear_case(fn, m, n, k, bf, bf, out_dtype, act, accumulate)
        _linear_case(fn, m, n, k, bf, bf, bf, 0, False, lda=k + 16)
    finally:
        fast.set_skinny_persistent(1)
        fast.set_skinny_wide(1)


def test_linear_skinny_is_the_same_on_every_run():
    from kestrel_amd.ops import fast

    torch.manual_seed(3)
    a = torch.randn(8, 8192).bfloat16().to(DEV)
    w = torch.randn(2048, 8192).bfloat16().to(DEV)
    outs = []
    for _ in range(5):
        out = torch.empty(8, 2048, device=DEV)
        assert fast.linear_bf16(a, w, None, out, 0, False)
        outs.append(out.clone())
    assert all(torch.equal(outs[0], o) for o in outs[1:])


@pytest.mark.parametrize("shape", [(65, 128, 64), (200, 2048, 2048), (129, 100, 200), (300, 333, 520),
                                   (2048, 512, 1024), (128, 6144, 2048), (70, 8, 8), (520, 2048, 8192), (300, 200, 1088)])
@pytest.mark.parametrize("library", [False, True])
def test_linear_tiled_bf16(shape, library, monkeypatch):
    """Linears of many rows with ragged edges in M, N and K: through the tiled MFMA kernel (K cut into
    parts where there are few tiles), and through the vendor library with its epilogues, which
    ``linear_bf16`` asks first."""
    from kestrel_amd.ops import fast

    m, n, k = shape
    bf, f32 = torch.bfloat16, torch.float32
    monkeypatch.setattr(fast, "LIBRARY_LINEAR", library)

    def fn(a, w, bias, out, act, accumulate):
        assert fast.linear_bf16(a, w, bias, out, act, accumulate)

    for out_dtype, act, accumulate in [(bf, 0, False), (bf, 1, False), (f32, 0, True), (f32, 0, False)]:
        _linear_case(fn, m, n, k, bf, bf, out_dtype, act, accumulate)
    _linear_case(fn, m, n, k, bf, bf, bf, 0, False, lda=k + 8)


_LARGE_TILE_SHAPES = [(65, 128, 64), (300, 333, 512), (513, 700, 192), (2048, 512, 1024), (100, 2048, 2048), (70, 90, 32)]
_LARGE_TILE_CONFIGS = [12222, 23212, 22224, 22232, 13122, 2023212, 5023212]


@pytest.mark.parametrize("shape,config", [(sh, c) for sh in _LARGE_TILE_SHAPES for c in _LARGE_TILE_CONFIGS
                                          if sh[2] % (32 * (c % 1000000 // 100 % 10)) == 0])   # K in the tile's K-steps
def test_linear_large_tile_bf16(shape, config, monkeypatch):
    """The kernel that loads straight into LDS, at every wave tile, with ragged edges in M and N
    (K in steps of 64); the last two with K cut into two and five parts."""
    from kestrel_amd.ops import fast

    m, n, k = shape
    bf, f32 = torch.bfloat16, torch.float32
    monkeypatch.setattr(fast, "TILED_CONFIG", config)

    def fn(a, w, bias, out, act, accumulate):
        assert fast.linear_bf16(a, w, bias, out, act, accumulate)

    for out_dtype, act, accumulate in [(bf, 0, False), (bf, 1, False), (f32, 0, True), (f32, 0, False)]:
        _linear_case(fn, m, n, k, bf, bf, out_dtype, act, accumulate)
    _linear_case(fn, m, n, k, bf, bf, bf, 0, False, lda=k + 8)


def test_the_vendor_library_takes_the_linears_of_a_prompt():
    """What ``linear_bf16`` hands to hipBLASLt is really run there (status 0, not "no kernel for the
    case") for the cases a model brings: bias + activation into bf16, bias + sum into the fp32
    residual, rows that are not packed; and it computes the tanh form of GELU, as the kernels here do."""
    from kestrel_amd.ops import fast
    from kestrel_amd.ops.core import stream_ptr

    bf, f32 = torch.bfloat16, torch.float32
    torch.manual_seed(9)
    m, n, k = 300, 520, 264
    a = torch.randn(m, k + 8).to(bf).to(DEV)[:, :k]
    w = (torch.randn(n, k) / k ** 0.5).to(bf).to(DEV)
    bias = torch.randn(n).to(DEV)
    space = fast._library_workspace(a.device)
    ref = a.double() @ w.double().T + bias.double()
    for out_dtype, act, accumulate in [(bf, 1, False), (f32, 1, False), (f32, 0, True), (bf, 0, False), (f32, 3, False), (f32, 2, False)]:
        start = torch.randn(m, n).to(out_dtype).to(DEV)
        out = start.clone()
        status = fast.lib().ka_linear_library_bf16(a.data_ptr(), a.stride(0), w.data_ptr(), w.stride(0), bias.data_ptr(),
                                                   out.data_ptr(), 0 if out_dtype == f32 else 1, out.stride(0), m, n, k, act,
                                                   int(accumulate), space.data_ptr(), space.numel(), stream_ptr())
        assert status == 0, (out_dtype, act, accumulate, status)
        expected = _ACTIVATE[act](ref) + (start.double() if accumulate else 0)
        if out_dtype == f32:        # tight enough to tell the tanh form of GELU from the erf form (they differ by 5e-4)
            assert (out.double() - expected).abs().max().item() < 2e-5
        else:
            _close(out, expected, bf, scale=2)
    with pytest.raises(fast.KernelError, match="accumulate needs an fp32 output"):
        fast._check(fast.lib().ka_linear_library_bf16(a.data_ptr(), a.stride(0), w.data_ptr(), w.stride(0), None,
                                                      out.data_ptr(), 1, n, m, n, k, 0, 1, space.data_ptr(), space.numel(),
                                                      stream_ptr()))


def test_fast_linear_declines_what_it_does_not_cover():
    from kestrel_amd.ops import fast

    a = torch.randn(4, 20).bfloat16().to(DEV)         # K no multiple of 8
    w = torch.randn(6, 20).bfloat16().to(DEV)
    assert not fast.linear_bf16(a, w, None, torch.empty(4, 6, dtype=torch.bfloat16, device=DEV), 0, False)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads", [(3, 1, 32, 16, 4), (6, 2, 48, 12, 16), (4, 4, 16, 16, 1), (2, 2, 80, 0, 16)])
def test_rope_and_cache_write(heads, dtype):
    from kestrel_amd.ops import core

    h, hkv, hd, rot, ps = heads
    torch.manual_seed(4)
    n, pages = 11, 12
    qkv = torch.randn(n, (h + 2 * hkv) * hd).to(dtype)
    positions = torch.tensor([0, 1, 2, 3, 40, 41, 7, 8, 9, 100, 101], dtype=torch.int32)
    slots = torch.randperm(pages * ps)[:n].to(torch.int32)
    slots[5] = -1                                        # this token writes nothing
    table = plain.rotary_table(rot, 128, 777.0, torch.float32) if rot else None
    k_cache = torch.zeros(pages, hkv, ps, hd, dtype=dtype, device=DEV)
    v_cache = torch.zeros(pages, hkv, hd, ps, dtype=dtype, device=DEV)
    dev = qkv.to(DEV)
    core.rope_cache(dev, positions.to(DEV), slots.to(DEV), None if table is None else table.to(DEV), k_cache, v_cache,
                    h, hkv, hd, ps)
    q = qkv[:, :h * hd].double().view(n, h, hd)
    k = qkv[:, h * hd:(h + hkv) * hd].double().view(n, hkv, hd)
    v = qkv[:, (h + hkv) * hd:].double().view(n, hkv, hd)
    if rot:
        t64 = plain.rotary_table(rot, 128, 777.0)
        q, k = plain.apply_rotary(q, positions, t64), plain.apply_rotary(k, positions, t64)
    _close(dev[:, :h * hd].view(n, h, hd), q, dtype)
    for t in range(n):
        if slots[t] < 0:
            continue
        page, off = int(slots[t]) // ps, int(slots[t]) % ps
        _close(k_cache[page, :, off, :], k[t], dtype)
        _close(v_cache[page, :, :, off], v[t], dtype)
    written = {int(s) for s in slots if s >= 0}
    for slot in range(pages * ps):
        if slot not in written:
            assert float(k_cache[slot // ps, :, slot % ps, :].abs().max()) == 0.0


@pytest.mark.parametrize("heads", [(4, 4, 64, 32), (6, 2, 48, 16), (3, 1, 128, 128), (2, 2, 80, 32)])
def test_rope_and_cache_write_by_pages(heads):
    """The bf16 kernel that takes 16 tokens per workgroup: tokens that fill whole pages in order
    (the fast way to store the values), a run that starts in the middle of a page, a token that
    is not cached, scattered slots and a ragged end; and with no slots at all, q alone."""
    from kestrel_amd.ops import fast

    h, hkv, hd, rot = heads
    bf = torch.bfloat16
    torch.manual_seed(14)
    ps, pages = 16, 12
    # tokens 0..31: pages 5 and 2 in order; 32..47: page 7 from offset 3 on, running into page 9;
    # 48..63: scattered, one not cached; 64..70: a ragged tail on page 0
    slots = list(range(5 * ps, 6 * ps)) + list(range(2 * ps, 3 * ps))
    slots += list(range(7 * ps + 3, 8 * ps)) + list(range(9 * ps, 9 * ps + 3))
    scattered = (torch.randperm(2 * ps)[:16] + 10 * ps).tolist()
    scattered[4] = -1
    slots += scattered + list(range(0, 7))
    n = len(slots)
    positions = torch.randint(0, 200, (n,), dtype=torch.int32)
    qkv = torch.randn(n, (h + 2 * hkv) * hd).to(bf)
    table = plain.rotary_table(rot, 256, 777.0, torch.float32)
    k_cache = torch.zeros(pages, hkv, ps, hd, dtype=bf, device=DEV)
    v_cache = torch.zeros(pages, hkv, hd, ps, dtype=bf, device=DEV)
    dev = qkv.to(DEV)
    slots_t = torch.tensor(slots, dtype=torch.int32)
    assert fast.rope_cache_bf16(dev, positions.to(DEV), slots_t.to(DEV), table.to(DEV), k_cache, v_cache, h, hkv, hd, ps)
    t64 = plain.rotary_table(rot, 256, 777.0)
    q = plain.apply_rotary(qkv[:, :h * hd].double().view(n, h, hd), positions, t64)
    k = plain.apply_rotary(qkv[:, h * hd:(h + hkv) * hd].double().view(n, hkv, hd), positions, t64)
    v = qkv[:, (h + hkv) * hd:].view(n, hkv, hd)
    _close(dev[:, :h * hd].view(n, h, hd), q, bf)
    assert torch.equal(dev[:, h * hd:].cpu(), qkv[:, h * hd:])          # k and v rows themselves stay as they were
    for t in range(n):
        if slots[t] < 0:
            continue
        page, off = slots[t] // ps, slots[t] % ps
        _close(k_cache[page, :, off, :], k[t], bf)
        assert torch.equal(v_cache[page, :, :, off].cpu(), v[t])
    written = {s for s in slots if s >= 0}
    for slot in range(pages * ps):
        if slot not in written:
            assert float(k_cache[slot // ps, :, slot % ps, :].abs().max()) == 0.0
            assert float(v_cache[slot // ps, :, :, slot % ps].abs().max()) == 0.0
    only_q = qkv.to(DEV)
    assert fast.rope_cache_bf16(only_q, positions.to(DEV), None, table.to(DEV), None, None, h, hkv, hd, ps)
    assert torch.equal(only_q[:, :h * hd], dev[:, :h * hd]) and torch.equal(only_q[:, h * hd:].cpu(), qkv[:, h * hd:])
    assert not fast.rope_cache_bf16(qkv.to(DEV), positions.to(DEV), None, torch.zeros(256, 24, device=DEV), None, None,
                                    h, hkv, hd, ps)               # a rotary size that is no multiple of 16


@pytest.mark.parametrize("heads", [(4, 4, 64, 32), (6, 2, 48, 16), (2, 2, 80, 32)])
def test_rope_and_cache_write_by_listed_runs(heads):
    """The same kernel with the runs of tokens that the step function lists: a second prompt whose
    pages start at odd places of the packed batch (its whole pages are runs of their own and take the
    fast way), the loose ends of both prompts and single tokens of other rows in runs of their own."""
    from kestrel_amd.engine.step import _PageRuns
    from kestrel_amd.ops import fast

    h, hkv, hd, rot = heads
    bf = torch.bfloat16
    torch.manual_seed(15)
    ps, pages = 16, 16
    order = torch.randperm(pages).tolist()
    runs = _PageRuns(ps)
    slots, positions = [], []
    at = 0
    # a prompt of 37 tokens from position 0 (pages order[0..2]), one of 50 from position 16 (its first page
    # is held already: pages order[4..7]), five single tokens of other rows
    for first_page, start, q in ((0, 0, 37), (3, 16, 50)):
        runs.add(at, start, q)
        for p in range(start, start + q):
            slots.append(order[first_page + p // ps] * ps + p % ps)
            positions.append(p)
        at += q
    for i in range(5):
        runs.add(at, 100 + i, 1)
        slots.append(order[8 + i] * ps + (100 + i) % ps if i != 2 else -1)
        positions.append(100 + i)
        at += 1
    n = at
    first, count = runs.first(), runs.count()
    assert sum(count) == n and max(count) <= ps and count.count(ps) == 2 + 3        # whole pages: 2 of the first prompt, 3 of the second
    assert 37 in first and 53 in first                   # (whole pages that start at odd places of the batch)
    qkv = torch.randn(n, (h + 2 * hkv) * hd).to(bf)
    table = plain.rotary_table(rot, 256, 777.0, torch.float32)
    k_cache = torch.zeros(pages, hkv, ps, hd, dtype=bf, device=DEV)
    v_cache = torch.zeros(pages, hkv, hd, ps, dtype=bf, device=DEV)
    dev = qkv.to(DEV)
    i32 = lambda xs: torch.tensor(xs, dtype=torch.int32, device=DEV)
    assert fast.rope_cache_bf16(dev, i32(positions), i32(slots), table.to(DEV), k_cache, v_cache, h, hkv, hd, ps,
                                runs=(i32(first), i32(count)))
    t64 = plain.rotary_table(rot, 256, 777.0)
    pos_t = torch.tensor(positions, dtype=torch.int32)
    q = plain.apply_rotary(qkv[:, :h * hd].double().view(n, h, hd), pos_t, t64)
    k = plain.apply_rotary(qkv[:, h * hd:(h + hkv) * hd].double().view(n, hkv, hd), pos_t, t64)
    v = qkv[:, (h + hkv) * hd:].view(n, hkv, hd)
    _close(dev[:, :h * hd].view(n, h, hd), q, bf)
    for t in range(n):
        if slots[t] < 0:
            continue
        page, off = slots[t] // ps, slots[t] % ps
        _close(k_cache[page, :, off, :], k[t], bf)
        assert torch.equal(v_cache[page, :, :, off].cpu(), v[t])
    written = {s for s in slots if s >= 0}
    for slot in range(pages * ps):
        if slot not in written:
            assert float(k_cache[slot // ps, :, slot % ps, :].abs().max()) == 0.0
            assert float(v_cache[slot // ps, :, :, slot % ps].abs().max()) == 0.0


class PagedCase:
    """Rows of cached keys and values scattered over shuffled pages, and packed query tokens."""

    def __init__(self, kv_lens, q_lens, h, hkv, hd, ps, dtype, seed=0, window=None, bidir=None):
        gen = torch.Generator().manual_seed(seed)
        self.h, self.hkv, self.hd, self.ps, self.dtype = h, hkv, hd, ps, dtype
        n_rows = len(kv_lens)
        pages_per_row = [-(-kv // ps) for kv in kv_lens]
        n_pages = sum(pages_per_row) + 3
        order = torch.randperm(n_pages, generator=gen).tolist()
        max_pages = max(pages_per_row) + 2
        table = torch.full((n_rows, max_pages), -1, dtype=torch.int32)
        self.k = [torch.randn(kv, hkv, hd, generator=gen).to(dtype) for kv in kv_lens]
        self.v = [torch.randn(kv, hkv, hd, generator=gen).to(dtype) for kv in kv_lens]
        k_cache = torch.full((n_pages, hkv, ps, hd), float("nan")).to(dtype)
        v_cache = torch.full((n_pages, hkv, hd, ps), float("nan")).to(dtype)
        at = 0
        for r, kv in enumerate(kv_lens):
            for logical in range(pages_per_row[r]):
                page = order[at]
                at += 1
                table[r, logical] = page
                lo, hi = logical * ps, min(kv, (logical + 1) * ps)
                k_cache[page, :, :hi - lo, :] = self.k[r][lo:hi].transpose(0, 1)
                v_cache[page, :, :, :hi - lo] = self.v[r][lo:hi].permute(1, 2, 0)
        token_row, kv_hi, kv_lo, cu_q = [], [], [], [0]
        for r, (kv, ql) in enumerate(zip(kv_lens, q_lens)):
            for i in range(ql):
                pos = kv - ql + i
                hi_t = pos + 1
                if bidir and bidir[r] and bidir[r][0] <= pos < bidir[r][1]:
                    hi_t = bidir[r][1]
                token_row.append(r)
                kv_hi.append(hi_t)
                kv_lo.append(max(0, pos + 1 - window) if window else 0)
            cu_q.append(len(token_row))
        n = len(token_row)
        self.q = torch.randn(n, h * hd, generator=gen).to(dtype)
        i32 = lambda xs: torch.tensor(xs, dtype=torch.int32, device=DEV)
        query_blocks = {}                            # blocks of 32 and of 64 queries of a row: (rows, first tokens)
        for size in (32, 64):
            listed = [(r, first) for r in range(n_rows) for first in range(cu_q[r], cu_q[r + 1], size)]
            query_blocks[size] = (i32([r for r, _ in listed]), i32([first for _, first in listed]))
        self.token_row, self.kv_hi = i32(token_row), i32(kv_hi)
        self.kv_lo = i32(kv_lo) if window else None
        self.table, self.k_cache, self.v_cache = table.to(DEV), k_cache.to(DEV), v_cache.to(DEV)
        self.batch = SimpleNamespace(decode_only=all(ql == 1 for ql in q_lens), max_kv=max(kv_lens), cu_q=i32(cu_q),
                                     kv_len=i32(kv_lens), query_blocks=query_blocks)
        self.lists = (token_row, kv_lo if window else [0] * n, kv_hi)

    def reference(self, scale):
        token_row, kv_lo, kv_hi = self.lists
        out = torch.empty(len(token_row), self.h, self.hd, dtype=torch.float64)
        group = self.h // self.hkv
        q = self.q.double().view(-1, self.h, self.hd)
        for t, (r, lo, hi) in enumerate(zip(token_row, kv_lo, kv_hi)):
            for head in range(self.h):
                keys = self.k[r][lo:hi, head // group].double()
                vals = self.v[r][lo:hi, head // group].double()
                w = torch.softmax(keys @ q[t, head] * scale, dim=0)
                out[t, head] = w @ vals
        return out.view(len(token_row), self.h * self.hd)


def _run_attention(case, fn_name, scale):
    from kestrel_amd.ops import core, fast

    q = case.q.to(DEV)
    out = torch.full((q.shape[0], case.h * case.hd), float("nan"), dtype=case.dtype, device=DEV)
    if fn_name == "generic":
        core.attention_generic(q, case.k_cache, case.v_cache, case.table, case.token_row, case.kv_lo, case.kv_hi, out,
                               scale, case.h, case.hkv, case.hd)
    else:
        assert fast.attention_bf16(q, case.k_cache, case.v_cache, case.table, case.token_row, case.kv_lo, case.kv_hi,
                                   out, scale, case.h, case.hkv, case.hd, case.batch)
        if not case.batch.decode_only and fast.prefill_query_block(case.hd) != 32:
            # the prompt kernel took blocks of 64 queries: the same through its form for blocks of 32
            narrow = SimpleNamespace(**{**vars(case.batch), "query_blocks": {32: case.batch.query_blocks[32]}})
            again = torch.full_like(out, float("nan"))
            assert fast.attention_bf16(q, case.k_cache, case.v_cache, case.table, case.token_row, case.kv_lo, case.kv_hi,
                                       again, scale, case.h, case.hkv, case.hd, narrow)
            _close(again, out, case.dtype, scale=0.5)
    return out


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(3, 1, 32, 4), (6, 2, 48, 16), (2, 2, 80, 16), (4, 4, 16, 1), (1, 1, 272, 16)])
def test_attention_generic(shape, dtype):
    h, hkv, hd, ps = shape
    case = PagedCase([70, 5, 129], [70, 1, 9], h, hkv, hd, ps, dtype, seed=5)
    out = _run_attention(case, "generic", hd ** -0.5)
    _close(out, case.reference(hd ** -0.5), dtype)
    windowed = PagedCase([70, 33], [20, 1], h, hkv, hd, ps, dtype, seed=6, window=17)
    _close(_run_attention(windowed, "generic", 0.3), windowed.reference(0.3), dtype)
    block = PagedCase([40], [40], h, hkv, hd, ps, dtype, seed=7, bidir=[(3, 21)])
    _close(_run_attention(block, "generic", hd ** -0.5), block.reference(hd ** -0.5), dtype)


@pytest.mark.parametrize("shape", [(4, 4, 64), (6, 2, 32), (3, 1, 96), (4, 2, 128), (32, 32, 64), (2, 2, 16), (6, 3, 48),
                                   (4, 4, 80), (3, 1, 112), (2, 1, 160), (2, 2, 192), (2, 1, 224), (1, 1, 256)])
def test_attention_prompt_kernel(shape):
    """Whole prompts, portions that continue a cache, single tokens in a mixed batch, a block that
    sees both ways, a window; query counts that do not fill a wave."""
    h, hkv, hd = shape
    bf = torch.bfloat16
    case = PagedCase([70, 5, 300, 33], [70, 1, 130, 2], h, hkv, hd, 16, bf, seed=8)
    _close(_run_attention(case, "fast", hd ** -0.5), case.reference(hd ** -0.5), bf)
    block = PagedCase([90, 64], [90, 40], h, hkv, hd, 16, bf, seed=9, bidir=[(0, 37), (30, 50)])
    _close(_run_attention(block, "fast", hd ** -0.5), block.reference(hd ** -0.5), bf)
    windowed = PagedCase([200, 45], [120, 3], h, hkv, hd, 16, bf, seed=10, window=40)
    _close(_run_attention(windowed, "fast", 0.2), windowed.reference(0.2), bf)


@pytest.mark.parametrize("shape", [(4, 4, 64), (6, 2, 128), (32, 32, 64), (8, 1, 64), (2, 2, 16), (4, 1, 32), (6, 3, 48),
                                   (4, 4, 80), (3, 1, 96), (2, 2, 112), (2, 1, 160), (2, 2, 192), (2, 1, 224), (1, 1, 256)])
def test_attention_decode_kernel(shape):
    """One token per row, contexts from one key to many splits' worth, with and without a window."""
    h, hkv, hd = shape
    bf = torch.bfloat16
    for kv_lens in ([1], [5, 64, 65, 1000], [17, 256, 257, 511, 2, 2048], [700] * 9):
        case = PagedCase(kv_lens, [1] * len(kv_lens), h, hkv, hd, 16, bf, seed=11 + len(kv_lens))
        assert case.batch.decode_only
        _close(_run_attention(case, "fast", hd ** -0.5), case.reference(hd ** -0.5), bf)
    windowed = PagedCase([300, 20, 129], [1, 1, 1], h, hkv, hd, 16, bf, seed=12, window=100)
    _close(_run_attention(windowed, "fast", 0.25), windowed.reference(0.25), bf)


@pytest.mark.parametrize("waves", [4, 8, 16])
@pytest.mark.parametrize("shape", [(4, 4, 64), (2, 1, 16), (6, 3, 48), (4, 2, 32), (2, 2, 80), (2, 1, 128), (64, 8, 64), (48, 48, 32)])
def test_decode_attention_deals_out_every_page_once(shape, waves, monkeypatch):
    """A row's pages are cut evenly over the four waves of a workgroup, or dealt out tile by tile to eight or
    sixteen: every number of pages from none to more than waves x tile, contexts that end on a page's first
    and last slot, a window whose start lies inside a page, at every wave count. With 48 or 64 heads the rows
    here make a few hundred workgroups, which at four waves run with tiles of two pages instead of four."""
    from kestrel_amd.ops import fast

    h, hkv, hd = shape
    bf = torch.bfloat16
    shape_of = fast.decode_shape
    monkeypatch.setattr(fast, "decode_shape", lambda max_kv, workgroups=1, head_dim=64: (shape_of(max_kv, workgroups, head_dim)[0], waves))
    for kv_lens in ([1, 15, 16, 17, 63, 64, 65, 81], [1040, 1041, 1279, 600, 2047, 1, 255, 513]):
        case = PagedCase(kv_lens, [1] * len(kv_lens), h, hkv, hd, 16, bf, seed=31 + len(kv_lens))
        _close(_run_attention(case, "fast", hd ** -0.5), case.reference(hd ** -0.5), bf)
    for window in (1, 2, 16, 17, 33, 250):
        windowed = PagedCase([300, 20, 129, 1041, 17, 16], [1] * 6, h, hkv, hd, 16, bf, seed=32, window=window)
        _close(_run_attention(windowed, "fast", 0.25), windowed.reference(0.25), bf)


def test_fused_decode_attention_with_a_window_of_one():
    """A window of one position: the token reads no cached key at all, only its own, at positions on a
    page's first slot (16, 32, 48: where the row's block table in LDS ends just before the token's page) and
    elsewhere. The output is the token's own value, and nothing outside its slot of the cache is written."""
    from kestrel_amd.ops import fast

    h, hkv, hd, rot = 4, 2, 64, 32
    bf = torch.bfloat16
    kv_lens = [17, 33, 49, 18, 1, 64, 65]             # the token stands at kv - 1
    case = PagedCase(kv_lens, [1] * len(kv_lens), h, hkv, hd, 16, bf, seed=33, window=1)
    n = len(kv_lens)
    torch.manual_seed(34)
    qkv = torch.randn(n, (h + 2 * hkv) * hd).to(bf).to(DEV)
    slots = torch.tensor([int(case.table[r, (kv - 1) // 16]) * 16 + (kv - 1) % 16 for r, kv in enumerate(kv_lens)],
                         dtype=torch.int32, device=DEV)
    table = plain.rotary_table(rot, 128, 10000.0, torch.float32).to(DEV)
    k_f, v_f = case.k_cache.clone(), case.v_cache.clone()
    out = torch.empty(n, h * hd, dtype=bf, device=DEV)
    q_dim, kv_dim = h * hd, hkv * hd
    for waves in (4, 16):
        shape_of = fast.decode_shape
        fast.decode_shape = lambda max_kv, workgroups=1, head_dim=64, w=waves: (shape_of(max_kv, workgroups, head_dim)[0], w)
        try:
            assert fast.attention_decode_bf16(qkv, k_f, v_f, case.table, case.token_row, case.kv_lo, case.kv_hi, out,
                                              hd ** -0.5, h, hkv, hd, case.batch,
                                              fuse=(qkv[:, q_dim:q_dim + kv_dim], qkv[:, q_dim + kv_dim:], table, slots))
        finally:
            fast.decode_shape = shape_of
        v_new = qkv[:, q_dim + kv_dim:].view(n, hkv, hd)
        expected = v_new.repeat_interleave(h // hkv, dim=1).reshape(n, h * hd)
        assert torch.equal(out, expected)


EDGE_HEADS = [(4, 4, 64), (4, 2, 80), (2, 1, 128), (6, 3, 48), (4, 1, 16), (2, 2, 96), (2, 2, 256)]


@pytest.mark.parametrize("heads", EDGE_HEADS)
def test_a_far_key_among_hundreds_is_found(heads):
    """One query and one far key are scaled so that this key takes almost all the weight: a
    kernel that loses it (a page's edge, a split's edge, a tile's edge) returns another value.
    At every kind of head size the kernels treat differently (64 and below, no multiple of 32,
    128, 256) and with grouped heads."""
    h, hkv, hd = heads
    bf = torch.bfloat16
    for target in (0, 15, 16, 255, 256, 511, 777):
        case = PagedCase([900], [1], h, hkv, hd, 16, bf, seed=13)
        case.q[0] *= 0
        case.q[0, :hd] = 4.0
        # key `target` of head 0 lines up with the query; rebuild its cache cell
        case.k[0][target, 0] = 4.0
        page, off = int(case.table[0, target // 16]), target % 16
        case.k_cache[page, 0, off, :] = 4.0
        for name in ("generic", "fast"):
            out = _run_attention(case, name, hd ** -0.5)
            _close(out[0, :hd], case.v[0][target, 0].double(), bf)
        prompt = PagedCase([900], [130], h, hkv, hd, 16, bf, seed=13)
        prompt.q[-1] *= 0
        prompt.q[-1, :hd] = 4.0
        prompt.k[0][target, 0] = 4.0
        page = int(prompt.table[0, target // 16])
        prompt.k_cache[page, 0, target % 16, :] = 4.0
        out = _run_attention(prompt, "fast", hd ** -0.5)
        _close(out[-1, :hd], prompt.v[0][target, 0].double(), bf)


def test_a_scale_that_is_not_positive_goes_to_the_generic_kernel():
    """The prompt kernel assumes a positive scale (it scales a tile's maximum, not every score): a
    negative or zero scale is declined by the fast path and refused by the library's entry point, and
    the dispatcher's result is that of the generic kernel, which takes any scale."""
    from kestrel_amd.ops import fast
    from kestrel_amd.ops.attention import paged_attention

    bf = torch.bfloat16
    case = PagedCase([70, 40], [70, 9], 4, 2, 64, 16, bf, seed=41)
    q = case.q.to(DEV)
    for scale in (-0.2, 0.0):
        out = torch.full((q.shape[0], case.h * case.hd), float("nan"), dtype=bf, device=DEV)
        assert not fast.attention_bf16(q, case.k_cache, case.v_cache, case.table, case.token_row, case.kv_lo, case.kv_hi,
                                       out, scale, case.h, case.hkv, case.hd, case.batch)
        paged_attention(q, case.k_cache, case.v_cache, case.table, case.token_row, case.kv_lo, case.kv_hi, out, scale,
                        case.h, case.hkv, case.hd, case.batch)
        _close(out, case.reference(scale), bf)
    rows, firsts = case.batch.query_blocks[64]
    out = torch.empty((q.shape[0], case.h * case.hd), dtype=bf, device=DEV)
    status = fast.lib().ka_attention_prefill_bf16(
        q.data_ptr(), q.stride(0), case.k_cache.data_ptr(), case.v_cache.data_ptr(), case.table.data_ptr(), case.table.shape[1],
        rows.data_ptr(), firsts.data_ptr(), int(rows.numel()), case.batch.cu_q.data_ptr(), case.batch.kv_len.data_ptr(), None,
        case.kv_hi.data_ptr(), out.data_ptr(), out.stride(0), -0.2, case.h, case.hkv, case.hd, 16, 70, 64, None)
    assert status != 0 and "positive" in fast.lib().ka_last_error().decode()


@pytest.mark.parametrize("heads", EDGE_HEADS)
def test_scores_that_climb_along_the_keys(heads):
    """Every key lines up with the queries a little better than the one before it, so that each
    tile of keys lies far above everything a query has seen so far: the prompt kernel, which takes
    its exponentials from the reference point a query already has and looks for a new maximum only
    when their sum says so, has to move that point again and again (by more than an exponential
    can hold between some tiles, by little between others). And the other way round: scores that
    fall, where the first tile's reference point serves to the end."""
    h, hkv, hd = heads
    bf = torch.bfloat16
    for step, q_len in ((0.05, 300), (0.004, 300), (-0.05, 300), (0.3, 70), (0.05, 1)):
        case = PagedCase([700], [q_len], h, hkv, hd, 16, bf, seed=31)
        ramp = (torch.arange(700, dtype=torch.float32) * step).to(bf)
        case.q[:, :hd] = 1.0
        case.k[0][:, 0, :] = ramp[:, None]
        for key in range(700):
            case.k_cache[int(case.table[0, key // 16]), 0, key % 16, :] = ramp[key]
        want = case.reference(hd ** -0.5)
        for name in ("generic", "fast"):
            _close(_run_attention(case, name, hd ** -0.5), want, bf)


@pytest.mark.parametrize("heads", EDGE_HEADS)
def test_a_windows_edge_is_kept(heads):
    """The key just outside a window lines up with the query far better than any other, the
    first key inside it second best: a kernel that lets the edge slip by one returns the wrong
    value. Edges on a page's first and last slot, on a tile's edge and in between."""
    h, hkv, hd = heads
    bf = torch.bfloat16
    for window in (100, 101, 115, 132, 388, 389):
        for q_len in (1, 130):
            case = PagedCase([900], [q_len], h, hkv, hd, 16, bf, seed=21, window=window)
            first = 900 - window                       # first key the last query sees
            case.q[-1] *= 0
            case.q[-1, :hd] = 4.0
            for key, strength in ((first - 1, 6.0), (first, 3.0)):
                case.k[0][key, 0] = strength
                page = int(case.table[0, key // 16])
                case.k_cache[page, 0, key % 16, :] = strength
            for name in ("generic", "fast"):
                out = _run_attention(case, name, hd ** -0.5)
                _close(out[-1, :hd], case.v[0][first, 0].double(), bf)
            _close(_run_attention(case, "fast", hd ** -0.5), case.reference(hd ** -0.5), bf)


def test_argmax_and_sampling():
    from kestrel_amd.ops import core
    from kestrel_amd.sampling import Sampler, mix_key

    torch.manual_seed(14)
    for vocab in (777, 51200, 70000):
        logits = torch.randn(5, vocab, device=DEV)
        logits[2, 3] = logits[2, vocab - 1] = 50.0            # a tie: the first index wins
        out = torch.empty(5, dtype=torch.int32, device=DEV)
        core.argmax(logits, out)
        expected = torch.argmax(logits.cpu(), dim=-1).tolist()
        expected[2] = 3                                       # whatever torch makes of the tie
        assert out.tolist() == expected
    sampler = Sampler(torch.device(DEV), seed=5)
    logits = torch.tensor([[2.0, 1.0, 0.5, -1.0, -3.0, float("-inf")]] * 4000, device=DEV)
    # temperature -> 0 is argmax; top_p tiny keeps the best token only
    assert set(sampler.sample(logits[:8], [0.0] * 8, [1.0] * 8, list(range(8)), [0] * 8).tolist()) == {0}
    assert set(sampler.sample(logits[:8], [1.0] * 8, [1e-4] * 8, list(range(8)), [0] * 8).tolist()) == {0}
    for temp, top_p in ((1.0, 1.0), (0.7, 1.0), (1.0, 0.8), (1.5, 0.5)):
        ids = sampler.sample(logits, [temp] * 4000, [top_p] * 4000, list(range(4000)), [3] * 4000).cpu()
        probs = plain.nucleus_probs(logits[0].cpu(), temp, top_p)
        counts = torch.bincount(ids.long(), minlength=6).double()
        assert counts[5] == 0 and bool((counts[probs == 0] == 0).all())
        keep = probs > 0
        chi2 = float((((counts[keep] - 4000 * probs[keep]) ** 2) / (4000 * probs[keep])).sum())
        assert chi2 < 30.0, (temp, top_p, counts.tolist(), probs.tolist())
    # a request's draw does not depend on its row or on the rest of the batch
    row = torch.randn(1, 1000, device=DEV)
    alone = sampler.sample(row, [0.9], [0.95], [42], [7]).item()
    mixed = sampler.sample(torch.cat([torch.randn(3, 1000, device=DEV), row]), [0.5, 0.0, 1.0, 0.9],
                           [1.0, 1.0, 0.3, 0.95], [1, 2, 3, 42], [0, 5, 9, 7])[3].item()
    assert alone == mixed
    assert 0.0 <= core.uniform(mix_key(5, 42), 7) < 1.0


def test_sampler_takes_slots_from_the_device_and_writes_ids_to_pinned_memory():
    """The table of latest tokens gets a row's token at the row's slot, whether the slots come as a
    list or as the int32 tensor that the step function has left on the device; a negative slot
    (a padding row) is passed over."""
    from kestrel_amd.sampling import Sampler

    torch.manual_seed(5)
    logits = torch.randn(5, 777, device=DEV)
    slots = [3, 0, -1, 6, 2]
    want = logits.argmax(dim=1).tolist()
    for sampled in (False, True):
        tables = []
        for on_device in (False, True):
            pending = torch.full((8,), -7, dtype=torch.int32, device=DEV)
            sampler = Sampler(torch.device(DEV), seed=3, pending=pending)
            given = torch.tensor(slots, dtype=torch.int32, device=DEV) if on_device else slots
            if sampled:
                ids = sampler.sample(logits.clone(), [0.0, 0.8, 0.8, 0.0, 0.8], [1.0, 0.9, 0.9, 1.0, 0.5], [1, 2, 3, 4, 5],
                                     [0, 1, 2, 3, 4], slots=given).tolist()
                assert ids[0] == want[0] and ids[3] == want[3]
            else:
                ids = sampler.greedy(logits, slots=given).tolist()
                assert ids == want
            table = pending.tolist()
            for row, slot in enumerate(slots):
                if slot >= 0:
                    assert table[slot] == ids[row]
            assert [table[i] for i in (1, 4, 5, 7)] == [-7] * 4
            tables.append((ids, table))
        assert tables[0] == tables[1]
    with pytest.raises(ValueError):
        Sampler(torch.device(DEV), seed=3, pending=torch.zeros(8, dtype=torch.int32, device=DEV)).greedy(
            logits, slots=torch.zeros(4, dtype=torch.int32, device=DEV))
    # the ids may go straight into pinned host memory: the same ids, there once the stream has got so far
    sampler = Sampler(torch.device(DEV), seed=3)
    args = ([0.0, 0.8, 0.8, 0.0, 0.8], [1.0, 0.9, 0.9, 1.0, 0.5], [1, 2, 3, 4, 5], [0, 1, 2, 3, 4])
    on_device = sampler.sample(logits.clone(), *args).tolist()
    host = torch.full((5,), -1, dtype=torch.int32).pin_memory()
    assert sampler.sample(logits.clone(), *args, out=host) is host
    torch.cuda.synchronize()
    assert host.tolist() == on_device
    host.fill_(-1)
    sampler.greedy(logits, out=host)
    torch.cuda.synchronize()
    assert host.tolist() == want
    with pytest.raises(Exception):
        sampler.greedy(logits, out=torch.empty(5, dtype=torch.int32))          # pageable host memory: refused


@pytest.mark.parametrize("passes_only", [False, True])
@pytest.mark.parametrize("vocab", [51200, 1003, 40000, 60000, 70000])
def test_every_draw_is_the_inversion_of_the_nucleus(vocab, passes_only):
    """The token drawn is the first, in index order, whose cumulative mass in the plain
    implementation's nucleus distribution exceeds the request's uniform number: for peaked, very
    peaked and flat rows, masked tokens, equal logits; by the kernel that keeps a row in registers and by
    the one that passes over it (which alone takes rows of more than 65536)."""
    from kestrel_amd.ops import core
    from kestrel_amd.sampling import Sampler, mix_key

    torch.manual_seed(31)
    rows = 24
    logits = torch.randn(rows, vocab)
    logits[:8] *= 4.0                                  # peaked rows
    logits[8:12] *= 0.02                               # almost flat rows
    logits[12, 100:200] = float("-inf")                # masked tokens
    logits[13, :] = 0.5                                # all equal
    logits[14, 7] = logits[14, 900] = 9.0              # two equal leaders
    logits[16:20] *= 25.0                              # a token or two hold the whole nucleus
    temps = [0.7] * 8 + [1.0] * 8 + [1.3] * 8
    tops = ([0.9, 0.5, 0.99, 0.3] * 6)
    tops[13] = 1.0                                     # (equal probabilities at the nucleus's edge are all kept by the
                                                       # kernels and taken in index order by the plain implementation)
    seeds, counters = list(range(100, 100 + rows)), list(range(rows))
    sampler = Sampler(torch.device(DEV), seed=9)
    core.set_sample_passes_only(passes_only)
    try:
        ids = sampler.sample(logits.to(DEV), temps, tops, seeds, counters).cpu().tolist()
    finally:
        core.set_sample_passes_only(False)
    exact = 0
    for r in range(rows):
        probs = plain.nucleus_probs(logits[r], temps[r], tops[r])
        u = core.uniform(mix_key(9, seeds[r]), counters[r])
        cdf = torch.cumsum(probs, dim=0)
        want = int(torch.searchsorted(cdf, torch.tensor(u, dtype=torch.float64), right=True))
        assert probs[ids[r]] > 0, (r, ids[r])                     # never outside the nucleus
        if ids[r] == want:
            exact += 1
        else:                                    # fp32 sums against fp64: off by a sliver of mass at most
            assert abs(float(cdf[ids[r]] - cdf[want])) < 3e-4, (r, ids[r], want)    # tens of thousands of fp32 additions
    assert exact >= rows - 6


def test_masks_before_sampling_and_logprobs_after():
    """Vectors of the reference's own tests (``tests/scheduler/test_logprobs.py``): suppression
    composes with an allow-list (``:923-939``); the log-probability of the chosen token follows the
    sampling epsilon (``:899-920``: temperatures 0, 5e-7, 2e-6 give 0, -inf and the temperature-scaled
    log-softmax); and both on a vocabulary that is no power of two against torch."""
    from kestrel_amd.ops import core
    from kestrel_amd.sampling import Sampler

    sampler = Sampler(torch.device(DEV), seed=1)
    logits = torch.tensor([[5.0, 4.0, 3.0]], device=DEV)
    ids, _ = sampler.sample_step(logits, [0.0], [1.0], [0], [0], suppress=[(0, 0)], allowed=[[0, 1]])
    assert ids.cpu().tolist() == [1]

    logits = torch.tensor([[1.0, 0.0, -1.0], [1.0, 0.0, -1.0], [0.0, -1e-6, -2e-6]], device=DEV)
    chosen = torch.tensor([0, 1, 1], dtype=torch.int32, device=DEV)
    temps = torch.tensor([0.0, 5e-7, 2e-6], device=DEV)
    out = torch.empty(3, device=DEV)
    core.token_logprobs(logits, chosen, temps, out)
    got = out.cpu()
    expected = torch.log_softmax(logits[2].cpu().double() / 2e-6, dim=-1)[1]
    assert got[0].item() == 0.0 and torch.isneginf(got[1]).item()
    assert abs(got[2].item() - expected.item()) < 1e-5

    torch.manual_seed(4)
    big = (torch.randn(5, 1003) * 3).to(DEV)
    work = big.clone()
    rows = torch.tensor([0, 0, 3, 4], dtype=torch.int32, device=DEV)
    tokens = torch.tensor([5, 1002, 0, 2000], dtype=torch.int32, device=DEV)     # the last lies outside: passed over
    core.suppress_tokens(work, rows, tokens)
    want = big.clone()
    want[0, 5] = want[0, 1002] = want[3, 0] = float("-inf")
    assert torch.equal(work, want)
    starts = torch.tensor([0, 0, 3, 3, 3, 4], dtype=torch.int32, device=DEV)      # rows 1 and 4 are restricted
    allowed = torch.tensor([7, 500, 1002, 64], dtype=torch.int32, device=DEV)
    core.allow_tokens(work, starts, allowed)
    keep = torch.full_like(want, float("-inf"))
    keep[1, [7, 500, 1002]] = want[1, [7, 500, 1002]]
    keep[4, 64] = want[4, 64]
    want[1], want[4] = keep[1], keep[4]
    assert torch.equal(work, want)
    temps = torch.tensor([0.7, 1.0, 0.0, 1.3, 2.0], device=DEV)
    chosen = torch.tensor([9, 500, int(want[2].argmax()), 11, 64], dtype=torch.int32, device=DEV)
    out = torch.empty(5, device=DEV)
    core.token_logprobs(work, chosen, temps, out)
    ref = []
    for r in range(5):
        t = float(temps[r])
        if t <= 1e-6:
            ref.append(0.0)
        else:
            ref.append(float(torch.log_softmax(want[r].cpu().double() / t, dim=-1)[int(chosen[r])]))
    assert torch.allclose(out.cpu().double(), torch.tensor(ref, dtype=torch.float64), atol=2e-5, rtol=1e-5)


@pytest.mark.parametrize("wide", [1, 0, 2])
@pytest.mark.parametrize("shape", [(8, 2048, 2048, 8192), (1, 40, 64, 200), (16, 2048, 2048, 8192), (33, 96, 120, 320),
                                   (64, 256, 8, 72), (64, 2048, 2048, 8192), (17, 515, 1032, 40), (48, 100, 264, 2056),
                                   (8, 2560, 64, 136), (16, 4104, 72, 40)])
def test_two_segment_skinny_linear(shape, wide):
    """out += a1 w1^T + b1 + a2 w2^T + b2 in one launch: by the kernel that shares the activations
    through LDS and cuts K into parts where the engine uses it (1: 17 rows and more, and fewer rows
    of more strips than CUs), nowhere (0: the kernel that gives a strip to a workgroup) and
    everywhere (2)."""
    from kestrel_amd.ops import fast

    m, n, k1, k2 = shape
    fast.set_skinny_wide(wide)
    torch.manual_seed(20)
    a1, a2 = torch.randn(m, k1).bfloat16().to(DEV), torch.randn(m, k2).bfloat16().to(DEV)
    w1 = (torch.randn(n, k1) / k1 ** 0.5).bfloat16().to(DEV)
    w2 = (torch.randn(n, k2) / k2 ** 0.5).bfloat16().to(DEV)
    b1, b2 = torch.randn(n).to(DEV), torch.randn(n).to(DEV)
    start = torch.randn(m, n).to(DEV)
    out = start.clone()
    assert fast.linear_pair_accumulate(a1, w1, b1, a2, w2, b2, out)
    ref = start.double() + a1.double() @ w1.double().T + b1.double() + a2.double() @ w2.double().T + b2.double()
    _close(out, ref, torch.float32, scale=200)          # bf16 operands, fp32 sums
    out2 = start.clone()
    assert fast.linear_pair_accumulate(a1, w1, None, a2, w2, None, out2)
    _close(out2, ref - b1.double() - b2.double(), torch.float32, scale=200)
    out3 = start.clone()
    assert fast.linear_pair_accumulate(a1, w1, None, a2, w2, None, out3)
    assert torch.equal(out2, out3)                      # the same bits on every run
    # with the norm that follows: the same sums bit for bit, and their LayerNorm (computed by the
    # kernel that adds up the parts of K where there is one, else by a launch behind the linear's)
    gamma, beta = (1 + 0.1 * torch.randn(n)).to(DEV), (0.1 * torch.randn(n)).to(DEV)
    for dtype, shift in ((torch.bfloat16, beta), (torch.float32, None)):
        out4 = start.clone()
        normed = torch.full((m, n), float("nan"), dtype=dtype, device=DEV)
        taken = fast.linear_pair_accumulate(a1, w1, b1, a2, w2, b2, out4, then_norm=(gamma, shift, 1e-5, normed))
        assert taken == (n % 4 == 0)
        if taken:
            assert torch.equal(out4, out)
            expected = F.layer_norm(out4.double(), (n,), gamma.double(), None if shift is None else shift.double(), 1e-5)
            _close(normed, expected, dtype, scale=4)
    fast.set_skinny_wide(1)


@pytest.mark.parametrize("shape", [(8, 2048, 6144, 8192), (1, 64, 40, 24), (16, 320, 100, 200), (5, 2048, 48, 8),
                                   (12, 1000, 24, 20000), (3, 2048, 8192, 16384), (8, 2560, 7680, 10240), (16, 2560, 64, 40),
                                   (1, 4096, 100, 200), (11, 3080, 48, 24), (5, 2056, 8, 16)])
def test_layernorm_prologue_skinny_linear(shape):
    """LayerNorm, then two linears from the normalised rows, in one launch."""
    from kestrel_amd.ops import fast

    m, k, na, nb = shape
    torch.manual_seed(21)
    x = (torch.randn(m, k) * 2 + 0.3).to(DEV)
    gamma, beta = (1 + 0.1 * torch.randn(k)).to(DEV), (0.1 * torch.randn(k)).to(DEV)
    wa = (torch.randn(na, k) / k ** 0.5).bfloat16().to(DEV)
    wb = (torch.randn(nb, k) / k ** 0.5).bfloat16().to(DEV)
    ba, bb = torch.randn(na).to(DEV), torch.randn(nb).to(DEV)
    out_a = torch.empty(m, na, dtype=torch.bfloat16, device=DEV)
    out_b = torch.empty(m, nb, dtype=torch.bfloat16, device=DEV)
    assert fast.layernorm_linear(x, gamma, beta, 1e-5, wa, ba, out_a, 0, wb, bb, out_b, 1)
    h = F.layer_norm(x.double(), (k,), gamma.double(), beta.double(), 1e-5).to(torch.bfloat16).double()
    _close(out_a, h @ wa.double().T + ba.double(), torch.bfloat16, scale=2)
    _close(out_b, plain.gelu_tanh(h @ wb.double().T + bb.double()), torch.bfloat16, scale=2)
    assert not fast.layernorm_linear(torch.randn(17, k, device=DEV), gamma, beta, 1e-5, wa, ba,
                                          torch.empty(17, na, dtype=torch.bfloat16, device=DEV), 0, wb, bb,
                                          torch.empty(17, nb, dtype=torch.bfloat16, device=DEV), 1)


@pytest.mark.parametrize("shape", [(4, 4, 64, 32), (6, 2, 128, 64), (8, 1, 64, 16), (2, 2, 16, 16), (4, 2, 48, 32), (4, 4, 80, 32),
                                   (2, 1, 112, 48), (2, 2, 160, 80), (1, 1, 256, 128)])
def test_decode_attention_that_rotates_and_stores(shape):
    """The decode kernel with rotary encoding and cache write fused in, against a float64
    computation (the query and the new key rotated at the row's last position, the new key and value
    behind the cached ones), and against the rotary kernel followed by the plain decode kernel: same
    outputs, same cache."""
    from kestrel_amd.ops import core, fast

    h, hkv, hd, rot = shape
    bf = torch.bfloat16
    kv_lens = [1, 16, 17, 300, 1024]
    case = PagedCase(kv_lens, [1] * len(kv_lens), h, hkv, hd, 16, bf, seed=22)
    n = len(kv_lens)
    torch.manual_seed(23)
    qkv = torch.randn(n, (h + 2 * hkv) * hd).to(bf).to(DEV)
    positions = torch.tensor([kv - 1 for kv in kv_lens], dtype=torch.int32, device=DEV)
    slots = torch.tensor([int(case.table[r, (kv - 1) // 16]) * 16 + (kv - 1) % 16 for r, kv in enumerate(kv_lens)],
                         dtype=torch.int32, device=DEV)
    table = plain.rotary_table(rot, 2048, 10000.0, torch.float32).to(DEV)
    # reference path
    qkv_ref, k_ref, v_ref = qkv.clone(), case.k_cache.clone(), case.v_cache.clone()
    core.rope_cache(qkv_ref, positions, slots, table, k_ref, v_ref, h, hkv, hd, 16)
    out_ref = torch.empty(n, h * hd, dtype=bf, device=DEV)
    assert fast.attention_decode_bf16(qkv_ref, k_ref, v_ref, case.table, case.token_row, None, case.kv_hi, out_ref,
                                      hd ** -0.5, h, hkv, hd, case.batch)
    # fused path
    k_f, v_f = case.k_cache.clone(), case.v_cache.clone()
    out_f = torch.empty(n, h * hd, dtype=bf, device=DEV)
    q_dim, kv_dim = h * hd, hkv * hd
    assert fast.attention_decode_bf16(qkv, k_f, v_f, case.table, case.token_row, None, case.kv_hi, out_f, hd ** -0.5,
                                      h, hkv, hd, case.batch,
                                      fuse=(qkv[:, q_dim:q_dim + kv_dim], qkv[:, q_dim + kv_dim:], table, slots))
    _close(out_f, out_ref, bf)
    # float64: rows of the fused q|k|v, rotated; keys and values that were cached before, then the new ones
    table64 = plain.rotary_table(rot, 2048, 10000.0)
    q64 = plain.apply_rotary(qkv[:, :q_dim].cpu().double().view(n, h, hd), positions.cpu(), table64)
    k64 = plain.apply_rotary(qkv[:, q_dim:q_dim + kv_dim].cpu().double().view(n, hkv, hd), positions.cpu(), table64)
    v64 = qkv[:, q_dim + kv_dim:].cpu().double().view(n, hkv, hd)
    expected = torch.empty(n, h, hd, dtype=torch.float64)
    for r, kv in enumerate(kv_lens):
        for head in range(h):
            g = head // (h // hkv)
            keys = torch.cat([case.k[r][:kv - 1, g].double(), k64[r, g].to(bf).double().unsqueeze(0)])
            vals = torch.cat([case.v[r][:kv - 1, g].double(), v64[r, g].unsqueeze(0)])
            w = torch.softmax(keys @ q64[r, head] * hd ** -0.5, dim=0)
            expected[r, head] = w @ vals
    _close(out_f, expected.view(n, h * hd), bf)
    for r, kv in enumerate(kv_lens):
        page, off = int(slots[r]) // 16, int(slots[r]) % 16
        _close(k_f[page, :, off, :], k64[r], bf)
        assert torch.equal(v_f[page, :, :, off].cpu().double(), v64[r])
        assert torch.equal(k_f[page, :, off, :], k_ref[page, :, off, :])
        assert torch.equal(v_f[page, :, :, off], v_ref[page, :, :, off])


@pytest.mark.parametrize("keys_per_workgroup", [4096, 256])
@pytest.mark.parametrize("shape", [(4, 4, 64, 32, 2048, 8192, 1), (6, 2, 48, 16, 200, 100, 0), (16, 16, 64, 32, 2048, 1000, 3),
                                   (2, 1, 16, 16, 1032, 24, 2), (3, 3, 32, 32, 64, 4100, 1)])
def test_decode_attention_with_a_linear_layer_beside_it(shape, keys_per_workgroup, monkeypatch):
    """One launch computes the decode attention (rotating and storing the tokens' own keys) and, in
    other workgroups, a linear layer on bf16 rows that an earlier launch normalised and left behind.
    Both results are, bit for bit, what the kernels give alone (attention with the same 8 waves a
    workgroup), and so is the cache; the rows left behind are the LayerNorm of the input."""
    from kestrel_amd.ops import fast
    from kestrel_amd.parts import SideLinear

    h, hkv, hd, rot, k, n_out, act = shape
    bf = torch.bfloat16
    monkeypatch.setattr(fast, "DECODE_KEYS_PER_WORKGROUP", keys_per_workgroup)
    shape_of = fast.decode_shape
    monkeypatch.setattr(fast, "decode_shape", lambda max_kv, workgroups=1, head_dim=64: (shape_of(max_kv, workgroups, head_dim)[0], 8))
    for kv_lens in ([1024, 16, 17, 300, 1], [700], [1000, 64, 65, 129, 2, 5, 33, 48]):
        # (as many rows as leave attention within the quarter of a 256-CU chip's places that the launch takes)
        kv_lens = kv_lens[:max(1, 128 // (h * shape_of(max(kv_lens))[0]))]
        case = PagedCase(kv_lens, [1] * len(kv_lens), h, hkv, hd, 16, bf, seed=31)
        n = len(kv_lens)
        torch.manual_seed(32)
        qkv = torch.randn(n, (h + 2 * hkv) * hd).to(bf).to(DEV)
        slots = torch.tensor([int(case.table[r, (kv - 1) // 16]) * 16 + (kv - 1) % 16 for r, kv in enumerate(kv_lens)],
                             dtype=torch.int32, device=DEV)
        table = plain.rotary_table(rot, 2048, 10000.0, torch.float32).to(DEV)
        x = (torch.randn(n, k) * 2 + 0.3).to(DEV)
        gamma, beta = (1 + 0.1 * torch.randn(k)).to(DEV), (0.1 * torch.randn(k)).to(DEV)
        w = (torch.randn(n_out, k) / k ** 0.5).bfloat16().to(DEV)
        bias = torch.randn(n_out).to(DEV)
        q_dim, kv_dim = h * hd, hkv * hd

        def run(beside):
            rows, k_c, v_c = qkv.clone(), case.k_cache.clone(), case.v_cache.clone()
            out = torch.empty(n, q_dim, dtype=bf, device=DEV)
            assert fast.attention_decode_bf16(rows, k_c, v_c, case.table, case.token_row, None, case.kv_hi, out,
                                              hd ** -0.5, h, hkv, hd, case.batch,
                                              fuse=(rows[:, q_dim:q_dim + kv_dim], rows[:, q_dim + kv_dim:], table, slots),
                                              beside=beside)
            return out, k_c, v_c

        # the launch before: LayerNorm + some linear, which leaves the normalised rows
        first = torch.empty(n, 24, dtype=bf, device=DEV)
        normed = torch.full((n, k), float("nan"), dtype=bf, device=DEV)
        w_first = (torch.randn(24, k) / k ** 0.5).bfloat16().to(DEV)
        assert fast.layernorm_linear(x, gamma, beta, 1e-5, w_first, None, first, 0, store=normed)
        hidden = F.layer_norm(x.double(), (k,), gamma.double(), beta.double(), 1e-5)
        _close(normed, hidden, bf, scale=2)
        without = torch.empty(n, 24, dtype=bf, device=DEV)
        assert fast.layernorm_linear(x, gamma, beta, 1e-5, w_first, None, without, 0)
        assert torch.equal(first, without)
        alone = torch.empty(n, n_out, dtype=bf, device=DEV)
        assert fast.linear_bf16(normed, w, bias, alone, act, False)
        out_ref, k_ref, v_ref = run(None)
        together = torch.full((n, n_out), float("nan"), dtype=bf, device=DEV)
        job = SideLinear(normed, w, bias, together, act)
        assert fast.attention_decode_takes(job, n, h, hd, 16, case.batch.max_kv)
        out, k_c, v_c = run(job)
        assert torch.equal(out, out_ref)
        # (places of the cache that no row holds are filled with NaN: compared as bit patterns)
        assert torch.equal(k_c.view(torch.int16), k_ref.view(torch.int16))
        assert torch.equal(v_c.view(torch.int16), v_ref.view(torch.int16))
        assert torch.equal(together, alone)
        _close(together, _ACTIVATE[act](normed.double() @ w.double().T + bias.double()), bf, scale=2)


def test_decode_attention_declines_a_linear_layer_it_cannot_carry():
    from kestrel_amd.ops import fast
    from kestrel_amd.parts import SideLinear

    def job(rows, k, n_out=64, a_dtype=torch.bfloat16):
        return SideLinear(torch.zeros(rows, k, dtype=a_dtype, device=DEV), torch.zeros(n_out, k, dtype=torch.bfloat16, device=DEV),
                          None, torch.empty(rows, n_out, dtype=torch.bfloat16, device=DEV), 0)

    assert fast.attention_decode_takes(job(8, 2048), 8, 4, 64, 16, 1024)
    assert not fast.attention_decode_takes(job(9, 2048), 9, 4, 64, 16, 1024)          # more rows than it takes
    assert not fast.attention_decode_takes(job(8, 2056), 8, 4, 64, 16, 1024)          # a row too long for its registers
    assert not fast.attention_decode_takes(job(8, 2048), 8, 4, 80, 16, 1024)          # a head size that needs a SIMD's registers
    assert not fast.attention_decode_takes(job(8, 2048, a_dtype=torch.float32), 8, 4, 64, 16, 1024)
    assert fast.attention_decode_takes(job(4, 2048), 4, 32, 64, 16, 1024)
    assert not fast.attention_decode_takes(job(5, 2048), 5, 32, 64, 16, 1024)         # attention that fills the chip by itself
    assert not fast.attention_decode_takes(job(2, 2048), 2, 32, 64, 16, 3 * fast.DECODE_KEYS_PER_WORKGROUP)


def test_decode_attention_splits_long_rows(monkeypatch):
    """Rows longer than a workgroup's share are cut into parts that a second kernel merges."""
    from kestrel_amd.ops import fast

    monkeypatch.setattr(fast, "DECODE_KEYS_PER_WORKGROUP", 256)
    h, hkv, hd = 4, 2, 64
    bf = torch.bfloat16
    case = PagedCase([1000, 3, 257, 700], [1, 1, 1, 1], h, hkv, hd, 16, bf, seed=24)
    assert fast.decode_shape(case.batch.max_kv)[0] == 4
    for _ in range(2):                                   # twice: nothing of the first run may be left in the way
        _close(_run_attention(case, "fast", hd ** -0.5), case.reference(hd ** -0.5), bf)
