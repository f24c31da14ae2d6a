"""The entry point that allocates nothing, called through ctypes as a caller outside Python would.

``ka_attention_decode_bf16_no_alloc`` is decode attention with the keys of a row cut into parts,
whose partial results go through a static array inside the library instead of a buffer from the
caller. Its output must equal, bit for bit, that of ``ka_attention_decode_bf16`` with a buffer of the
caller's (same kernels, same order of the parts), on two calls in a row, the second with a smaller
input, so that what the first call left in the array lies under the second's records.
"""

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

_c_void_p, _c_int, _c_long, _c_float = ctypes.c_void_p, ctypes.c_int, ctypes.c_long, ctypes.c_float
_COMMON = [_c_void_p, _c_long, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_void_p,
           _c_long, _c_float, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int]
_TAIL = [_c_void_p, _c_void_p, _c_long, _c_void_p, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_void_p]
SCRATCH_FLOATS = 1 << 20


def _library():
    from kestrel_amd.csrc import build

    lib = build.load("fast")
    no_alloc = lib.ka_attention_decode_bf16_no_alloc
    no_alloc.argtypes = _COMMON + _TAIL
    no_alloc.restype = _c_int
    with_buffer = lib.ka_attention_decode_bf16
    with_buffer.argtypes = _COMMON + [_c_void_p, _c_long] + _TAIL
    with_buffer.restype = _c_int
    lib.ka_last_error.restype = ctypes.c_char_p
    return lib, no_alloc, with_buffer


class _Case:
    """Rows of cached keys and values on shuffled pages of 16 and one query token per row."""

    def __init__(self, kv_lens, h, hkv, hd, seed):
        gen = torch.Generator().manual_seed(seed)
        bf = torch.bfloat16
        self.n, self.h, self.hkv, self.hd = len(kv_lens), h, hkv, hd
        pages_per_row = [-(-kv // 16) for kv in kv_lens]
        n_pages = sum(pages_per_row) + 2
        order = torch.randperm(n_pages, generator=gen).tolist()
        self.max_pages = max(pages_per_row) + 1
        table = torch.full((self.n, self.max_pages), -1, dtype=torch.int32)
        self.keys = [torch.randn(kv, hkv, hd, generator=gen).to(bf) for kv in kv_lens]
        self.values = [torch.randn(kv, hkv, hd, generator=gen).to(bf) for kv in kv_lens]
        k_cache = torch.zeros(n_pages, hkv, 16, hd, dtype=bf)
        v_cache = torch.zeros(n_pages, hkv, hd, 16, dtype=bf)
        at = 0
        for r, kv in enumerate(kv_lens):
            for logical in range(pages_per_row[r]):
                page = order[at]
                at += 1
                table[r, logical] = page
                lo, hi = logical * 16, min(kv, logical * 16 + 16)
                k_cache[page, :, :hi - lo, :] = self.keys[r][lo:hi].transpose(0, 1)
                v_cache[page, :, :, :hi - lo] = self.values[r][lo:hi].permute(1, 2, 0)
        self.q = torch.randn(self.n, h * hd, generator=gen).to(bf).to(DEV)
        self.table, self.k_cache, self.v_cache = table.to(DEV), k_cache.to(DEV), v_cache.to(DEV)
        self.token_row = torch.arange(self.n, dtype=torch.int32, device=DEV)
        self.kv_hi = torch.tensor(kv_lens, dtype=torch.int32, device=DEV)
        self.kv_lens = kv_lens

    def common(self, out, splits, waves):
        return [self.q.data_ptr(), self.q.stride(0), self.k_cache.data_ptr(), self.v_cache.data_ptr(),
                self.table.data_ptr(), self.max_pages, self.token_row.data_ptr(), None, self.kv_hi.data_ptr(),
                out.data_ptr(), out.stride(0), float(self.hd) ** -0.5, self.n, self.h, self.hkv, self.hd, 16, splits, waves]

    def reference(self):
        out = torch.empty(self.n, self.h, self.hd, dtype=torch.float64)
        q = self.q.cpu().double().view(self.n, self.h, self.hd)
        group = self.h // self.hkv
        for r in range(self.n):
            for head in range(self.h):
                keys, values = self.keys[r][:, head // group].double(), self.values[r][:, head // group].double()
                out[r, head] = torch.softmax(keys @ q[r, head] * self.hd ** -0.5, dim=0) @ values
        return out.view(self.n, self.h * self.hd)


def test_decode_attention_that_allocates_nothing():
    lib, no_alloc, with_buffer = _library()
    tail = [None, None, 0, None, 0, None, None, None, None]      # nothing fused; the default stream
    splits, waves = 4, 4
    # two calls in a row on the same array: the second is smaller in every way (rows, heads' worth of
    # records, keys), so its records lie over the first call's
    cases = [_Case([1500, 700, 33, 1024, 260, 1], 8, 2, 64, seed=41), _Case([400, 90, 17], 4, 4, 64, seed=42)]
    for index, case in enumerate(cases):
        got = torch.full((case.n, case.h * case.hd), float("nan"), dtype=torch.bfloat16, device=DEV)
        status = no_alloc(*case.common(got, splits, waves), *tail)
        assert status == 0, lib.ka_last_error().decode()
        torch.cuda.synchronize()
        want = torch.full_like(got, float("nan"))
        buffer = torch.empty(case.n * case.h * splits * (case.hd + 2), dtype=torch.float32, device=DEV)
        status = with_buffer(*case.common(want, splits, waves), buffer.data_ptr(), buffer.numel(), *tail)
        assert status == 0, lib.ka_last_error().decode()
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"call {index}: the two entry points differ"
        torch.testing.assert_close(got.cpu().double(), case.reference(), atol=2e-2, rtol=2e-2)


def test_it_allocates_nothing_and_runs_under_graph_capture():
    """What gives the entry point its name: after a first call (which looks up the array's address on this
    device) a call leaves the device's free memory as it was, and it can be recorded into a HIP graph (an
    allocation inside a capture fails the capture). The graph is replayed several times with eager work of
    the program's own between the replays, and every replay gives the eager call's bits."""
    lib, no_alloc, _ = _library()
    case = _Case([1500, 700, 33, 1024], 8, 2, 64, seed=44)
    splits, waves = 4, 4
    eager = torch.full((case.n, case.h * case.hd), float("nan"), dtype=torch.bfloat16, device=DEV)
    tail = [None, None, 0, None, 0, None, None, None]
    assert no_alloc(*case.common(eager, splits, waves), *tail, None) == 0, lib.ka_last_error().decode()
    again = torch.full_like(eager, float("nan"))
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    assert no_alloc(*case.common(again, splits, waves), *tail, None) == 0, lib.ka_last_error().decode()
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before, "the call changed the device's free memory"
    assert torch.equal(again, eager)
    replayed = torch.full_like(eager, float("nan"))
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        status = no_alloc(*case.common(replayed, splits, waves), *tail, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert status == 0, lib.ka_last_error().decode()
    other = _Case([90, 400], 4, 4, 64, seed=45)                 # eager work on the same static array between the replays
    scratch_user = torch.empty(other.n, other.h * other.hd, dtype=torch.bfloat16, device=DEV)
    for _ in range(3):
        replayed.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(replayed, eager)
        assert no_alloc(*other.common(scratch_user, splits, waves), *tail, None) == 0
        torch.cuda.synchronize()


def test_a_batch_beyond_the_static_array_is_refused():
    lib, no_alloc, _ = _library()
    case = _Case([40, 50], 4, 4, 64, seed=43)
    out = torch.zeros(case.n, case.h * case.hd, dtype=torch.bfloat16, device=DEV)
    args = case.common(out, 4, 4)
    args[12] = SCRATCH_FLOATS          # n: as many tokens as the array has floats, far beyond the tensors
    # refused on the host before anything is launched: nothing reads the (too small) tensors
    assert no_alloc(*args, None, None, 0, None, 0, None, None, None, None) == -1
    message = lib.ka_last_error().decode()
    assert "floats of scratch" in message and str(SCRATCH_FLOATS) in message
    torch.cuda.synchronize()
    assert bool((out == 0).all())
