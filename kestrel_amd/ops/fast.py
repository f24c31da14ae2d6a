"""Python faces of the bf16 MFMA kernels (library ``fast``).

Each function returns ``False`` when the kernels do not cover the operands (the
caller then takes the generic kernel) and raises when they do but the call fails.
"""

from __future__ import annotations

import ctypes
from typing import Dict, NamedTuple, Optional

import torch

from ..csrc import build as _build
from .core import KA_BF16, KA_F32, KernelError, _ptr, stream_ptr

_c_void_p, _c_int, _c_long, _c_float = ctypes.c_void_p, ctypes.c_int, ctypes.c_long, ctypes.c_float

_SIGNATURES = {
    "ka_linear_skinny_bf16": [_c_void_p, _c_long, _c_void_p, _c_long, _c_void_p, _c_void_p, _c_int, _c_long, _c_int,
                              _c_int, _c_int, _c_int, _c_int, _c_int, _c_void_p, _c_long, _c_void_p],
    "ka_linear_skinny_fused": [
        _c_void_p, _c_long, _c_int,                                   # A1, lda1, K1
        _c_void_p, _c_long, _c_int, _c_void_p, _c_long, _c_void_p,    # A2, lda2, K2, W2, ldw2, bias2
        _c_void_p, _c_void_p, _c_void_p, _c_float,                    # ln_x, gamma, beta, eps
        _c_void_p, _c_long, _c_void_p, _c_void_p, _c_int, _c_long, _c_int, _c_int, _c_int,   # target a
        _c_void_p, _c_long, _c_void_p, _c_void_p, _c_int, _c_long, _c_int, _c_int,           # target b
        _c_int, _c_int, _c_void_p, _c_long, _c_void_p],               # M, target_waves, partial sums and how many, stream
    "ka_linear_skinny_pair_norm": [
        _c_void_p, _c_long, _c_int, _c_void_p, _c_long, _c_int,                  # A1, lda1, K1, A2, lda2, K2
        _c_void_p, _c_long, _c_void_p, _c_void_p, _c_long, _c_void_p,            # W1, ldw1, bias1, W2, ldw2, bias2
        _c_void_p, _c_long, _c_int, _c_int, _c_int, _c_int, _c_void_p, _c_long,  # out, ldo, N, accumulate, M, target_waves, partial sums
        _c_void_p, _c_void_p, _c_float, _c_void_p, _c_int, _c_long, _c_void_p],  # gamma, beta, eps, normed, its type and stride, stream
    "ka_linear_skinny_pair_in_parts": [_c_int, _c_int],
    "ka_linear_library_bf16": [_c_void_p, _c_long, _c_void_p, _c_long, _c_void_p, _c_void_p, _c_int, _c_long, _c_int,
                               _c_int, _c_int, _c_int, _c_int, _c_void_p, _c_long, _c_void_p],
    "ka_linear_tiled_bf16": [_c_void_p, _c_long, _c_void_p, _c_long, _c_void_p, _c_void_p, _c_int, _c_long, _c_int,
                             _c_int, _c_int, _c_int, _c_int, _c_int, _c_void_p, _c_long, _c_void_p],
    "ka_attention_prefill_bf16": [_c_void_p, _c_long, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_void_p,
                                  _c_int, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_long, _c_float,
                                  _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void_p],
    "ka_rope_cache_pages_bf16": [_c_void_p, _c_long, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_void_p,
                                 _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void_p, _c_void_p, _c_int, _c_void_p],
    "ka_attention_decode_bf16": [_c_void_p, _c_long, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_void_p,
                                 _c_void_p, _c_void_p, _c_long, _c_float, _c_int, _c_int, _c_int, _c_int, _c_int,
                                 _c_int, _c_int, _c_void_p, _c_long,
                                 _c_void_p, _c_void_p, _c_long, _c_void_p, _c_int, _c_void_p, _c_void_p, _c_void_p,
                                 _c_void_p],
    "ka_attention_decode_beside_bf16": [
        _c_void_p, _c_long, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_long,
        _c_float, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void_p, _c_long,                # ..., splits, partial sums
        _c_void_p, _c_void_p, _c_long, _c_void_p, _c_int, _c_void_p, _c_void_p, _c_void_p,          # the tokens' own keys and values
        _c_void_p, _c_long, _c_int,                                                                  # A, lda, K
        _c_void_p, _c_long, _c_void_p, _c_void_p, _c_int, _c_long, _c_int, _c_int, _c_void_p],      # W, ldw, bias, out, ..., stream
    "ka_linear_skinny_norm_store": [_c_void_p, _c_void_p, _c_void_p, _c_float, _c_int, _c_void_p, _c_long, _c_void_p, _c_void_p,
                                    _c_int, _c_long, _c_int, _c_int, _c_int, _c_void_p, _c_long, _c_void_p],
}

# Rows up to which the weight-streaming kernel is used instead of the tiled one.
SKINNY_MAX_ROWS = 64
# Rows (and their width) up to which the weight-streaming kernel can normalise its input itself.
SKINNY_LN_MAX_ROWS = 16
SKINNY_LN_MAX_WIDTH = 4096
# Width of rows up to which a norm can follow a pair of skinny linears in their own launches.
NORM_AFTER_MAX_WIDTH = 8192
# Whether blocks let the weight-streaming kernel normalise its input itself. Every workgroup of
# the persistent kernel then repeats the LayerNorm of all rows once; with a few hundred workgroups
# that is cheaper than a launch of its own (measured on MI355X: 3 % of a decode step at batch 8).
FUSE_LAYERNORM_PROLOGUE = True
# Whether the decode attention of a few rows (whose workgroups fill at most a quarter of the chip)
# takes the feed-forward's first linear into its own launch instead of leaving it to the launch of
# the q|k|v projection before it (measured on MI355X at Moondream 2's sizes: 3 to 5 % of a decode
# step at batch 1 to 4).
ATTENTION_TAKES_LINEAR = True
# Tile of the tiled kernels: 0 lets them choose by size; 221, 211 (any K), 12222, 23212, 22224, 22232, 13122
# (K in steps of 64 or 32, loads straight into LDS) force one, and 1000000 * parts + 23212 forces K to be cut into
# that many parts as well (for measurements and tests).
TILED_CONFIG = 0
# Whether linears of more than SKINNY_MAX_ROWS rows go to the vendor library (hipBLASLt) where it has
# a kernel for the case, bias, activation and the sum into the residual being its epilogues; the
# tiled kernels of this package then take what it declines. Measured on MI355X at Moondream 2's
# four linears: 201 against 242 us a layer at 2,048 rows, 112 against 151 at 730, 64 against 72 at 96.
LIBRARY_LINEAR = True
LIBRARY_WORKSPACE_BYTES = 128 << 20
_library_space = {}
SCRATCH_FLOATS = 8 << 20
WIDE_FLOATS = 8 << 20              # 32 MB of partial sums for the wide skinny kernel
_wide_scratch = {}
# Keys of one row a workgroup of the decode attention kernel takes before the row is split.
DECODE_KEYS_PER_WORKGROUP = 4096
# Longest row for which workgroups of four waves run with tiles of 32 keys, eight to a CU (the kernel goes by the
# width of the block table: 128 pages).
DECODE_SMALL_TILE_KEYS = 2048


class ChipSizes(NamedTuple):
    """What the choices between kernel forms need to know of the GPU at hand, all of it following
    from its number of compute units (four SIMDs each)."""

    compute_units: int
    # waves the split weight-streaming kernel aims to have on the chip: 8 per compute unit (one workgroup
    # of 8 waves per strip where there are as many strips as compute units; measured best on an MI355X
    # for an output projection + second feed-forward linear of 2048 outputs)
    skinny_target_waves: int
    # waves of the decode attention kernel that the chip holds at once (16 per compute unit: four per
    # SIMD at the registers the kernel needs), its workgroups of four waves (five per compute unit), and
    # its workgroups of four waves with tiles of two pages, which the kernel takes where all of them then
    # fit on the chip at once (eight per compute unit)
    decode_wave_slots: int
    decode_four_wave_places: int
    decode_small_tile_places: int


_chips: Dict[int, ChipSizes] = {}


def chip_sizes(device=None) -> ChipSizes:
    """The sizes for ``device`` (default: the current one), asked from the driver once per device."""
    index = torch.cuda.current_device() if device is None else _device_index(device)
    if index not in _chips:
        units = int(torch.cuda.get_device_properties(index).multi_processor_count)
        _chips[index] = ChipSizes(units, 8 * units, 16 * units, 5 * units, 8 * units)
    return _chips[index]


ACT_GATED = 0x100                  # (ops.linear.ACT_GATED)

_lib = None
_scratch: Dict[int, torch.Tensor] = {}
_OUT_CODE = {torch.float32: KA_F32, torch.bfloat16: KA_BF16}


def lib():
    global _lib
    if _lib is None:
        handle = _build.load("fast")
        for name, argtypes in _SIGNATURES.items():
            fn = getattr(handle, name)
            fn.argtypes = argtypes
            fn.restype = _c_int
        handle.ka_last_error.restype = ctypes.c_char_p
        handle.ka_linear_library_stats.argtypes = [ctypes.POINTER(ctypes.c_long)] * 5
        handle.ka_linear_library_set_tuning.argtypes = [_c_int]
        handle.ka_linear_library_set_tuning.restype = None
        handle.ka_linear_library_stats.restype = None
        handle.ka_skinny_set_persistent.argtypes = [_c_int]
        handle.ka_skinny_set_persistent.restype = None
        handle.ka_rope_cache_pages_supported.argtypes = [_c_int, _c_int, _c_int]
        handle.ka_rope_cache_pages_supported.restype = _c_int
        for name in ("ka_attention_prefill_supported", "ka_attention_decode_supported"):
            getattr(handle, name).argtypes = [_c_int, _c_int]
            getattr(handle, name).restype = _c_int
        handle.ka_attention_decode_beside_supported.argtypes = [_c_int] * 6
        handle.ka_attention_decode_beside_supported.restype = _c_int
        for name in ("ka_attention_prefill_max_keys", "ka_attention_prefill_query_block"):
            getattr(handle, name).argtypes = [_c_int]
            getattr(handle, name).restype = _c_int
        _lib = handle
    return _lib


def set_skinny_persistent(enabled: int) -> None:
    """Whether one-segment skinny linears may use the persistent kernel where it fits (1, the
    default) or all go to the split kernel (0): for measurements, and for tests of the split kernel
    on sizes that it otherwise never sees."""
    lib().ka_skinny_set_persistent(int(enabled))


def set_skinny_wide(enabled: int) -> None:
    """Where skinny linears use the kernel that shares the activations through LDS and cuts K
    into parts: 1 (the default) where it was measured faster (two K-segments at 17 to 64 rows or
    with more strips than CUs at 5 to 16 rows; one segment too long for the persistent kernel's
    registers at 17 to 64 rows), 2 wherever it can run (for tests), 0 nowhere."""
    lib().ka_skinny_set_wide(int(enabled))


def _check(status: int) -> None:
    if status != 0:
        raise KernelError(lib().ka_last_error().decode())


def _device_index(device) -> int:
    """One key per GPU, whether or not the device's name carries its index."""
    device = torch.device(device)
    return torch.cuda.current_device() if device.index is None else device.index


def scratch(device: torch.device) -> torch.Tensor:
    """Partial results that the parts of a row's keys meet through in decode attention (one
    buffer per device). Calls on one device must not overlap."""
    key = _device_index(device)
    if key not in _scratch:
        _scratch[key] = torch.zeros(SCRATCH_FLOATS, dtype=torch.float32, device=device)
    return _scratch[key]


def _wide_args(device: torch.device, rows: int):
    """Scratch memory for the parts of K of a skinny linear that goes to the wide kernel: fp32
    partial sums, one buffer per device, made at the first skinny call (a step's first run is
    never inside a graph capture). Calls on one device must not overlap."""
    buf = _wide_scratch_buffer(device)
    return buf.data_ptr(), buf.numel()


def _wide_scratch_buffer(device: torch.device) -> torch.Tensor:
    key = _device_index(device)
    if key not in _wide_scratch:
        _wide_scratch[key] = torch.empty(WIDE_FLOATS, dtype=torch.float32, device=device)
    return _wide_scratch[key]


def _library_workspace(device: torch.device) -> torch.Tensor:
    """Scratch memory the vendor library's kernels may use (parts of K that meet in it), one buffer
    per device, made at the first call (a step's first run is never inside a graph capture).
    Calls on one device must not overlap."""
    key = _device_index(device)
    if key not in _library_space:
        _library_space[key] = torch.empty(LIBRARY_WORKSPACE_BYTES, dtype=torch.uint8, device=device)
    return _library_space[key]


def prepare(device: torch.device) -> int:
    """Everything these kernels keep per device, made now instead of at the first call that needs it
    (which may be the first step of a live request): the partial results of decode attention, the
    partial sums of the wide skinny kernel and the vendor library's workspace. Returns their bytes."""
    buffers = (scratch(device), _library_workspace(device), _wide_scratch_buffer(device))
    return sum(b.numel() * b.element_size() for b in buffers)


def library_stats() -> Dict[str, int]:
    """Plans the vendor-library linears keep, how often the library's heuristic was asked for an
    algorithm, how many plans had to make room, how many were tuned and how many of those took another
    algorithm than the first named (all since the process started)."""
    handle = lib()
    values = [ctypes.c_long(0) for _ in range(5)]
    handle.ka_linear_library_stats(*[ctypes.byref(v) for v in values])
    return dict(zip(("plans", "heuristic_calls", "evicted", "tuned", "tuned_other"), (int(v.value) for v in values)))


def set_library_tuning(runs: int) -> None:
    """``runs`` > 0: a plan of the vendor-library linears that is made from now on times, at its first call, every
    algorithm the library's heuristic named (``runs`` products each, on that call's operands, whose content is
    run over several times: a warm-up's) and keeps the fastest. 0 (the default): the first named."""
    lib().ka_linear_library_set_tuning(int(runs))


def _operand_ok(t: torch.Tensor, k: int) -> bool:
    return (t.dtype == torch.bfloat16 and t.dim() == 2 and t.shape[1] == k and t.stride(1) == 1 and t.stride(0) % 8 == 0
            and t.data_ptr() % 16 == 0)


def _bias_ok(bias: Optional[torch.Tensor], n: int) -> bool:
    return bias is None or (bias.dtype == torch.float32 and bias.numel() == n and bias.is_contiguous())


def _out_ok(out: torch.Tensor, m: int, n: int, act: int = 0) -> bool:
    """``out`` is ``[m, columns]`` of a linear of ``n`` weight rows (half of them if ``act`` says gated)."""
    n_out = n // 2 if act & ACT_GATED else n
    return (out.dtype in _OUT_CODE and tuple(out.shape) == (m, n_out) and out.stride(1) == 1 and out.data_ptr() % 16 == 0)


def linear_bf16(a, weight, bias, out, act, accumulate) -> bool:
    m, k = a.shape
    n = weight.shape[0]
    if m == 0:
        return True
    if k % 8 or not _operand_ok(a, k) or not _operand_ok(weight, k) or out.dtype not in _OUT_CODE \
            or out.data_ptr() % 16 or out.stride(1) != 1:
        return False
    if act & ACT_GATED and (n % 2 or accumulate):
        raise KernelError("linear: a gated linear needs an even number of weight rows and no accumulation")
    if tuple(out.shape) != (m, n // 2 if act & ACT_GATED else n):
        raise KernelError(f"linear: shapes a {tuple(a.shape)}, weight {tuple(weight.shape)}, out {tuple(out.shape)}")
    if not _bias_ok(bias, n):
        raise KernelError("linear: bias must be fp32 [N]")
    if accumulate and out.dtype != torch.float32:
        raise KernelError("linear: accumulate needs an fp32 output")
    handle = lib()
    if m <= SKINNY_MAX_ROWS:
        _check(handle.ka_linear_skinny_bf16(a.data_ptr(), a.stride(0), weight.data_ptr(), weight.stride(0), _ptr(bias),
                                            out.data_ptr(), _OUT_CODE[out.dtype], out.stride(0), m, n, k, act,
                                            int(accumulate), chip_sizes(a.device).skinny_target_waves, *_wide_args(a.device, m), stream_ptr()))
    else:
        if LIBRARY_LINEAR and TILED_CONFIG == 0:
            space = _library_workspace(a.device)
            status = handle.ka_linear_library_bf16(a.data_ptr(), a.stride(0), weight.data_ptr(), weight.stride(0),
                                                   _ptr(bias), out.data_ptr(), _OUT_CODE[out.dtype], out.stride(0), m, n, k,
                                                   act, int(accumulate), space.data_ptr(), space.numel(), stream_ptr())
            if status == 0:
                return True
            if status < 0:
                _check(status)
        _check(handle.ka_linear_tiled_bf16(a.data_ptr(), a.stride(0), weight.data_ptr(), weight.stride(0), _ptr(bias),
                                           out.data_ptr(), _OUT_CODE[out.dtype], out.stride(0), m, n, k, act,
                                           int(accumulate), TILED_CONFIG, *_wide_args(a.device, m), stream_ptr()))
    return True


def linear_pair_accumulate(a1, w1, b1, a2, w2, b2, out, then_norm=None) -> bool:
    """``out += a1 @ w1.T + b1 + a2 @ w2.T + b2`` in one launch (few rows, fp32 ``out``).
    ``then_norm = (gamma, beta or None, eps, normed)``: also ``normed = LayerNorm(out)``, in the kernel
    that finishes the rows where there is one (more than 8 rows), else in a launch behind it. False:
    not covered, nothing was run (with ``then_norm``: try without)."""
    m, k1 = a1.shape
    k2 = a2.shape[1]
    n = w1.shape[0]
    if not (0 < m <= SKINNY_MAX_ROWS) or k1 % 8 or k2 % 8 or a2.shape[0] != m or w2.shape[0] != n:
        return False
    if not (_operand_ok(a1, k1) and _operand_ok(w1, k1) and _operand_ok(a2, k2) and _operand_ok(w2, k2)):
        return False
    if out.dtype != torch.float32 or not _out_ok(out, m, n) or not _bias_ok(b1, n) or not _bias_ok(b2, n):
        return False
    if then_norm is not None:
        gamma, beta, eps, normed = then_norm
        if n % 4 or n > NORM_AFTER_MAX_WIDTH or out.stride(0) % 4 or normed.dtype not in _OUT_CODE or not _out_ok(normed, m, n) \
                or normed.stride(0) % 4 or gamma.dtype != torch.float32 or gamma.numel() != n or gamma.data_ptr() % 16:
            return False
        if beta is not None and (beta.dtype != torch.float32 or beta.numel() != n or beta.data_ptr() % 16):
            return False
        if any(b is not None and b.data_ptr() % 16 for b in (b1, b2)):
            return False
        _check(lib().ka_linear_skinny_pair_norm(
            a1.data_ptr(), a1.stride(0), k1, a2.data_ptr(), a2.stride(0), k2, w1.data_ptr(), w1.stride(0), _ptr(b1),
            w2.data_ptr(), w2.stride(0), _ptr(b2), out.data_ptr(), out.stride(0), n, 1, m, chip_sizes(a1.device).skinny_target_waves,
            *_wide_args(a1.device, m), gamma.data_ptr(), _ptr(beta), float(eps), normed.data_ptr(), _OUT_CODE[normed.dtype],
            normed.stride(0), stream_ptr()))
        return True
    _check(lib().ka_linear_skinny_fused(
        a1.data_ptr(), a1.stride(0), k1, a2.data_ptr(), a2.stride(0), k2, w2.data_ptr(), w2.stride(0), _ptr(b2),
        None, None, None, 0.0,
        w1.data_ptr(), w1.stride(0), _ptr(b1), out.data_ptr(), KA_F32, out.stride(0), n, 0, 1,
        None, 0, None, None, 0, 0, 0, 0, m, chip_sizes(a1.device).skinny_target_waves, *_wide_args(a1.device, m), stream_ptr()))
    return True


def pair_finishes_rows(m: int, n: int) -> bool:
    """Whether ``linear_pair_accumulate`` of ``m`` rows and ``n`` outputs ends in a kernel that finishes
    whole rows (K cut into parts): that kernel normalises them as well at no launch of its own."""
    return bool(lib().ka_linear_skinny_pair_in_parts(int(m), int(n)))


def linear_two_outputs(a, wa, ba, out_a, act_a, wb, bb, out_b, act_b) -> bool:
    """``out_a = act_a(a @ wa.T + ba)`` and ``out_b = act_b(a @ wb.T + bb)`` in one launch (few rows)."""
    m, k = a.shape
    na, nb = wa.shape[0], wb.shape[0]
    if not (0 < m <= SKINNY_MAX_ROWS) or k % 8:
        return False
    if not (_operand_ok(a, k) and _operand_ok(wa, k) and _operand_ok(wb, k) and _out_ok(out_a, m, na, act_a)
            and _out_ok(out_b, m, nb, act_b) and _bias_ok(ba, na) and _bias_ok(bb, nb)):
        return False
    _check(lib().ka_linear_skinny_fused(
        a.data_ptr(), a.stride(0), k, None, 0, 0, None, 0, None,
        None, None, None, 0.0,
        wa.data_ptr(), wa.stride(0), _ptr(ba), out_a.data_ptr(), _OUT_CODE[out_a.dtype], out_a.stride(0), na, act_a, 0,
        wb.data_ptr(), wb.stride(0), _ptr(bb), out_b.data_ptr(), _OUT_CODE[out_b.dtype], out_b.stride(0), nb, act_b,
        m, chip_sizes(a.device).skinny_target_waves, *_wide_args(a.device, m), stream_ptr()))
    return True


def layernorm_linear(x, gamma, beta, eps, wa, ba, out_a, act_a, wb=None, bb=None, out_b=None, act_b=0, store=None) -> bool:
    """``h = LayerNorm(x)``; ``out_a = act_a(h @ wa.T + ba)`` and, if a second target is given,
    ``out_b = act_b(h @ wb.T + bb)`` in one launch: the kernel normalises the fp32 rows itself
    (at most 16 of them, at most 4096 wide, and no more than fit in 96 KB of LDS as bf16).
    ``store`` (one target only): bf16 ``[m, k]`` that also receives ``h``, for launches that follow."""
    m, k = x.shape
    if not (0 < m <= SKINNY_LN_MAX_ROWS) or k % 8 or k > SKINNY_LN_MAX_WIDTH or x.dtype != torch.float32 \
            or not x.is_contiguous():
        return False
    if x.data_ptr() % 16 or gamma.dtype != torch.float32 or gamma.numel() != k or gamma.data_ptr() % 16:
        return False
    if beta is not None and (beta.dtype != torch.float32 or beta.numel() != k or beta.data_ptr() % 16):
        return False
    na = wa.shape[0]
    if not (_operand_ok(wa, k) and _out_ok(out_a, m, na, act_a) and _bias_ok(ba, na)):
        return False
    two = wb is not None
    nb = wb.shape[0] if two else 0
    if two and not (_operand_ok(wb, k) and _out_ok(out_b, m, nb, act_b) and _bias_ok(bb, nb)):
        return False
    if m * (k + 8) * 2 > 96 * 1024:
        return False
    for bias, n in ((ba, na), (bb, nb)):
        if bias is not None and (n % 4 or bias.data_ptr() % 16):
            return False
    if store is not None:
        if two or store.dtype != torch.bfloat16 or not _out_ok(store, m, k) or store.stride(0) % 8:
            return False
        _check(lib().ka_linear_skinny_norm_store(
            x.data_ptr(), gamma.data_ptr(), _ptr(beta), float(eps), k, wa.data_ptr(), wa.stride(0), _ptr(ba),
            out_a.data_ptr(), _OUT_CODE[out_a.dtype], out_a.stride(0), na, act_a, m, store.data_ptr(), store.stride(0),
            stream_ptr()))
        return True
    _check(lib().ka_linear_skinny_fused(
        None, 0, k, None, 0, 0, None, 0, None,
        x.data_ptr(), gamma.data_ptr(), _ptr(beta), float(eps),
        wa.data_ptr(), wa.stride(0), _ptr(ba), out_a.data_ptr(), _OUT_CODE[out_a.dtype], out_a.stride(0), na, act_a, 0,
        _ptr(wb), wb.stride(0) if two else 0, _ptr(bb) if two else None, _ptr(out_b),
        _OUT_CODE[out_b.dtype] if two else 0, out_b.stride(0) if two else 0, nb, act_b,
        m, chip_sizes(x.device).skinny_target_waves, None, 0, stream_ptr()))
    return True


def rope_cache_bf16(qkv, positions, slots, table, k_cache, v_cache, n_heads, n_kv_heads, head_dim, page_size,
                    runs=None) -> bool:
    """Rotary encoding of q (in place) and k, and the cache write of k and v, a page's worth of
    tokens per workgroup (``ops.core.rope_cache`` says what the operands are). ``runs``: (int32 first
    token, int32 count) of the runs the tokens are cut into, every token in exactly one and none longer
    than a page (``StepBatch.page_runs``); without them every 16 tokens are a run. False: not covered
    (another page size, a rotary size that is no multiple of 16, rows that are not 16-byte aligned)."""
    if table is None or qkv.dtype != torch.bfloat16 or qkv.stride(1) != 1 or qkv.stride(0) % 8 or qkv.data_ptr() % 16:
        return False
    rot = int(table.shape[1])
    handle = lib()
    if not handle.ka_rope_cache_pages_supported(head_dim, rot, page_size) or table.data_ptr() % 16:
        return False
    if slots is not None and (k_cache.data_ptr() % 16 or v_cache.data_ptr() % 16):
        return False
    first, count = runs if runs is not None else (None, None)
    _check(handle.ka_rope_cache_pages_bf16(qkv.data_ptr(), qkv.stride(0), positions.data_ptr(), _ptr(slots), table.data_ptr(),
                                           int(table.shape[0]), _ptr(k_cache), _ptr(v_cache), qkv.shape[0], n_heads,
                                           n_kv_heads, head_dim, rot, page_size, _ptr(first), _ptr(count),
                                           int(first.numel()) if first is not None else 0, stream_ptr()))
    return True


def decode_shape(max_kv: int, workgroups: int = 1, head_dim: int = 64):
    """``(splits, waves)`` of the decode attention kernel: a workgroup of up to 16 waves takes a
    64-key tile per wave and round; rows longer than 4096 keys are cut into parts whose sums
    a second kernel merges (cutting the keys of a few short rows further, to put more CUs to
    work, was measured and changes nothing: 0.887 ms a step at batch 1 either way). With many
    workgroups (rows x heads) each gets fewer waves, so that they all fit on the chip at once.
    Head sizes up to 64 (measured at 32 heads and 1,024 keys): 16 waves up to 256 workgroups, 4
    beyond, which the kernel runs with tiles of 32 keys, eight workgroups to a CU, while the chip
    holds them all at once (four waves against eight: 6.70k against 6.53k tok/s at 9 rows, 10.6k
    against 10.4k at 16, 12.8k against 11.9k at 24, 16.5k against 15.9k at 48, 18.0k against 16.5k at
    64; rows of up to 2,048 keys: behind 4,096 keys the larger tile is 2 to 3 % ahead at 24 and 32
    rows). Larger head sizes, whose registers leave a CU eight waves, and longer rows: 16 waves up to
    256 workgroups, 8 up to 512, 4 beyond. Workgroups of four waves with tiles of 64 keys fit five to a CU; where they
    would end in a round that leaves much of the chip idle, eight waves again."""
    chip = chip_sizes()
    splits = max(1, -(-max_kv // DECODE_KEYS_PER_WORKGROUP))
    tiles = -(-max_kv // (64 * splits))
    waves = 4 if tiles <= 4 else 8 if tiles <= 8 else 16
    groups = workgroups * splits
    if groups <= chip.decode_wave_slots // 16:
        fit = 16
    elif head_dim <= 64 and groups <= chip.decode_small_tile_places and max_kv <= DECODE_SMALL_TILE_KEYS:
        fit = 4
    elif groups <= chip.decode_wave_slots // 8:
        fit = 8
    else:
        # workgroups of four waves run in rounds of as many as the chip has places for; where the last round
        # would leave much of the chip idle, workgroups of eight waves come out better (48 rows x 32 heads are
        # 1.2 rounds of the one, 3 rounds of the other: 14.9k against 15.2k tok/s)
        fit = 4
        rounds = -(-groups // chip.decode_four_wave_places)
        if groups < 0.7 * rounds * chip.decode_four_wave_places:
            fit = 8
    return splits, min(waves, fit)


def _attention_operands_ok(q, out) -> bool:
    return not (q.data_ptr() % 16 or q.stride(0) % 8 or out.data_ptr() % 16 or out.stride(0) % 4)


def _side_linear_ok(job) -> bool:
    """Operands of a ``parts.SideLinear`` that the persistent skinny kernel takes."""
    a, w, out = job.a, job.weight, job.out
    if a.dim() != 2 or a.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        return False
    m, k = a.shape
    n = w.shape[0]
    if k % 8 or not (_operand_ok(a, k) and _operand_ok(w, k) and _out_ok(out, m, n, int(job.act)) and _bias_ok(job.bias, n)):
        return False
    return job.bias is None or (n % 4 == 0 and job.bias.data_ptr() % 16 == 0)


def attention_decode_takes(job, n: int, n_heads: int, head_dim: int, page_size: int, max_kv: int) -> bool:
    """Whether ``attention_decode_bf16`` runs ``job`` (a ``parts.SideLinear``) in its own launch: a few
    rows whose attention leaves most of the chip idle."""
    if not ATTENTION_TAKES_LINEAR or n == 0 or not _side_linear_ok(job) or job.a.shape[0] != n:
        return False
    splits = decode_shape(max_kv, n * n_heads, head_dim)[0]
    return bool(lib().ka_attention_decode_beside_supported(n, n_heads, splits, head_dim, page_size, job.a.shape[1]))


def attention_decode_bf16(q, k_cache, v_cache, block_table, token_row, kv_lo, kv_hi, out, scale, n_heads,
                          n_kv_heads, head_dim, batch, fuse=None, beside=None) -> bool:
    """One token per row. ``fuse = (k_new, v_new, table, slots)``: the kernel also rotates q and the
    token's key and stores key and value in the cache (the rotary kernel is then not run).
    ``beside``: a ``parts.SideLinear`` for which ``attention_decode_takes`` said yes; the launch
    computes it on the side (False: it does not after all, and nothing was run)."""
    n = q.shape[0]
    page_size = k_cache.shape[2]
    if n == 0:
        return beside is None
    handle = lib()
    if batch is None or not batch.decode_only or not _attention_operands_ok(q, out) \
            or not handle.ka_attention_decode_supported(head_dim, page_size):
        return False
    if beside is not None and not attention_decode_takes(beside, n, n_heads, head_dim, page_size, batch.max_kv):
        return False
    splits, waves = decode_shape(batch.max_kv, n * n_heads, head_dim)
    partial = scratch(q.device)
    if n * n_heads * splits * (head_dim + 2) > partial.numel():
        return False
    k_new = v_new = table = slots = None
    new_stride = rot = 0
    if fuse is not None:
        k_new, v_new, table, slots = fuse
        rot = int(table.shape[1])
        new_stride = k_new.stride(0)
        if rot % 16 or rot > head_dim or k_new.data_ptr() % 16 or v_new.data_ptr() % 16 \
                or new_stride % 8 or v_new.stride(0) != new_stride:
            return False
    if beside is not None:
        w, lin_out = beside.weight, beside.out
        _check(handle.ka_attention_decode_beside_bf16(
            q.data_ptr(), q.stride(0), k_cache.data_ptr(), v_cache.data_ptr(), block_table.data_ptr(),
            block_table.shape[1], token_row.data_ptr(), _ptr(kv_lo), kv_hi.data_ptr(), out.data_ptr(), out.stride(0),
            float(scale), n, n_heads, n_kv_heads, head_dim, page_size, splits, partial.data_ptr(), partial.numel(),
            _ptr(k_new), _ptr(v_new), new_stride, _ptr(table), rot, _ptr(slots), k_cache.data_ptr(), v_cache.data_ptr(),
            beside.a.data_ptr(), beside.a.stride(0), beside.a.shape[1], w.data_ptr(), w.stride(0), _ptr(beside.bias),
            lin_out.data_ptr(), _OUT_CODE[lin_out.dtype], lin_out.stride(0), w.shape[0], int(beside.act), stream_ptr()))
        return True
    _check(handle.ka_attention_decode_bf16(
        q.data_ptr(), q.stride(0), k_cache.data_ptr(), v_cache.data_ptr(), block_table.data_ptr(),
        block_table.shape[1], token_row.data_ptr(), _ptr(kv_lo), kv_hi.data_ptr(), out.data_ptr(), out.stride(0),
        float(scale), n, n_heads, n_kv_heads, head_dim, page_size, splits, waves, partial.data_ptr(), partial.numel(),
        _ptr(k_new), _ptr(v_new), new_stride, _ptr(table), rot, _ptr(slots),
        k_cache.data_ptr(), v_cache.data_ptr(), stream_ptr()))
    return True


def prefill_query_block(head_dim: int) -> int:
    """Queries of one row that a workgroup of the prompt attention kernel takes at this head size:
    the size the step's lists of blocks of queries must be cut to for it."""
    return int(lib().ka_attention_prefill_query_block(head_dim))


def _query_blocks(batch, head_dim: int):
    """``(rows, first tokens, size)`` of the blocks of queries of a step, at the size the kernel likes
    best among those the step lists (``batch.query_blocks``: size -> lists), else at 32."""
    listed = getattr(batch, "query_blocks", None) or {}
    best = prefill_query_block(head_dim)
    if best in listed:
        return (*listed[best], best)
    if 32 in listed:
        return (*listed[32], 32)
    if getattr(batch, "qblk_row", None) is not None:
        return batch.qblk_row, batch.qblk_tok, 32
    return None


def attention_bf16(q, k_cache, v_cache, block_table, token_row, kv_lo, kv_hi, out, scale, n_heads, n_kv_heads,
                   head_dim, batch) -> bool:
    n = q.shape[0]
    page_size = k_cache.shape[2]
    if n == 0:
        return True
    if batch is None or not _attention_operands_ok(q, out):
        return False
    if attention_decode_bf16(q, k_cache, v_cache, block_table, token_row, kv_lo, kv_hi, out, scale, n_heads,
                             n_kv_heads, head_dim, batch):
        return True
    handle = lib()
    # the longest row's block table must fit in LDS (the whole table's width where the length is not known)
    longest = int(batch.max_kv) if batch.max_kv > 1 else block_table.shape[1] * page_size
    blocks = _query_blocks(batch, head_dim) if handle.ka_attention_prefill_supported(head_dim, page_size) else None
    # (the prompt kernel is written for a positive scale; any other goes to the generic kernel)
    if blocks is not None and longest <= handle.ka_attention_prefill_max_keys(head_dim) and 0.0 < scale < float("inf"):
        rows, first_tokens, size = blocks
        _check(handle.ka_attention_prefill_bf16(
            q.data_ptr(), q.stride(0), k_cache.data_ptr(), v_cache.data_ptr(), block_table.data_ptr(),
            block_table.shape[1], rows.data_ptr(), first_tokens.data_ptr(), int(rows.numel()),
            batch.cu_q.data_ptr(), batch.kv_len.data_ptr(), _ptr(kv_lo), kv_hi.data_ptr(), out.data_ptr(),
            out.stride(0), float(scale), n_heads, n_kv_heads, head_dim, page_size,
            int(batch.max_kv) if batch.max_kv > 1 else 0, size, stream_ptr()))
        return True
    return False
