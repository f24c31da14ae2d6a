"""Python faces of the bf16 MFMA kernels (library ``fast``).

Each function returns ``False`` when the kernels do not cover the operands (the
caller then takes the generic kernel) and raises when they do but the call fails.
"""

from __future__ import annotations

import ctypes
from typing import Dict, Optional

import torch

from ..csrc import build as _build
from .core import KA_BF16, KA_F32, KernelError, _ptr, stream_ptr

_c_void_p, _c_int, _c_long, _c_float = ctypes.c_void_p, ctypes.c_int, ctypes.c_long, ctypes.c_float

_SIGNATURES = {
    "ka_linear_skinny_bf16": [_c_void_p, _c_long, _c_void_p, _c_long, _c_void_p, _c_void_p, _c_int, _c_long, _c_int,
                              _c_int, _c_int, _c_int, _c_int, _c_int, _c_void_p],
    "ka_linear_tiled_bf16": [_c_void_p, _c_long, _c_void_p, _c_long, _c_void_p, _c_void_p, _c_int, _c_long, _c_int,
                             _c_int, _c_int, _c_int, _c_int, _c_void_p],
    "ka_attention_prefill_bf16": [_c_void_p, _c_long, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_void_p,
                                  _c_int, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_long, _c_float,
                                  _c_int, _c_int, _c_int, _c_int, _c_void_p],
    "ka_attention_decode_bf16": [_c_void_p, _c_long, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_void_p,
                                 _c_void_p, _c_void_p, _c_long, _c_float, _c_int, _c_int, _c_int, _c_int, _c_int,
                                 _c_int, _c_int, _c_void_p, _c_long, _c_void_p, _c_int, _c_void_p],
}

# Rows up to which the weight-streaming kernel is used instead of the tiled one.
SKINNY_MAX_ROWS = 64
# Waves the weight-streaming kernel aims to have on the chip (256 CUs, 16 to 32 waves each).
SKINNY_TARGET_WAVES = 6144
SCRATCH_FLOATS = 8 << 20
SCRATCH_COUNTERS = 1 << 16

_lib = None
_scratch: Dict[torch.device, tuple] = {}


def lib():
    global _lib
    if _lib is None:
        handle = _build.load("fast")
        for name, argtypes in _SIGNATURES.items():
            fn = getattr(handle, name)
            fn.argtypes = argtypes
            fn.restype = _c_int
        handle.ka_last_error.restype = ctypes.c_char_p
        for name in ("ka_attention_prefill_supported", "ka_attention_decode_supported"):
            getattr(handle, name).argtypes = [_c_int, _c_int]
            getattr(handle, name).restype = _c_int
        _lib = handle
    return _lib


def _check(status: int) -> None:
    if status != 0:
        raise KernelError(lib().ka_last_error().decode())


def scratch(device: torch.device):
    """Partial sums and arrival counters the split kernels add up through (one pair per device;
    the kernels leave the counters at zero). Calls on one device must not overlap."""
    key = torch.device(device)
    if key not in _scratch:
        _scratch[key] = (torch.zeros(SCRATCH_FLOATS, dtype=torch.float32, device=device),
                         torch.zeros(SCRATCH_COUNTERS, dtype=torch.int32, device=device))
    return _scratch[key]


_OUT_CODE = {torch.float32: KA_F32, torch.bfloat16: KA_BF16}


def linear_bf16(a, weight, bias, out, act, accumulate) -> bool:
    m, k = a.shape
    n = weight.shape[0]
    if m == 0:
        return True
    if (k % 8 or a.stride(0) % 8 or weight.stride(0) % 8 or a.data_ptr() % 16 or weight.data_ptr() % 16
            or out.dtype not in _OUT_CODE or out.data_ptr() % 16 or a.stride(1) != 1 or weight.stride(1) != 1
            or out.stride(1) != 1):
        return False
    if tuple(weight.shape) != (n, k) or tuple(out.shape) != (m, n):
        raise KernelError(f"linear: shapes a {tuple(a.shape)}, weight {tuple(weight.shape)}, out {tuple(out.shape)}")
    if bias is not None and (bias.dtype != torch.float32 or bias.numel() != n or not bias.is_contiguous()):
        raise KernelError("linear: bias must be fp32 [N]")
    if accumulate and out.dtype != torch.float32:
        raise KernelError("linear: accumulate needs an fp32 output")
    handle = lib()
    if m <= SKINNY_MAX_ROWS:
        _check(handle.ka_linear_skinny_bf16(a.data_ptr(), a.stride(0), weight.data_ptr(), weight.stride(0), _ptr(bias),
                                            out.data_ptr(), _OUT_CODE[out.dtype], out.stride(0), m, n, k, act,
                                            int(accumulate), SKINNY_TARGET_WAVES, stream_ptr()))
    else:
        _check(handle.ka_linear_tiled_bf16(a.data_ptr(), a.stride(0), weight.data_ptr(), weight.stride(0), _ptr(bias),
                                           out.data_ptr(), _OUT_CODE[out.dtype], out.stride(0), m, n, k, act,
                                           int(accumulate), stream_ptr()))
    return True


DECODE_KEYS_PER_WORKGROUP = 4096


def decode_shape(max_kv: int):
    """``(splits, waves)`` of the decode attention kernel: a workgroup of up to 16 waves takes a
    64-key tile per wave and round; rows longer than 4096 keys are cut into splits that meet
    through scratch memory."""
    splits = max(1, -(-max_kv // DECODE_KEYS_PER_WORKGROUP))
    tiles = -(-max_kv // (64 * splits))
    waves = 4 if tiles <= 4 else 8 if tiles <= 8 else 16
    return splits, waves


def attention_bf16(q, k_cache, v_cache, block_table, token_row, kv_lo, kv_hi, out, scale, n_heads, n_kv_heads,
                   head_dim, batch) -> bool:
    n = q.shape[0]
    page_size = k_cache.shape[2]
    if n == 0:
        return True
    if batch is None or q.data_ptr() % 16 or q.stride(0) % 8 or out.data_ptr() % 16 or out.stride(0) % 4:
        return False
    handle = lib()
    if batch.decode_only and handle.ka_attention_decode_supported(head_dim, page_size):
        splits, waves = decode_shape(batch.max_kv)
        partial, counters = scratch(q.device)
        if n * n_heads * splits * (head_dim + 2) <= partial.numel() and n * n_heads <= counters.numel():
            _check(handle.ka_attention_decode_bf16(
                q.data_ptr(), q.stride(0), k_cache.data_ptr(), v_cache.data_ptr(), block_table.data_ptr(),
                block_table.shape[1], token_row.data_ptr(), _ptr(kv_lo), kv_hi.data_ptr(), out.data_ptr(),
                out.stride(0), float(scale), n, n_heads, n_kv_heads, head_dim, page_size, splits, waves, partial.data_ptr(),
                partial.numel(), counters.data_ptr(), counters.numel(), stream_ptr()))
            return True
    if handle.ka_attention_prefill_supported(head_dim, page_size) and batch.qblk_row is not None:
        _check(handle.ka_attention_prefill_bf16(
            q.data_ptr(), q.stride(0), k_cache.data_ptr(), v_cache.data_ptr(), block_table.data_ptr(),
            block_table.shape[1], batch.qblk_row.data_ptr(), batch.qblk_tok.data_ptr(), int(batch.qblk_row.numel()),
            batch.cu_q.data_ptr(), batch.kv_len.data_ptr(), _ptr(kv_lo), kv_hi.data_ptr(), out.data_ptr(),
            out.stride(0), float(scale), n_heads, n_kv_heads, head_dim, page_size, stream_ptr()))
        return True
    return False
