"""Python faces of the generic HIP kernels (library ``core``).

Each function checks what the kernel assumes about its operands (device, type,
contiguity, sizes), then passes raw pointers and the current HIP stream to the C
entry point. Nothing here computes on the CPU and nothing falls back to a library.
"""

from __future__ import annotations

import ctypes
from typing import Optional

import torch

from ..csrc import build as _build

KA_F32, KA_BF16 = 0, 1
_DTYPE_CODE = {torch.float32: KA_F32, torch.bfloat16: KA_BF16}

_c_void_p, _c_int, _c_long, _c_float = ctypes.c_void_p, ctypes.c_int, ctypes.c_long, ctypes.c_float

_SIGNATURES = {
    "ka_embed": [_c_void_p, _c_int, _c_void_p, _c_void_p, _c_int, _c_int, _c_void_p, _c_int, _c_int, _c_float, _c_void_p],
    "ka_adjust_logits": [_c_void_p, _c_long, _c_float, _c_float, _c_void_p],
    "ka_scatter_rows": [_c_void_p, _c_int, _c_void_p, _c_void_p, _c_int, _c_int, _c_void_p],
    "ka_layernorm": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_float, _c_void_p, _c_int, _c_int, _c_int,
                     _c_void_p],
    "ka_rope_cache": [_c_void_p, _c_int, _c_long, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_void_p,
                      _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void_p],
    "ka_linear_generic": [_c_void_p, _c_int, _c_long, _c_void_p, _c_int, _c_long, _c_void_p, _c_void_p, _c_int,
                          _c_long, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void_p],
    "ka_attention_generic": [_c_void_p, _c_int, _c_long, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p,
                             _c_void_p, _c_void_p, _c_void_p, _c_long, _c_float, _c_int, _c_int, _c_int, _c_int,
                             _c_int, _c_void_p],
    "ka_argmax": [_c_void_p, _c_long, _c_void_p, _c_int, _c_int, _c_void_p, _c_void_p, _c_int, _c_void_p],
    "ka_suppress_tokens": [_c_void_p, _c_long, _c_void_p, _c_void_p, _c_int, _c_int, _c_void_p],
    "ka_allow_tokens": [_c_void_p, _c_long, _c_void_p, _c_void_p, _c_int, _c_int, _c_void_p],
    "ka_token_logprobs": [_c_void_p, _c_long, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_void_p],
    "ka_sample": [_c_void_p, _c_long, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int,
                  _c_void_p, _c_void_p, _c_int, _c_void_p],
}

_lib = None


class KernelError(RuntimeError):
    """A HIP entry point refused its arguments or failed to launch."""


def lib():
    global _lib
    if _lib is None:
        handle = _build.load("core")
        for name, argtypes in _SIGNATURES.items():
            fn = getattr(handle, name)
            fn.argtypes = argtypes
            fn.restype = _c_int
        handle.ka_last_error.restype = ctypes.c_char_p
        handle.ka_uniform_host.argtypes = [ctypes.c_ulonglong, ctypes.c_ulonglong]
        handle.ka_uniform_host.restype = _c_float
        handle.ka_sample_set_passes_only.argtypes = [_c_int]
        handle.ka_sample_set_passes_only.restype = None
        _lib = handle
    return _lib


def _check(status: int, handle=None) -> None:
    if status != 0:
        handle = handle or lib()
        raise KernelError(handle.ka_last_error().decode())


# torch's own short way to the current stream's handle (what its compiled kernels call before a launch);
# `torch.cuda.current_stream()` builds a Python object per call: 2.8 us against 0.07 us, some 170 times a step
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def stream_ptr() -> int:
    """The handle of the current stream of the current device."""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def code_of(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise KernelError(f"unsupported tensor type {dtype}: the kernels take float32 and bfloat16") from None


def _need(cond: bool, message: str) -> None:
    if not cond:
        raise KernelError(message)


def _dev(*tensors) -> None:
    for t in tensors:
        if t is not None:
            _need(t.is_cuda, "kernel operand is not on the GPU")


def _dev_or_pinned(t: torch.Tensor) -> None:
    """A small output may lie in pinned host memory, which the GPU writes directly: the host then
    needs no copy behind the kernel, only its end."""
    _need(t.is_cuda or t.is_pinned(), "kernel output is neither on the GPU nor in pinned host memory")


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _check_caches(who: str, k_cache, v_cache, dtype, n_kv_heads: int, page_size: int, head_dim: int) -> None:
    """Keys ``[pages, Hkv, page_size, hd]``, values ``[pages, Hkv, hd, page_size]``, both contiguous."""
    _need(k_cache.dtype == dtype and k_cache.is_contiguous() and k_cache.dim() == 4
          and tuple(k_cache.shape[1:]) == (n_kv_heads, page_size, head_dim),
          f"{who}: key cache must be [pages, Hkv, page_size, hd] of the activation type")
    _need(v_cache.dtype == dtype and v_cache.is_contiguous() and v_cache.dim() == 4
          and tuple(v_cache.shape[1:]) == (n_kv_heads, head_dim, page_size) and v_cache.shape[0] == k_cache.shape[0],
          f"{who}: value cache must be [pages, Hkv, hd, page_size] of the activation type")


def measured_peaks(device: torch.device, read_bytes: int = 2 << 30) -> dict:
    """What this GPU reaches on a plain read stream of ``read_bytes`` (GB/s) and on a loop of bf16
    matrix instructions that waits for nothing (TFLOP/s): the best of a few runs each."""
    handle = lib()
    for name, argtypes in (("ka_peak_read", [_c_void_p, _c_long, _c_int, _c_void_p, _c_void_p]),
                           ("ka_peak_mfma_bf16", [_c_void_p, _c_int, _c_int, _c_void_p])):
        getattr(handle, name).argtypes = argtypes
        getattr(handle, name).restype = _c_int
    sink = torch.zeros(16, dtype=torch.float32, device=device)
    buffer = torch.ones(read_bytes // 4, dtype=torch.int32, device=device)
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)

    def best_ms(launch, repeats=5):
        launch()
        torch.cuda.synchronize(device)
        best = None
        for _ in range(repeats):
            start.record()
            launch()
            stop.record()
            stop.synchronize()
            ms = start.elapsed_time(stop)
            best = ms if best is None else min(best, ms)
        return best

    read_ms = min(best_ms(lambda g=g: _check(handle.ka_peak_read(buffer.data_ptr(), read_bytes, g, sink.data_ptr(), stream_ptr())))
                  for g in (2048, 4096, 8192))
    workgroups, iters = 1024, 8000
    mfma_ms = best_ms(lambda: _check(handle.ka_peak_mfma_bf16(sink.data_ptr(), workgroups, iters, stream_ptr())))
    flops = workgroups * 4 * iters * 8 * 2 * 32 * 32 * 16
    del buffer
    return {"hbm_read_gbs": read_bytes / (read_ms * 1e-3) / 1e9, "mfma_bf16_tflops": flops / (mfma_ms * 1e-3) / 1e12}


def uniform(key: int, counter: int) -> float:
    """The uniform number the sampling kernel draws for (key, counter)."""
    return float(lib().ka_uniform_host(key & (2 ** 64 - 1), counter))


def embed(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor, pending: Optional[torch.Tensor] = None,
          scale: float = 1.0) -> None:
    """``out[t] = scale * table[ids[t]]`` in fp32. A row with id -1 is left untouched; an id ``<= -2`` is
    replaced by ``pending[-2 - id]`` (int32 token ids kept on the device by earlier sampling)."""
    _dev(table, ids, out, pending)
    _need(pending is None or (pending.dtype == torch.int32 and pending.is_contiguous()), "embed: pending must be int32")
    n, dim = out.shape
    _need(table.dim() == 2 and table.shape[1] == dim and table.is_contiguous(), "embed: table must be [vocab, dim]")
    _need(ids.dtype == torch.int32 and ids.numel() == n and ids.is_contiguous(), "embed: ids must be int32 [n]")
    _need(out.dtype == torch.float32 and out.is_contiguous(), "embed: out must be contiguous fp32")
    _check(lib().ka_embed(table.data_ptr(), code_of(table.dtype), ids.data_ptr(), _ptr(pending),
                          0 if pending is None else pending.numel(), table.shape[0], out.data_ptr(), n, dim,
                          float(scale), stream_ptr()))


def adjust_logits(logits: torch.Tensor, scale: float = 1.0, softcap: Optional[float] = None) -> None:
    """In place: ``logits *= scale``, then ``softcap * tanh(logits / softcap)`` if a cap is given."""
    _dev(logits)
    _need(logits.dtype == torch.float32 and logits.is_contiguous(), "adjust_logits: logits must be contiguous fp32")
    _need(softcap is None or softcap > 0, "adjust_logits: the cap must be positive")
    _check(lib().ka_adjust_logits(logits.data_ptr(), logits.numel(), float(scale), float(softcap or 0.0), stream_ptr()))


def scatter_rows(src: torch.Tensor, rows: torch.Tensor, out: torch.Tensor) -> None:
    """``out[rows[i]] = src[i]`` in fp32 (given embeddings spliced into the stream); a negative ``rows[i]``
    is passed over."""
    _dev(src, rows, out)
    m, dim = src.shape
    _need(out.dim() == 2 and out.shape[1] == dim and out.dtype == torch.float32 and out.is_contiguous(),
          "scatter_rows: out must be contiguous fp32 [n, dim]")
    _need(src.is_contiguous(), "scatter_rows: src must be contiguous")
    _need(rows.dtype == torch.int32 and rows.numel() == m and rows.is_contiguous(), "scatter_rows: rows int32 [m]")
    _check(lib().ka_scatter_rows(src.data_ptr(), code_of(src.dtype), rows.data_ptr(), out.data_ptr(), m, dim,
                                 stream_ptr()))


def layernorm(x: torch.Tensor, gamma: torch.Tensor, beta: Optional[torch.Tensor], eps: float, out: torch.Tensor,
              rows: Optional[torch.Tensor] = None) -> None:
    """LayerNorm of fp32 rows of ``x`` (all, or those named by ``rows``) into ``out``."""
    _dev(x, gamma, beta, out, rows)
    n, dim = out.shape
    _need(x.dtype == torch.float32 and x.dim() == 2 and x.shape[1] == dim and x.is_contiguous(),
          "layernorm: x must be contiguous fp32 [*, dim]")
    _need(gamma.dtype == torch.float32 and gamma.numel() == dim, "layernorm: gamma must be fp32 [dim]")
    _need(beta is None or (beta.dtype == torch.float32 and beta.numel() == dim), "layernorm: beta must be fp32 [dim]")
    _need(out.is_contiguous(), "layernorm: out must be contiguous")
    if rows is None:
        _need(x.shape[0] == n, "layernorm: row counts differ")
    else:
        _need(rows.dtype == torch.int32 and rows.numel() == n and rows.is_contiguous(), "layernorm: rows int32 [n]")
    _check(lib().ka_layernorm(x.data_ptr(), _ptr(rows), gamma.data_ptr(), _ptr(beta), float(eps), out.data_ptr(),
                              code_of(out.dtype), n, dim, stream_ptr()))


ROTARY_PAIRINGS = {"halves": 0, "interleaved": 1}


def rope_cache(qkv: torch.Tensor, positions: torch.Tensor, slots: Optional[torch.Tensor],
               table: Optional[torch.Tensor], k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor],
               n_heads: int, n_kv_heads: int, head_dim: int, page_size: int, pairing: str = "halves") -> None:
    """Rotate q in place and write rotated k and v into the paged cache.

    ``qkv``: ``[n, (H + 2 Hkv) hd]``; ``table``: fp32 ``[positions, R]`` (the cosines of the R/2
    angles of a position, then their sines) or ``None`` for no rotation; ``pairing``: which
    channels angle ``i`` turns, ``"halves"`` (``i`` and ``i + R/2``) or ``"interleaved"`` (``2i`` and
    ``2i + 1``); key cache ``[pages, Hkv, page_size, hd]``, value cache ``[pages, Hkv, hd, page_size]``;
    ``slots`` ``None`` writes nothing.
    """
    _need(pairing in ROTARY_PAIRINGS, f"rope_cache: pairing {pairing!r} is not one of {sorted(ROTARY_PAIRINGS)}")
    _dev(qkv, positions, slots, table, k_cache, v_cache)
    n = qkv.shape[0]
    _need(qkv.dim() == 2 and qkv.stride(1) == 1 and qkv.shape[1] == (n_heads + 2 * n_kv_heads) * head_dim,
          "rope_cache: qkv must be [n, (H + 2 Hkv) hd]")
    _need(positions.dtype == torch.int32 and positions.numel() == n and positions.is_contiguous(),
          "rope_cache: positions int32 [n]")
    rot, rows = 0, 0
    if table is not None:
        _need(table.dtype == torch.float32 and table.dim() == 2 and table.is_contiguous(),
              "rope_cache: table must be contiguous fp32 [positions, R]")
        rows, rot = table.shape
    if slots is not None:
        _need(slots.dtype == torch.int32 and slots.numel() == n and slots.is_contiguous(), "rope_cache: slots int32 [n]")
        _need(k_cache is not None and v_cache is not None, "rope_cache: cache tensors missing")
        _check_caches("rope_cache", k_cache, v_cache, qkv.dtype, n_kv_heads, page_size, head_dim)
    _check(lib().ka_rope_cache(qkv.data_ptr(), code_of(qkv.dtype), qkv.stride(0), positions.data_ptr(), _ptr(slots),
                               _ptr(table), rows, _ptr(k_cache), _ptr(v_cache), n, n_heads, n_kv_heads, head_dim,
                               rot, page_size, ROTARY_PAIRINGS[pairing], stream_ptr()))


def linear_generic(a: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
                   act: int = 0, accumulate: bool = False) -> None:
    """``out = act(a @ weight.T + bias)`` or ``out += ...``; plain fp32 FMA, any sizes and type mix."""
    _dev(a, weight, bias, out)
    m, k = a.shape
    n = weight.shape[0]
    _need(weight.dim() == 2 and weight.shape[1] == k, f"linear: weight {tuple(weight.shape)} does not match K={k}")
    gated = bool(act & 0x100)          # (ops.linear.ACT_GATED: pairs of weight rows make one output)
    _need(not gated or (n % 2 == 0 and not accumulate), "linear: a gated linear needs an even number of weight rows and no accumulation")
    n_out = n // 2 if gated else n
    _need(out.dim() == 2 and tuple(out.shape) == (m, n_out), f"linear: out {tuple(out.shape)} is not [{m}, {n_out}]")
    _need(a.stride(1) == 1 and weight.stride(1) == 1 and out.stride(1) == 1, "linear: rows must be contiguous")
    _need(bias is None or (bias.dtype == torch.float32 and bias.numel() == n and bias.is_contiguous()),
          "linear: bias must be fp32 [N]")
    _check(lib().ka_linear_generic(a.data_ptr(), code_of(a.dtype), a.stride(0), weight.data_ptr(),
                                   code_of(weight.dtype), weight.stride(0), _ptr(bias), out.data_ptr(),
                                   code_of(out.dtype), out.stride(0), m, n, k, act, int(accumulate), stream_ptr()))


def attention_generic(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
                      token_row: torch.Tensor, kv_lo: Optional[torch.Tensor], kv_hi: torch.Tensor,
                      out: torch.Tensor, scale: float, n_heads: int, n_kv_heads: int, head_dim: int) -> None:
    """Paged attention of ``n`` packed tokens; ``q`` may be a strided view into a qkv buffer."""
    _dev(q, k_cache, v_cache, block_table, token_row, kv_lo, kv_hi, out)
    n = q.shape[0]
    _need(q.dim() == 2 and q.stride(1) == 1 and q.shape[1] >= n_heads * head_dim, "attention: q must be [n, >= H hd]")
    _need(out.dim() == 2 and out.stride(1) == 1 and tuple(out.shape) == (n, n_heads * head_dim) and out.dtype == q.dtype,
          "attention: out must be [n, H hd] of the q type")
    page_size = k_cache.shape[2]
    _check_caches("attention", k_cache, v_cache, q.dtype, n_kv_heads, page_size, head_dim)
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous(),
          "attention: block table must be contiguous int32 [rows, pages]")
    for t in (token_row, kv_hi) + ((kv_lo,) if kv_lo is not None else ()):
        _need(t.dtype == torch.int32 and t.numel() == n and t.is_contiguous(), "attention: per-token int32 [n] expected")
    _check(lib().ka_attention_generic(q.data_ptr(), code_of(q.dtype), q.stride(0), k_cache.data_ptr(),
                                      v_cache.data_ptr(), block_table.data_ptr(), block_table.shape[1],
                                      token_row.data_ptr(), _ptr(kv_lo), kv_hi.data_ptr(), out.data_ptr(),
                                      out.stride(0), float(scale), n, n_heads, n_kv_heads, head_dim, page_size,
                                      stream_ptr()))


def _pending_args(who: str, rows: int, pending, pending_at):
    if pending is None:
        return None, None, 0
    _need(pending.dtype == torch.int32 and pending.is_contiguous(), f"{who}: pending must be int32")
    _need(pending_at is not None and pending_at.dtype == torch.int32 and pending_at.numel() == rows
          and pending_at.is_contiguous(), f"{who}: pending_at int32 [rows]")
    return pending.data_ptr(), pending_at.data_ptr(), pending.numel()


def argmax(logits: torch.Tensor, out: torch.Tensor, pending: Optional[torch.Tensor] = None,
           pending_at: Optional[torch.Tensor] = None) -> None:
    """Index of the largest logit of every fp32 row into int32 ``out`` (on the device or in pinned
    host memory), and into ``pending[pending_at[row]]`` if a table of latest tokens is given
    (negative place: skipped)."""
    _dev(logits, pending, pending_at)
    _dev_or_pinned(out)
    rows, vocab = logits.shape
    _need(logits.dtype == torch.float32 and logits.stride(1) == 1, "argmax: logits must be fp32 rows")
    _need(out.dtype == torch.int32 and out.numel() == rows and out.is_contiguous(), "argmax: out int32 [rows]")
    _check(lib().ka_argmax(logits.data_ptr(), logits.stride(0), out.data_ptr(), rows, vocab,
                           *_pending_args("argmax", rows, pending, pending_at), stream_ptr()))


def sample(logits: torch.Tensor, temps: torch.Tensor, top_ps: Optional[torch.Tensor], rng_key: torch.Tensor,
           rng_counter: torch.Tensor, out: torch.Tensor, pending: Optional[torch.Tensor] = None,
           pending_at: Optional[torch.Tensor] = None) -> None:
    """Temperature and top-p sampling of every row (greedy where temperature <= 1e-6); the
    token also goes to ``pending[pending_at[row]]`` if given."""
    _dev(logits, temps, top_ps, rng_key, rng_counter, pending, pending_at)
    _dev_or_pinned(out)
    rows, vocab = logits.shape
    _need(logits.dtype == torch.float32 and logits.stride(1) == 1, "sample: logits must be fp32 rows")
    _need(temps.dtype == torch.float32 and temps.numel() == rows, "sample: temps fp32 [rows]")
    _need(top_ps is None or (top_ps.dtype == torch.float32 and top_ps.numel() == rows), "sample: top_ps fp32 [rows]")
    _need(rng_key.dtype == torch.int64 and rng_key.numel() == rows, "sample: rng_key int64 [rows]")
    _need(rng_counter.dtype == torch.int32 and rng_counter.numel() == rows, "sample: rng_counter int32 [rows]")
    _need(out.dtype == torch.int32 and out.numel() == rows and out.is_contiguous(), "sample: out int32 [rows]")
    _check(lib().ka_sample(logits.data_ptr(), logits.stride(0), temps.data_ptr(), _ptr(top_ps), rng_key.data_ptr(),
                           rng_counter.data_ptr(), out.data_ptr(), rows, vocab,
                           *_pending_args("sample", rows, pending, pending_at), stream_ptr()))


def set_sample_passes_only(on: bool) -> None:
    """Sends every row through the sampling kernel that passes over the row many times (it
    otherwise serves rows of more than 65536 logits only): for tests."""
    lib().ka_sample_set_passes_only(int(bool(on)))


def _logit_rows(who: str, logits: torch.Tensor):
    _need(logits.dim() == 2 and logits.dtype == torch.float32 and logits.stride(1) == 1, f"{who}: logits must be fp32 rows")
    return logits.shape


def suppress_tokens(logits: torch.Tensor, rows: torch.Tensor, tokens: torch.Tensor) -> None:
    """``logits[rows[i], tokens[i]] = -inf`` (ids outside the vocabulary are passed over)."""
    _dev(logits, rows, tokens)
    n_rows, vocab = _logit_rows("suppress_tokens", logits)
    _need(rows.dtype == torch.int32 and tokens.dtype == torch.int32 and rows.numel() == tokens.numel()
          and rows.is_contiguous() and tokens.is_contiguous(), "suppress_tokens: rows and tokens int32 of one length")
    _check(lib().ka_suppress_tokens(logits.data_ptr(), logits.stride(0), rows.data_ptr(), tokens.data_ptr(),
                                    rows.numel(), vocab, stream_ptr()))


def allow_tokens(logits: torch.Tensor, starts: torch.Tensor, allowed: torch.Tensor) -> None:
    """Row ``r`` keeps only the tokens ``allowed[starts[r]:starts[r + 1]]`` (sorted ascending);
    a row with an empty list is left alone."""
    _dev(logits, starts, allowed)
    n_rows, vocab = _logit_rows("allow_tokens", logits)
    _need(starts.dtype == torch.int32 and starts.numel() == n_rows + 1 and starts.is_contiguous(),
          "allow_tokens: starts int32 [rows + 1]")
    _need(allowed.dtype == torch.int32 and allowed.is_contiguous(), "allow_tokens: allowed int32")
    _check(lib().ka_allow_tokens(logits.data_ptr(), logits.stride(0), starts.data_ptr(), allowed.data_ptr(), n_rows,
                                 vocab, stream_ptr()))


def token_logprobs(logits: torch.Tensor, ids: torch.Tensor, temps: Optional[torch.Tensor], out: torch.Tensor) -> None:
    """Log-probability of ``ids[r]`` under ``softmax(logits[r] / T)``; greedy rows (``T <= 1e-6`` or
    no temperatures) give 0 for the argmax and -inf otherwise."""
    _dev(logits, ids, temps, out)
    n_rows, vocab = _logit_rows("token_logprobs", logits)
    _need(ids.dtype == torch.int32 and ids.numel() == n_rows and ids.is_contiguous(), "token_logprobs: ids int32 [rows]")
    _need(temps is None or (temps.dtype == torch.float32 and temps.numel() == n_rows), "token_logprobs: temps fp32 [rows]")
    _need(out.dtype == torch.float32 and out.numel() == n_rows and out.is_contiguous(), "token_logprobs: out fp32 [rows]")
    _check(lib().ka_token_logprobs(logits.data_ptr(), logits.stride(0), ids.data_ptr(), _ptr(temps), out.data_ptr(),
                                   n_rows, vocab, stream_ptr()))
