"""The Python entry point: ``InferenceEngine.create(cfg)`` and its ways to generate.

In the reference's manner (``kestrel/engine/core.py:262-319`` ``create``, ``:556,767``
``submit`` / ``submit_streaming``, ``:486`` ``shutdown``; results
``kestrel/engine/_types.py:35-56``): an asynchronous facade over one scheduler thread that
owns the GPU. Request options keep the reference's names and meanings: ``temperature``
(>= 0, ``None`` -> 0.0), ``top_p`` (in (0, 1], ``None`` -> 1.0), ``max_tokens`` / ``max_new_tokens``
(``core.py:1161-1174``). The reference's skills, tokenizer and image encoder are outside
this engine: prompts are token ids, an image is a block of given embeddings.
"""

from __future__ import annotations

import asyncio
import logging
import queue
import threading
import time
from concurrent.futures import Future
from dataclasses import dataclass
from collections.abc import Mapping, Sequence as Sequence_abc
from typing import AsyncIterator, Dict, List, Optional, Sequence

import torch

from ..config.runtime import RuntimeConfig
from ..sampling.sampler import Sampler
from .loading import load_model, make_runner
from .scheduler import GenerationScheduler
from .types import GeneratedPrefix, GenerationRequest, SchedulerResult

_LOGGER = logging.getLogger(__name__)


@dataclass
class EngineMetrics:
    """Token counts and timing of one request (``kestrel/engine/_types.py:35-44``)."""

    input_tokens: int
    output_tokens: int
    prefill_time_ms: float
    decode_time_ms: float
    ttft_ms: float


@dataclass
class EngineResult:
    """What a caller gets back (``kestrel/engine/_types.py:47-56``)."""

    request_id: int
    tokens: List[int]
    finish_reason: str
    metrics: EngineMetrics
    output: Dict[str, object]
    logprobs: Optional[List[float]] = None      # of the tokens, if the request asked for them


@dataclass
class StreamUpdate:
    request_id: int
    token: int
    token_index: int


class _Pending:
    def __init__(self, request: GenerationRequest, future: Future, stream: Optional["queue.Queue"]) -> None:
        self.request, self.future, self.stream = request, future, stream


def _generated_prefix(raw) -> GeneratedPrefix:
    """What a resumed request brings: ``None``, a ``GeneratedPrefix``, or a mapping with ``tokens`` and
    optionally ``logprobs`` (the reference's private setting, ``kestrel/engine/core.py:1260-1294``)."""
    if raw is None:
        return GeneratedPrefix()
    if isinstance(raw, GeneratedPrefix):
        tokens, logprobs = raw.tokens, raw.logprobs
    elif isinstance(raw, Mapping):
        unknown = sorted(str(key) for key in set(raw) - {"tokens", "logprobs"})
        if unknown:
            raise TypeError(f"generated_prefix takes the keys 'tokens' and 'logprobs', not {', '.join(unknown)}")
        if "tokens" not in raw:
            raise ValueError("generated_prefix needs 'tokens': the ids the request generated before")
        tokens, logprobs = raw["tokens"], raw.get("logprobs")
    else:
        raise TypeError(f"generated_prefix is a mapping with 'tokens' (and 'logprobs') or None, got {type(raw).__name__}")

    def listed(values, what):
        if isinstance(values, (str, bytes)) or not isinstance(values, (Sequence_abc, torch.Tensor)):
            raise TypeError(f"generated_prefix: {what} must be a sequence, got {type(values).__name__}")
        return values

    tokens = tuple(int(t) for t in listed(() if tokens is None else tokens, "'tokens'"))
    if logprobs is not None:
        logprobs = tuple(float(v) for v in listed(logprobs, "'logprobs'"))
        if len(logprobs) != len(tokens):
            raise ValueError(f"generated_prefix: {len(logprobs)} log-probabilities for {len(tokens)} tokens")
    return GeneratedPrefix(tokens, logprobs)


def pool_pages(cfg: RuntimeConfig, bytes_per_page: int, max_seq: int, free_bytes: Optional[int]) -> int:
    """Pages of the cache pool (each group of layers gets that many), from the one knob that is set:
    pages, a byte budget (``kestrel/kv_cache.py:52-136``), tokens, or by default ``max_batch_size``
    full contexts. ``bytes_per_page``: what a page costs over all layers. ``free_bytes``: what the
    device has free (``None``: not checked); a pool beyond it is refused here, before anything is
    allocated, instead of failing somewhere inside the allocation."""
    if cfg.kv_cache_pages is not None:
        n_pages = cfg.kv_cache_pages
    elif cfg.kv_cache_bytes is not None:
        n_pages = cfg.kv_cache_bytes // max(bytes_per_page, 1)
        if n_pages < 1:
            raise MemoryError(f"kv_cache_bytes={cfg.kv_cache_bytes} holds less than one page of {bytes_per_page} bytes")
    elif cfg.kv_cache_tokens is not None:
        n_pages = -(-cfg.kv_cache_tokens // cfg.page_size)
    else:
        n_pages = cfg.max_batch_size * -(-max_seq // cfg.page_size)
    needed = n_pages * bytes_per_page
    if free_bytes is not None and needed > free_bytes:
        gib = float(1 << 30)
        raise MemoryError(f"the cache pool of {n_pages} pages needs {needed / gib:.1f} GiB, the device has "
                          f"{free_bytes / gib:.1f} GiB free: lower kv_cache_pages / kv_cache_bytes / max_batch_size")
    return n_pages


def _normalise(temperature, top_p):
    temperature = 0.0 if temperature is None else float(temperature)
    top_p = 1.0 if top_p is None else float(top_p)
    if temperature < 0.0:
        raise ValueError("temperature must be non-negative")
    if not 0.0 < top_p <= 1.0:
        raise ValueError("top_p must be in the range (0, 1]")
    return temperature, top_p


class InferenceEngine:
    """Loads a model folder, keeps the cache and runs the scheduler on a thread of its own."""

    def __init__(self, cfg: RuntimeConfig) -> None:
        self.cfg = cfg
        self._inbox: "queue.Queue" = queue.Queue()
        self._thread: Optional[threading.Thread] = None
        self._started = threading.Event()
        self._startup_error: Optional[BaseException] = None
        self._fatal: Optional[BaseException] = None
        self._stop = False
        self._run_gate = threading.Event()          # set: the scheduler thread may launch steps
        self._run_gate.set()
        self._paused = threading.Event()            # set by the scheduler thread once a pause has drained
        self._next_id = 0
        self._id_lock = threading.Lock()
        self.runner = None
        self.scheduler: Optional[GenerationScheduler] = None
        self.plan = None

    # ------------------------------------------------------------------ life cycle
    @classmethod
    async def create(cls, cfg: RuntimeConfig) -> "InferenceEngine":
        engine = cls(cfg)
        await asyncio.get_running_loop().run_in_executor(None, engine.start)
        return engine

    @classmethod
    def create_sync(cls, cfg: RuntimeConfig) -> "InferenceEngine":
        engine = cls(cfg)
        engine.start()
        return engine

    def start(self) -> None:
        if self._thread is not None:
            return
        self._thread = threading.Thread(target=self._scheduler_loop, name="kestrel-scheduler", daemon=True)
        self._thread.start()
        self._started.wait()
        if self._startup_error is not None:
            raise self._startup_error

    def _build(self) -> None:
        cfg = self.cfg
        if cfg.model_path is None:
            raise ValueError("RuntimeConfig.model_path must name a folder with config.json and model.safetensors")
        device = cfg.resolved_device()
        torch.cuda.set_device(device)
        started = time.perf_counter()
        net = load_model(cfg.model_path, cfg.dtype, device, cfg.model)
        self.plan = net.plan
        _LOGGER.info("loaded %s from %s as %s on %s in %.2f s (%d layers, width %d, vocabulary %d)", net.plan.architecture,
                     cfg.model_path, str(cfg.dtype).replace("torch.", ""), device, time.perf_counter() - started,
                     len(net.plan.layers), net.plan.dim, net.plan.vocab_size)
        max_seq = min(cfg.max_seq_len or net.plan.max_positions, net.plan.max_positions)
        from ..cache.manager import CacheManager

        sizing = CacheManager(net.cache_needs(), cfg.page_size, 1, 1, dtype=net.dtype)      # books only: no device memory
        free_bytes, _total = torch.cuda.mem_get_info(device)
        n_pages = pool_pages(cfg, sizing.bytes_per_page(), max_seq, free_bytes)
        self.runner = make_runner(net, cfg.page_size, n_pages, cfg.max_batch_size,
                                  max_tokens_per_step=cfg.max_num_batched_tokens, enable_graphs=cfg.enable_graphs)
        _LOGGER.info("cache pool: %d pages of %d tokens per group of layers (%.2f GiB), %d request slots, contexts up to %d",
                     n_pages, cfg.page_size, n_pages * sizing.bytes_per_page() / float(1 << 30), cfg.max_batch_size, max_seq)
        sampler = Sampler(device, cfg.seed, pending=self.runner.pending)
        self.scheduler = GenerationScheduler(self.runner, sampler, cfg.max_batch_size, cfg.max_num_batched_tokens,
                                             net.plan.eos_token_ids, max_seq, pipeline_depth=cfg.pipeline_depth)
        if cfg.warmup:
            # graphs, scratch memory and plans now, not in the middle of the first steps that need them
            done = self.runner.prepare(cfg.max_num_batched_tokens, wanted_rows=cfg.max_batch_size, tune_linears=cfg.tune_linears)
            sampler.reserve(cfg.max_batch_size)
            _LOGGER.info("warm-up: %d decode graphs and %d graphs of other steps captured in %.2f s, %d prompt steps in %.2f s, "
                         "%.0f MiB of kernel scratch",
                         int(done.get("graphs", 0)), int(done.get("step_graphs", 0)), done.get("capture_s", 0.0), int(done.get("prompt_steps", 0)),
                         done.get("prompt_s", 0.0), done.get("kernel_scratch_bytes", 0) / float(1 << 20))
            if "library_tuned" in done:
                _LOGGER.info("warm-up: %d plans of the vendor library timed, %d of them took another algorithm than the first named",
                             int(done["library_tuned"]), int(done["library_tuned_other"]))

    def _scheduler_loop(self) -> None:
        try:
            self._build()
        except BaseException as exc:  # surfaced to the caller of start()
            _LOGGER.error("start-up failed: %s: %s", type(exc).__name__, exc)
            self._startup_error = exc
            self._started.set()
            return
        self._started.set()
        pending: Dict[int, _Pending] = {}
        scheduler = self.scheduler
        try:
            while True:
                block = not scheduler.has_pending_work()
                while True:
                    try:
                        item = self._inbox.get(block=block, timeout=0.05 if block else None)
                    except queue.Empty:
                        break
                    block = False
                    if item is None:
                        self._stop = True
                        continue
                    try:
                        scheduler.enqueue_request(item.request)
                        pending[item.request.request_id] = item
                    except Exception as exc:
                        _LOGGER.warning("request %d refused at the door: %s: %s", item.request.request_id,
                                        type(exc).__name__, exc)
                        self._deliver_error(item, exc)
                if self._stop and not scheduler.has_pending_work():
                    break
                if not self._run_gate.is_set():
                    # paused: what is in flight is read, the device is left idle, and nothing is
                    # launched until resume(); requests that arrive meanwhile wait in the scheduler
                    scheduler.drain()
                    for result in scheduler.pop_completed():
                        self._deliver(pending.pop(result.request_id), result)
                    torch.cuda.synchronize(self.runner.device)
                    self._paused.set()
                    self._run_gate.wait(timeout=0.1)
                    continue
                if scheduler.has_pending_work():
                    scheduler.advance()
                    for result in scheduler.pop_completed():
                        self._deliver(pending.pop(result.request_id), result)
        except BaseException as exc:
            self._fatal = exc
            _LOGGER.exception("the scheduler thread has stopped; %d requests fail with it", len(pending))
            for item in pending.values():
                self._deliver_error(item, exc)
            while True:
                try:
                    item = self._inbox.get_nowait()
                except queue.Empty:
                    break
                if item is not None:
                    self._deliver_error(item, exc)

    def _deliver(self, item: _Pending, result: SchedulerResult) -> None:
        if result.finish_reason == "error":
            self._deliver_error(item, RuntimeError(result.error or "request failed"))
            return
        m = result.metrics
        out = EngineResult(result.request_id, result.tokens, result.finish_reason,
                           EngineMetrics(m.prompt_tokens, m.decode_tokens, m.prefill_time_ms, m.decode_time_ms, m.ttft_ms),
                           {"tokens": result.tokens}, result.logprobs)
        if item.stream is not None:
            item.stream.put(None)
        item.future.set_result(out)

    def _deliver_error(self, item: _Pending, exc: BaseException) -> None:
        if item.stream is not None:
            item.stream.put(exc)
        if not item.future.done():
            item.future.set_exception(exc)

    def pause(self, *, timeout: Optional[float] = None) -> bool:
        """Stop launching steps and wait until the device is idle (``kestrel/engine/core.py:810-825``).
        Requests in flight keep their pages and go on after ``resume``; requests submitted meanwhile
        wait. Returns whether the scheduler thread has acknowledged within ``timeout`` seconds."""
        if self._thread is None or self._fatal is not None:
            return True
        self._paused.clear()
        self._run_gate.clear()
        return self._paused.wait(timeout)

    def resume(self) -> None:
        """Let the scheduler thread launch steps again (``kestrel/engine/core.py:827-836``)."""
        self._paused.clear()
        self._run_gate.set()

    def shutdown_sync(self) -> None:
        if self._thread is None:
            return
        self._run_gate.set()
        self._inbox.put(None)
        self._thread.join()
        self._thread = None

    async def shutdown(self) -> None:
        await asyncio.get_running_loop().run_in_executor(None, self.shutdown_sync)

    # ------------------------------------------------------------------ requests
    def _make_request(self, prompt_ids, max_new_tokens, temperature, top_p, prefix_embeds, prefix_ids, stop_ids, seed,
                      on_token, return_logprobs=False, suppress_next_token_ids=(), suppressed_token_ids=(),
                      allowed_token_ids=None, generated_prefix=None, prompt_embeds=None, blocks=None) -> GenerationRequest:
        if self._fatal is not None:
            raise RuntimeError("the engine has stopped after an error") from self._fatal
        if self._thread is None:
            raise RuntimeError("the engine is not running")
        temperature, top_p = _normalise(temperature, top_p)
        if max_new_tokens is None or int(max_new_tokens) <= 0:
            raise ValueError("max_new_tokens must be positive")
        with self._id_lock:
            request_id = self._next_id
            self._next_id += 1
        return GenerationRequest(request_id, list(prompt_ids), int(max_new_tokens), temperature, top_p, prefix_embeds,
                                 tuple(prefix_ids), None if stop_ids is None else tuple(stop_ids), seed, on_token,
                                 return_logprobs=bool(return_logprobs),
                                 suppress_next_token_ids=tuple(int(t) for t in suppress_next_token_ids or ()),
                                 suppressed_token_ids=tuple(int(t) for t in suppressed_token_ids or ()),
                                 allowed_token_ids=None if allowed_token_ids is None
                                 else tuple(int(t) for t in allowed_token_ids),
                                 generated_prefix=_generated_prefix(generated_prefix), prompt_embeds=prompt_embeds,
                                 blocks=None if blocks is None else tuple((int(lo), int(hi)) for lo, hi in blocks))

    def submit_sync(self, prompt_ids: Sequence[int], *, max_new_tokens: int, temperature: Optional[float] = None,
                    top_p: Optional[float] = None, prefix_embeds: Optional[torch.Tensor] = None,
                    prefix_ids: Sequence[int] = (), stop_ids: Optional[Sequence[int]] = None,
                    seed: Optional[int] = None, _stream: Optional["queue.Queue"] = None, **sampling) -> Future:
        """Queue a request; the returned future resolves to an ``EngineResult``. ``sampling`` takes
        ``return_logprobs``, ``suppress_next_token_ids``, ``suppressed_token_ids``,
        ``allowed_token_ids`` and ``generated_prefix`` (tokens the request generated before: they are
        fed after the prompt, count against ``max_new_tokens`` and head the result)
        (``kestrel/engine/core.py:556-597``); and, for prompts with more than one block of given
        embeddings, ``prompt_embeds`` (rows for the places of ``prompt_ids`` that hold -1) and ``blocks``
        (the position ranges that see each other both ways)."""
        unknown = set(sampling) - {"return_logprobs", "suppress_next_token_ids", "suppressed_token_ids",
                                   "allowed_token_ids", "generated_prefix", "prompt_embeds", "blocks"}
        if unknown:
            raise TypeError(f"unknown options: {sorted(unknown)}")
        on_token = None
        if _stream is not None:
            def on_token(token, index, _q=_stream):
                _q.put((token, index))
        request = self._make_request(prompt_ids, max_new_tokens, temperature, top_p, prefix_embeds, prefix_ids,
                                     stop_ids, seed, on_token, **sampling)
        future: Future = Future()
        future.request_id = request.request_id
        self._inbox.put(_Pending(request, future, _stream))
        return future

    def generate_sync(self, prompt_ids: Sequence[int], **options) -> EngineResult:
        return self.submit_sync(prompt_ids, **options).result()

    def generate_batch_sync(self, prompts: Sequence[Sequence[int]], **options) -> List[EngineResult]:
        futures = [self.submit_sync(p, **options) for p in prompts]
        return [f.result() for f in futures]

    async def submit(self, prompt_ids: Sequence[int], *, max_new_tokens: int, temperature: Optional[float] = None,
                     top_p: Optional[float] = None, prefix_embeds: Optional[torch.Tensor] = None,
                     prefix_ids: Sequence[int] = (), stop_ids: Optional[Sequence[int]] = None,
                     seed: Optional[int] = None, **sampling) -> EngineResult:
        future = self.submit_sync(prompt_ids, max_new_tokens=max_new_tokens, temperature=temperature, top_p=top_p,
                                  prefix_embeds=prefix_embeds, prefix_ids=prefix_ids, stop_ids=stop_ids, seed=seed,
                                  **sampling)
        return await asyncio.wrap_future(future)

    async def generate(self, prompt_ids: Sequence[int], *, settings: Optional[dict] = None, **options) -> EngineResult:
        """``settings`` takes the reference's keys: ``temperature``, ``top_p``, ``max_tokens`` and the
        private ``_logprobs``, ``_suppress_next_token_ids`` and ``_generated_prefix``
        (``kestrel/engine/core.py:556-597``)."""
        settings = dict(settings or {})
        if "max_tokens" in settings:
            options.setdefault("max_new_tokens", settings.pop("max_tokens"))
        if "_logprobs" in settings:
            options.setdefault("return_logprobs", bool(settings.pop("_logprobs")))
        if "_suppress_next_token_ids" in settings:
            options.setdefault("suppress_next_token_ids", settings.pop("_suppress_next_token_ids"))
        if "_generated_prefix" in settings:
            options.setdefault("generated_prefix", settings.pop("_generated_prefix"))
        for key in ("temperature", "top_p"):
            if key in settings:
                options.setdefault(key, settings.pop(key))
        if settings:
            raise ValueError(f"unknown settings: {sorted(settings)}")
        return await self.submit(prompt_ids, **options)

    async def submit_streaming(self, prompt_ids: Sequence[int], **options) -> AsyncIterator[StreamUpdate]:
        """Yields a ``StreamUpdate`` per token as it is committed."""
        stream: "queue.Queue" = queue.Queue()
        future = self.submit_sync(prompt_ids, _stream=stream, **options)
        loop = asyncio.get_running_loop()
        request_id = future.request_id
        while True:
            item = await loop.run_in_executor(None, stream.get)
            if item is None:
                break
            if isinstance(item, BaseException):
                raise item
            token, index = item
            yield StreamUpdate(request_id, token, index)
        await asyncio.wrap_future(future)
