"""Decode and prefill throughput of the engine on one MI355X.

``python bench.py --gpus 1 --steps K --warmup W`` prints one JSON line. A step is one
decode step of the default batch (8 requests, each holding ``context`` tokens: a block of
prefix embeddings and text ids) through the engine's step function with greedy sampling
on the GPU. The model has the layer sizes of the Moondream 2 text decoder with seeded
random weights N(0, 0.02) in bf16; inputs are synthetic. Besides ``value`` (decoded tokens
a second) the line carries a 2,048-token prefill, the decode step's HBM roofline and
decode throughput at batch 1 and 64. Beside the nominal peaks the line names what this GPU reaches on a plain
read stream and on a loop of matrix instructions (``peak_measured``; ``--no-peaks`` leaves that out).

``--workload waves256`` and ``--workload mixed48`` (the latter meant for ``--sizes phi2``) measure
the whole engine instead: a model folder is written with seeded random weights, loaded through the
loader, and requests go through ``InferenceEngine`` (scheduler, sampler, paged cache under
pressure); the line then reports generated tokens a second. With ``--check N`` (meant for ``--layers 2``) the first N
greedy requests of such a run are compared, token by token, with the plain implementation under ``tests/``.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# Layer sizes of the benchmark model (Moondream 2 text decoder) and its workload.
MODEL = {"dim": 2048, "ff_dim": 8192, "n_layers": 24, "vocab_size": 51200, "max_context": 2048, "n_heads": 32,
         "n_kv_heads": 32, "rope_theta": 10000.0, "prefix_attn": 730, "layer_norm_eps": 1e-5}
# Another member of the family for measurements beside the default: Phi-2's layer sizes (head size 80).
SIZES = {
    "moondream2": MODEL,
    "phi2": {"dim": 2560, "ff_dim": 10240, "n_layers": 32, "vocab_size": 51200, "max_context": 2048, "n_heads": 32,
             "n_kv_heads": 32, "rope_theta": 10000.0, "prefix_attn": 0, "layer_norm_eps": 1e-5, "rotary_dim": 32},
}
LABELS = {"moondream2": ("Moondream 2 text decoder sizes", "moondream2-text"), "phi2": ("Phi-2 layer sizes", "phi2-sizes")}
CONTEXT = 1024          # tokens each request holds when decoding starts (730 prefix + 294 text)
PREFILL_TOKENS = 2048
PAGE_SIZE = 16
SEED = 2
PEAK_HBM = 8.0e12
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}


def build_model(layers: int, dtype, device, sizes=None):
    """The benchmark model with random weights drawn on the GPU (nothing is read from disk)."""
    import torch

    from kestrel_amd.config import get_spec
    from kestrel_amd.models import DecoderModel
    from kestrel_amd.weights import InitRecipe, random_tensor

    spec = get_spec("moondream2")
    typed = spec.read_config({"text": dict(sizes or MODEL, n_layers=layers)})
    net = DecoderModel(spec.build_plan(typed))
    recipe = InitRecipe(std=0.02)
    store = torch.bfloat16
    tensors = {name: random_tensor(name, pspec, SEED, recipe, device=device).to(store if dtype == torch.bfloat16 else dtype)
               for name, pspec in net.params().items()}
    net.bind(tensors, dtype, device)
    return net, typed


def model_bytes(net, dtype_size: int) -> int:
    """Bytes of weights a decode step reads once: every linear, norm and the head (the
    embedding table is read only at the rows of the batch)."""
    total = 0
    emb = net.plan.names["embedding"]
    for name, pspec in net.params().items():
        if name == emb:
            continue
        count = 1
        for s in pspec.shape:
            count *= s
        total += count * dtype_size
    return total


def prefill_flops(typed, tokens: int, prefix: int) -> float:
    """Multiply-adds x 2 of one prompt of ``tokens`` positions whose first ``prefix`` are a
    bidirectional block; the head runs on the last position only."""
    d, ff, hd = typed.dim, typed.ff_dim, typed.head_dim
    qkv = (typed.n_heads + 2 * typed.n_kv_heads) * hd
    per_token_linear = 2 * (d * qkv + typed.n_heads * hd * d + 2 * d * ff)
    pairs = prefix * prefix + sum(q + 1 for q in range(prefix, tokens))
    attention = 4 * hd * typed.n_heads * pairs
    return typed.n_layers * (tokens * per_token_linear + attention) + 2 * d * typed.vocab_size


class DecodeBench:
    """A batch of requests prefilled to ``context`` tokens, then decoded step by step."""

    def __init__(self, net, typed, batch: int, context: int, steps_total: int):
        import torch

        from kestrel_amd.engine.loading import make_runner
        from kestrel_amd.engine.step import PENDING_TOKEN, StepEntry
        from kestrel_amd.sampling import Sampler

        self.torch, self.StepEntry, self.PENDING = torch, StepEntry, PENDING_TOKEN
        self.net, self.typed, self.batch, self.context = net, typed, batch, context
        pages_per_request = -(-(context + steps_total + 1) // PAGE_SIZE)
        self.runner = make_runner(net, PAGE_SIZE, batch * pages_per_request, batch, max_tokens_per_step=max(4096, context),
                                  enable_graphs=True)
        self.sampler = Sampler(net.device, pending=self.runner.pending)
        self.host = [torch.empty(batch, dtype=torch.int32, pin_memory=True) for _ in range(2)]
        self.unread = None                      # (event, pinned tokens) of the step launched last
        self.n_steps = 0
        gen = torch.Generator().manual_seed(SEED)
        prefix = min(typed.prefix_attn, context - 1)
        self.slots = []
        last = []
        for _ in range(batch):
            slot = self.runner.admit()
            embeds = torch.randn(prefix, typed.dim, generator=gen)
            ids = torch.randint(0, typed.vocab_size, (context - prefix,), generator=gen).tolist()
            entry = StepEntry(slot, [-1] * prefix + ids, want=[context - 1], embeds=embeds.to(net.device),
                              bidirectional=[(0, prefix)] if prefix else [])
            logits = self.runner.step([entry])
            last.append(int(self.sampler.greedy(logits, slots=[slot])[0]))
            self.slots.append(slot)
        self.last = last

    def step(self):
        """One decode step as the scheduler runs it with two steps in flight: the next step is
        launched with the tokens that sampling left on the device, then the tokens of the step
        before are read on the host."""
        torch = self.torch
        entries = [self.StepEntry(slot, [self.PENDING], want=[0]) for slot in self.slots]
        logits = self.runner.step(entries)
        host = self.host[self.n_steps % 2]
        self.sampler.greedy(logits, out=host, slots=self.runner.logit_slots)      # (the kernel writes into the pinned memory)
        event = torch.cuda.Event()
        event.record()
        if self.unread is not None:
            self.unread[0].synchronize()
            self.last = self.unread[1].tolist()
        self.unread = (event, host)
        self.n_steps += 1

    def kv_bytes_now(self, dtype_size: int) -> int:
        t = self.typed
        per_token = 2 * t.n_kv_heads * t.head_dim * dtype_size * t.n_layers
        return per_token * sum(self.runner.held[s] for s in self.slots)

    def close(self):
        for slot in self.slots:
            self.runner.release(slot)
        self.runner = None


def time_decode(net, typed, batch, context, steps, warmup):
    import torch

    bench = DecodeBench(net, typed, batch, context, steps + warmup)
    for _ in range(warmup):
        bench.step()
    torch.cuda.synchronize()
    kv_start = bench.kv_bytes_now(2)
    started = time.perf_counter()
    for _ in range(steps):
        bench.step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - started
    kv_end = bench.kv_bytes_now(2)
    bench.close()
    torch.cuda.empty_cache()
    return elapsed, 0.5 * (kv_start + kv_end)


def time_prefill(net, typed, tokens, repeats=8):
    import torch

    from kestrel_amd.engine.loading import make_runner
    from kestrel_amd.engine.step import StepEntry

    # (as the engine runs it: a step short enough for the host's launches to take longer than its kernels is a replayed graph)
    runner = make_runner(net, PAGE_SIZE, -(-tokens // PAGE_SIZE) + 1, 1, max_tokens_per_step=tokens, enable_graphs=True)
    gen = torch.Generator().manual_seed(SEED + 1)
    prefix = min(typed.prefix_attn, tokens - 1)
    embeds = torch.randn(prefix, typed.dim, generator=gen).to(net.device)
    ids = torch.randint(0, typed.vocab_size, (tokens - prefix,), generator=gen).tolist()
    times = []
    for i in range(repeats + 1):
        slot = runner.admit()
        entry = StepEntry(slot, [-1] * prefix + ids, want=[tokens - 1], embeds=embeds,
                          bidirectional=[(0, prefix)] if prefix else [])
        torch.cuda.synchronize()
        started = time.perf_counter()
        runner.step([entry])
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - started
        runner.release(slot)
        if i > 0:                      # the first run warms up
            times.append(elapsed)
    times.sort()
    return times[len(times) // 2], times[0]          # the median of the runs, and the best of them


def write_model_folder(sizes: dict, layers: int, seed: int) -> str:
    """A model folder (config.json, model.safetensors) with seeded random weights N(0, 0.02)."""
    import tempfile

    from kestrel_amd.weights import InitRecipe, write_random_model

    folder = tempfile.mkdtemp(prefix="kestrel_amd_bench_")
    write_random_model(folder, {"text": dict(sizes, n_layers=layers)}, seed, InitRecipe(std=0.02))
    return folder


def check_greedy(args, sizes: dict, folder: str, greedy: dict, results, prefix) -> int:
    """``--check N``: the first N greedy requests of a workload against the plain implementation under ``tests/``
    (float64, whole sequences, no cache): every token the engine generated must be the plain model's choice
    after the engine's own earlier tokens, up to what the precision leaves of a near tie (twice the bound the
    tests put on a bf16 logit: 3 % of the row's spread + 1 % of the value). Returns how many were compared;
    raises if a token is not."""
    if args.check <= 0:
        return 0
    from safetensors.torch import load_file

    from tests.plain import moondream_plain as plain

    weights = {k: v.double() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    cfg = dict(sizes, n_layers=args.layers)
    done = 0
    for index in sorted(greedy)[:args.check]:
        ids, tokens = greedy[index], results[index].tokens
        logits = plain.forward(cfg, weights, list(ids) + tokens[:-1], prefix)
        first = (0 if prefix is None else prefix.shape[0]) + len(ids) - 1
        for i, token in enumerate(tokens):
            row = logits[first + i]
            gap, allowed = float(row.max() - row[token]), 2 * float(0.03 * row.std() + 0.01 * row.max().abs())
            if args.dtype == "fp32":
                allowed = 1e-4
            if gap > allowed:
                raise AssertionError(f"request {index}: token {i} is {token}, the plain implementation prefers "
                                     f"{int(row.argmax())} by {gap:.3g} (allowed {allowed:.3g})")
        done += 1
    return done


def run_workload(args, sizes: dict) -> dict:
    """Requests through the entry point. ``waves256``: 256 requests in 4 waves, each a block of 730
    given embeddings and 32 to 128 ids, 128 new tokens, half greedy and half at temperature 1, in
    a cache pool of about 60 GB. ``mixed48``: 48 requests with prompts of 64 to 1,536 ids fed in
    portions of at most 512 tokens beside the decoded tokens of the others, 128 new tokens each at
    temperature 0.7."""
    import random
    import shutil

    import torch

    from kestrel_amd import InferenceEngine, RuntimeConfig

    waves = args.workload == "waves256"
    seed = 4 if waves else 3
    started = time.perf_counter()
    folder = write_model_folder(sizes, args.layers, seed)
    written = time.perf_counter() - started
    n_requests, n_new = (256, 128) if waves else (48, 128)
    if waves:
        cfg = RuntimeConfig(model_path=folder, dtype=args.dtype, max_batch_size=args.max_batch_size or 64,
                            kv_cache_bytes=60 * 10 ** 9 * args.layers // sizes["n_layers"], max_seq_len=2048, seed=seed,
                            tune_linears=args.tune_linears)
    else:
        cfg = RuntimeConfig(model_path=folder, dtype=args.dtype, max_batch_size=args.max_batch_size or 48,
                            max_num_batched_tokens=512, max_seq_len=2048, seed=seed, tune_linears=args.tune_linears)
    started = time.perf_counter()
    engine = InferenceEngine.create_sync(cfg)
    loaded = time.perf_counter() - started
    try:
        rng = random.Random(seed)
        vocab, dim = sizes["vocab_size"], sizes["dim"]
        prefix = torch.randn(730, dim, generator=torch.Generator().manual_seed(seed)).to("cuda:0") if waves else None

        greedy = {}                    # index of a timed greedy request -> its prompt ids

        def submit(i):
            if waves:
                ids = [rng.randrange(0, vocab) for _ in range(rng.randint(32, 128))]
                options = dict(temperature=1.0, top_p=1.0, seed=i) if i % 2 else {}
                if not options and i < 1000:
                    greedy[i] = ids
                return engine.submit_sync(ids, max_new_tokens=n_new, prefix_embeds=prefix, stop_ids=(), **options)
            ids = [rng.randrange(0, vocab) for _ in range(rng.randint(64, 1536))]
            if i < args.check:             # (to be compared with the plain implementation: these decode greedily)
                greedy[i] = ids
                return engine.submit_sync(ids, max_new_tokens=n_new, stop_ids=())
            return engine.submit_sync(ids, max_new_tokens=n_new, temperature=0.7, top_p=1.0, seed=i, stop_ids=())

        for future in [submit(1000 + i) for i in range(8 if waves else 4)]:      # warm-up: graphs, workspaces
            future.result()
        steps_before = engine.scheduler.steps
        started = time.perf_counter()
        futures = []
        for wave in range(4 if waves else 1):
            count = n_requests // 4 if waves else n_requests
            futures += [submit(wave * count + j) for j in range(count)]
            if waves:
                time.sleep(0.05)
        results = [f.result() for f in futures]
        elapsed = time.perf_counter() - started
        steps = engine.scheduler.steps - steps_before
        pages = engine.runner.cache.n_pages
        checked = check_greedy(args, sizes, folder, greedy, results, None if prefix is None else prefix.cpu())
    finally:
        engine.shutdown_sync()
        shutil.rmtree(folder, ignore_errors=True)
    generated = sum(len(r.tokens) for r in results)
    prompt = sum(r.metrics.input_tokens for r in results)
    what = ("256 requests in 4 waves, 730 given embeddings + 32-128 ids each, 128 new tokens, half greedy half T=1" if waves
            else "48 requests, prompts of 64-1536 ids in portions of at most 512 beside decodes, 128 new tokens at T=0.7")
    return {
        "metric": f"generated tok/s through the entry point ({LABELS[args.sizes][0]}; {what})",
        "value": round(generated / elapsed, 1), "unit": "tok/s", "n_gpus": 1, "steps": steps, "warmup": 8 if waves else 4,
        "ms_per_step": round(elapsed / max(steps, 1) * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": args.dtype,
        "data": "synthetic (seeded random token ids and prefix embeddings; a folder of random weights N(0,0.02) read by the loader)",
        "config": {"model": LABELS[args.sizes][1], "workload": args.workload, "n_layers": args.layers,
                   "n_layers_full": sizes["n_layers"], "dim": sizes["dim"], "ff_dim": sizes["ff_dim"],
                   "n_heads": sizes["n_heads"], "vocab_size": sizes["vocab_size"], "requests": n_requests,
                   "max_batch_size": cfg.max_batch_size, "max_num_batched_tokens": cfg.max_num_batched_tokens,
                   "kv_cache_pages": pages, "page_size": PAGE_SIZE, "parallelism": "single-gpu"},
        "seconds": round(elapsed, 3), "generated_tokens": generated, "prompt_tokens": prompt,
        "all_tokens_per_second": round((generated + prompt) / elapsed, 1),
        "finish_reasons": sorted({r.finish_reason for r in results}), "checked_against_plain": checked,
        "setup_seconds": {"write_folder": round(written, 1), "load": round(loaded, 1)},
    }


def main() -> int:
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=128)
    parser.add_argument("--warmup", type=int, default=8)
    parser.add_argument("--batch", type=int, default=8)
    parser.add_argument("--sizes", default="moondream2", choices=sorted(SIZES), help="layer sizes (the default is the benchmark's)")
    parser.add_argument("--layers", type=int, default=None, help="fewer layers than the model has (named in config)")
    parser.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    parser.add_argument("--context", type=int, default=CONTEXT, help="tokens each request holds when decoding starts")
    parser.add_argument("--prefill-tokens", type=int, default=PREFILL_TOKENS, help="length of the timed prompt")
    parser.add_argument("--skip-points", action="store_true", help="only the default batch (no batch 1 / 64, no prefill)")
    parser.add_argument("--only-prefill", action="store_true", help="only the 2,048-token prefill (for profiling)")
    parser.add_argument("--peaks", action=argparse.BooleanOptionalAction, default=True,
                        help="also measure a plain read stream and a loop of matrix instructions on this GPU and report "
                             "against them (about 0.1 s; --no-peaks leaves it out)")
    parser.add_argument("--tune-linears", type=int, default=0,
                        help="with --workload: RuntimeConfig.tune_linears (time the vendor library's algorithms at warm-up)")
    parser.add_argument("--check", type=int, default=0,
                        help="with --workload: compare this many greedy requests with the plain implementation (for --layers 2)")
    parser.add_argument("--workload", default="decode", choices=["decode", "waves256", "mixed48"],
                        help="decode: the benchmark's decode step (default); the others run requests through InferenceEngine")
    parser.add_argument("--max-batch-size", type=int, default=None, help="for the workloads through the entry point")
    parser.add_argument("--linears", default="library", choices=["library", "own"],
                        help="linears of more than 64 rows (a prompt's): through hipBLASLt (the engine's default) or "
                             "through this package's tiled kernels only")
    args = parser.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2
    import torch

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible")
        return 1
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    from kestrel_amd.ops import fast

    fast.LIBRARY_LINEAR = args.linears == "library"
    dtype = torch.bfloat16 if args.dtype == "bf16" else torch.float32
    size = 2 if dtype == torch.bfloat16 else 4
    sizes = dict(SIZES[args.sizes])
    # a longer context than the model's own is measured with its position table made longer
    sizes["max_context"] = max(sizes["max_context"], args.context + max(args.steps, 16) + args.warmup + 8, args.prefill_tokens)
    if args.layers is None:
        args.layers = sizes["n_layers"]
    if args.workload != "decode":
        print(json.dumps(run_workload(args, dict(SIZES[args.sizes]))))
        return 0
    net, typed = build_model(args.layers, dtype, device, sizes)
    weights = model_bytes(net, size)

    if args.only_prefill:
        seconds, best = time_prefill(net, typed, args.prefill_tokens)
        print(json.dumps({"prefill_ms": round(seconds * 1e3, 3), "best_ms": round(best * 1e3, 3), "tokens": args.prefill_tokens,
                          "dtype": args.dtype}))
        return 0
    elapsed, kv_bytes = time_decode(net, typed, args.batch, args.context, args.steps, args.warmup)
    ms_per_step = elapsed / args.steps * 1e3
    value = args.batch * args.steps / elapsed
    step_bytes = weights + kv_bytes * (size / 2) + args.batch * typed.dim * size
    achieved = step_bytes / (elapsed / args.steps)
    record = {
        "metric": f"decode tok/s ({LABELS[args.sizes][0]}, batch {args.batch}, context {args.context})",
        "value": round(value, 1),
        "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic (seeded random token ids and prefix embeddings, random weights N(0,0.02))",
        "config": {"model": LABELS[args.sizes][1], "n_layers": args.layers, "n_layers_full": sizes["n_layers"],
                   "dim": typed.dim, "ff_dim": typed.ff_dim, "n_heads": typed.n_heads, "n_kv_heads": typed.n_kv_heads,
                   "head_dim": typed.head_dim, "rotary_dim": typed.rotary_dim, "vocab_size": typed.vocab_size,
                   "global_batch": args.batch, "seq_len": args.context, "prefix_attn": typed.prefix_attn,
                   "page_size": PAGE_SIZE, "parallelism": "single-gpu",
                   "prompt_linears": "hipblaslt" if args.linears == "library" else "own"},
        "roofline": {"bound": "hbm", "achieved": round(achieved / 1e9, 1), "peak": PEAK_HBM / 1e9, "unit": "GB/s",
                     "frac": round(achieved / PEAK_HBM, 4)},
    }
    if not args.skip_points:
        seconds, best = time_prefill(net, typed, args.prefill_tokens)         # the median of eight runs, and the best
        flops = prefill_flops(typed, args.prefill_tokens, min(typed.prefix_attn, args.prefill_tokens - 1))
        record["prefill"] = {"value": round(args.prefill_tokens / seconds, 1), "tokens": args.prefill_tokens,
                             "ms": round(seconds * 1e3, 3), "frac": round(flops / seconds / PEAK_FLOPS[args.dtype], 4),
                             "best_ms": round(best * 1e3, 3)}
        points, detail = {}, {}
        for batch, steps in ((1, args.steps), (64, max(16, args.steps // 4))):
            e, kv = time_decode(net, typed, batch, args.context, steps, min(args.warmup, 4))
            points[f"decode_b{batch}"] = round(batch * steps / e, 1)
            moved = weights + kv * (size / 2) + batch * typed.dim * size
            detail[f"decode_b{batch}"] = {"ms_per_step": round(e / steps * 1e3, 4), "steps": steps,
                                          "frac": round(moved / (e / steps) / PEAK_HBM, 4)}
        record["points"] = points
        record["points_detail"] = detail
    if args.peaks:
        from kestrel_amd.ops import core

        peaks = core.measured_peaks(device)
        record["roofline"]["peak_measured"] = round(peaks["hbm_read_gbs"], 1)
        record["roofline"]["frac_measured"] = round(achieved / 1e9 / peaks["hbm_read_gbs"], 4)
        if "prefill" in record and args.dtype == "bf16":
            record["prefill"]["peak_measured"] = round(peaks["mfma_bf16_tflops"], 1)
            record["prefill"]["frac_measured"] = round(flops / seconds / 1e12 / peaks["mfma_bf16_tflops"], 4)
    print(json.dumps(record))
    return 0


if __name__ == "__main__":
    sys.exit(main())
