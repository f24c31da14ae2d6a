"""Command line: ``python -m kestrel_amd <generate | random-weights | replay | profile-decode>``.

Option names follow the reference's ``RuntimeConfig`` fields (``kestrel/config.py:155-179``:
``--model-path --dtype --max-batch-size --page-size --kv-cache-pages``) and its request
settings (``temperature``, ``top_p``, ``max_tokens``; ``kestrel/engine/core.py:1161-1174``).
Prompts are token ids: the tokenizer is outside this engine. ``profile-decode`` takes the options
of the reference's decode profiling script (``scripts/profile_decode.py:243-256``).
"""

from __future__ import annotations

import argparse
import json
import sys
import time
from typing import List


def _add_runtime_options(parser: argparse.ArgumentParser) -> None:
    parser.add_argument("--model-path", required=True, help="folder with config.json and model.safetensors (or a .pt checkpoint)")
    parser.add_argument("--model", default=None, help="architecture name (default: taken from config.json)")
    parser.add_argument("--device", default="cuda")
    parser.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    parser.add_argument("--max-batch-size", type=int, default=4)
    parser.add_argument("--page-size", type=int, default=16)
    parser.add_argument("--kv-cache-pages", type=int, default=None)
    parser.add_argument("--kv-cache-bytes", type=int, default=None, help="size the cache pool by a byte budget instead")
    parser.add_argument("--max-num-batched-tokens", type=int, default=2048)
    parser.add_argument("--seed", type=int, default=0)
    parser.add_argument("--disable-graphs", action="store_true", help="do not replay steps as HIP graphs")
    parser.add_argument("--pipeline-depth", type=int, default=2, choices=(1, 2),
                        help="2: launch a step before the previous step's tokens have reached the host")
    parser.add_argument("--no-warmup", action="store_true",
                        help="do not capture the graphs and make scratch memory and plans at start")
    parser.add_argument("--tune-linears", type=int, default=0,
                        help="at warm-up, time the vendor library's algorithms for the prompt's linears (this many products "
                             "each) once per bucket of rows and keep the fastest; 0: the first the library names")
    parser.add_argument("--log-level", default="WARNING", choices=["DEBUG", "INFO", "WARNING", "ERROR"],
                        help="what the engine's logger reports on stderr (INFO: load, pool size, warm-up)")


def _parse_ids(text: str) -> List[int]:
    return [int(t) for t in text.replace(",", " ").split()]


def _generate(args) -> int:
    import logging

    import torch

    from .config import RuntimeConfig
    from .engine import InferenceEngine

    logging.basicConfig(level=getattr(logging, args.log_level), format="%(asctime)s %(name)s %(levelname)s %(message)s")
    prompts: List[List[int]] = []
    for text in args.prompt_ids or []:
        prompts.append(_parse_ids(text))
    if args.prompt_file:
        with open(args.prompt_file) as handle:
            data = json.load(handle)
        prompts.extend([list(map(int, p)) for p in data])
    cfg = RuntimeConfig(model_path=args.model_path, model=args.model, device=args.device, dtype=args.dtype,
                        max_batch_size=args.max_batch_size, page_size=args.page_size,
                        kv_cache_pages=args.kv_cache_pages, kv_cache_bytes=args.kv_cache_bytes,
                        max_num_batched_tokens=args.max_num_batched_tokens,
                        seed=args.seed, enable_graphs=not args.disable_graphs, pipeline_depth=args.pipeline_depth,
                        warmup=not args.no_warmup, tune_linears=args.tune_linears)
    engine = InferenceEngine.create_sync(cfg)
    try:
        if args.random_prompts:
            gen = torch.Generator().manual_seed(args.seed)
            vocab = engine.plan.vocab_size
            prompts.extend(torch.randint(0, vocab, (args.prompt_len,), generator=gen).tolist()
                           for _ in range(args.random_prompts))
        if not prompts:
            print("generate: give --prompt-ids, --prompt-file or --random-prompts", file=sys.stderr)
            return 2
        started = time.perf_counter()
        results = engine.generate_batch_sync(prompts, max_new_tokens=args.max_tokens, temperature=args.temperature,
                                             top_p=args.top_p, return_logprobs=args.logprobs,
                                             suppressed_token_ids=_parse_ids(args.suppress_ids or ""))
        elapsed = time.perf_counter() - started
        for result in results:
            record = {"request_id": result.request_id, "tokens": result.tokens,
                      "finish_reason": result.finish_reason, "input_tokens": result.metrics.input_tokens,
                      "output_tokens": result.metrics.output_tokens, "ttft_ms": round(result.metrics.ttft_ms, 3),
                      "decode_time_ms": round(result.metrics.decode_time_ms, 3)}
            if result.logprobs is not None:
                record["logprobs"] = [round(lp, 6) for lp in result.logprobs]
            print(json.dumps(record))
        total = sum(r.metrics.output_tokens for r in results)
        print(f"# {len(results)} requests, {total} tokens in {elapsed:.3f} s", file=sys.stderr)
    finally:
        engine.shutdown_sync()
    return 0


def _random_weights(args) -> int:
    from .config import get_spec
    from .weights import InitRecipe, write_random_model

    if args.config:
        with open(args.config) as handle:
            config = json.load(handle)
    else:
        spec = get_spec(args.preset)
        if spec.default_config is None:
            print(f"random-weights: {args.preset} has no preset configuration; give --config", file=sys.stderr)
            return 2
        config = dict(spec.default_config())
        config.setdefault("model", spec.name)
    recipe = InitRecipe(std=args.std, bias_std=args.bias_std, gain_std=args.gain_std, shift_std=args.shift_std)
    folder = write_random_model(args.out, config, args.seed, recipe, store_dtype=args.store_dtype, model=args.model)
    print(folder)
    return 0


def _profile_decode(args) -> int:
    """Steady-state decode steps of one batch, timed one by one: what the reference's
    ``scripts/profile_decode.py`` measures (``:309-470``: a batch of equal prompts is fed, the
    decode step is warmed up, the last ``--profile-iters`` of ``--decode-iters`` steps are timed
    with events and summarised in one ``PROFILE:`` line)."""
    import torch

    from .config.runtime import parse_dtype
    from .engine.loading import load_model, make_runner
    from .engine.step import PENDING_TOKEN, StepEntry
    from .sampling import Sampler

    device = torch.device(args.device)
    if device.index is None:
        device = torch.device("cuda", torch.cuda.current_device())
    print(f"Loading model from {args.weights}...")
    net = load_model(args.weights, parse_dtype(args.dtype), device)
    plan = net.plan
    print(f"Model loaded. Config: {len(plan.layers)} layers, hidden={plan.dim}")
    total = max(1, args.decode_iters)
    profiled = max(1, min(args.profile_iters, total))
    batch, prompt_len = args.batch_size, max(1, args.prompt_len)
    if prompt_len + args.warmup + total + 1 > plan.max_positions:
        print(f"profile-decode: {prompt_len} + {args.warmup + total} tokens exceed the model's context of "
              f"{plan.max_positions}", file=sys.stderr)
        return 2
    pages = -(-(prompt_len + args.warmup + total + 1) // args.page_size)
    runner = make_runner(net, args.page_size, batch * pages, batch, max_tokens_per_step=max(4096, prompt_len),
                         enable_graphs=True)
    sampler = Sampler(device, pending=runner.pending)
    # the prompt: the first token id of the model, then ids counting up (taken into the vocabulary)
    prompt = [plan.bos_token_id] + [(100 + i) % plan.vocab_size for i in range(prompt_len - 1)]
    slots = []
    for _ in range(batch):
        slot = runner.admit()
        logits = runner.step([StepEntry(slot, prompt, want=[prompt_len - 1])])
        sampler.greedy(logits, slots=[slot])
        slots.append(slot)

    def run_decode():
        logits = runner.step([StepEntry(slot, [PENDING_TOKEN], want=[0]) for slot in slots])
        sampler.greedy(logits, slots=runner.logit_slots)

    print(f"Running {args.warmup} warmup decode iterations...")
    for _ in range(args.warmup):
        run_decode()
    torch.cuda.synchronize(device)
    print(f"Running profiled decode iterations (HIP graph replay)... total={total}, profiled={profiled}")
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(profiled)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(profiled)]
    at = 0
    for i in range(total):
        timed = i >= total - profiled
        if timed:
            starts[at].record()
        run_decode()
        if timed:
            ends[at].record()
            at += 1
    torch.cuda.synchronize(device)
    times = sorted(a.elapsed_time(b) for a, b in zip(starts, ends))
    avg = sum(times) / len(times)
    p50, p90 = times[len(times) // 2], times[max(0, int(0.9 * (len(times) - 1)))]
    print(f"PROFILE: batch={batch}, prompt_len={prompt_len}, profile_iters={profiled}, avg_ms={avg:.3f}, "
          f"p50_ms={p50:.3f}, p90_ms={p90:.3f}, min_ms={times[0]:.3f}, max_ms={times[-1]:.3f}")
    return 0


def main(argv=None) -> int:
    parser = argparse.ArgumentParser(prog="kestrel_amd", description="MI355X inference engine")
    sub = parser.add_subparsers(dest="command", required=True)

    gen = sub.add_parser("generate", help="generate tokens for prompts given as token ids")
    _add_runtime_options(gen)
    gen.add_argument("--prompt-ids", action="append", help="token ids of one prompt, e.g. '5,17,3' (repeatable)")
    gen.add_argument("--prompt-file", help="JSON file with a list of prompts, each a list of token ids")
    gen.add_argument("--random-prompts", type=int, default=0, help="this many random prompts")
    gen.add_argument("--prompt-len", type=int, default=32, help="length of the random prompts")
    gen.add_argument("--logprobs", action="store_true", help="also print the log-probability of every generated token")
    gen.add_argument("--suppress-ids", help="token ids that must never be generated, e.g. '0,50256'")
    gen.add_argument("--max-tokens", type=int, default=16, help="tokens to generate per prompt")
    gen.add_argument("--temperature", type=float, default=0.0)
    gen.add_argument("--top-p", type=float, default=1.0)
    gen.set_defaults(run=_generate)

    rw = sub.add_parser("random-weights", help="write a model folder with seeded random weights")
    rw.add_argument("--out", required=True)
    rw.add_argument("--config", help="config.json to build the model from")
    rw.add_argument("--preset", default="moondream2", help="registered model whose preset sizes are used without --config")
    rw.add_argument("--model", default=None)
    rw.add_argument("--seed", type=int, default=0)
    rw.add_argument("--std", type=float, default=0.02)
    rw.add_argument("--bias-std", type=float, default=None)
    rw.add_argument("--gain-std", type=float, default=0.0)
    rw.add_argument("--shift-std", type=float, default=0.0)
    rw.add_argument("--store-dtype", default="bfloat16", choices=["bfloat16", "float32"])
    rw.set_defaults(run=_random_weights)

    pd = sub.add_parser("profile-decode", help="time steady-state decode steps of one batch")
    pd.add_argument("--weights", required=True, help="folder with config.json and model.safetensors")
    pd.add_argument("--batch-size", type=int, default=33, help="decode batch size")
    pd.add_argument("--prompt-len", type=int, default=740, help="prompt length (prefill tokens)")
    pd.add_argument("--warmup", type=int, default=5, help="warmup decode iterations")
    pd.add_argument("--decode-iters", type=int, default=50, help="total decode iterations")
    pd.add_argument("--profile-iters", type=int, default=20, help="steady-state decode iterations that are timed (the last N)")
    pd.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    pd.add_argument("--page-size", type=int, default=16)
    pd.add_argument("--device", default="cuda")
    pd.set_defaults(run=_profile_decode)

    rp = sub.add_parser("replay", help="trace replay (the same program as bin/trace_run)", add_help=False)
    rp.set_defaults(run=None)

    if argv is None:
        argv = sys.argv[1:]
    if argv and argv[0] == "replay":
        from .engine.replay import main as replay_main
        return replay_main(argv[1:])
    args = parser.parse_args(argv)
    return args.run(args)


if __name__ == "__main__":
    sys.exit(main())
