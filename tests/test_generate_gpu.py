"""Generation through the Python entry point and the command line."""

import asyncio
import json
import os
import subprocess
import sys

import pytest
import torch

from tests import helpers
from tests.plain import moondream_plain as plain

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _engine(name, dtype, **kw):
    from kestrel_amd import InferenceEngine, RuntimeConfig

    options = dict(model_path=helpers.model_dir(name), dtype=dtype, max_batch_size=4, kv_cache_pages=40,
                   max_num_batched_tokens=48)
    options.update(kw)
    return InferenceEngine.create_sync(RuntimeConfig(**options))


def _assert_greedy(result_tokens, expected, margins, slack, what):
    """For a path that must agree token by token (float32, where ``slack`` is far below any margin
    the tests' prompts have)."""
    assert len(result_tokens) == len(expected), what
    for i, (got, want) in enumerate(zip(result_tokens, expected)):
        assert got == want or margins[i] < slack, \
            f"{what}: token {i} is {got}, the plain implementation gives {want} (margin {margins[i]:.3g})"
        if got != want:
            return


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "D"])
def test_greedy_generation_matches_the_plain_implementation(name, dtype):
    """Requests of different lengths submitted together: prompts are cut into portions of 48
    tokens beside the decoding of the others; with and without HIP graphs, with every step read
    before the next and with two steps in flight."""
    cfg = helpers.flat_config(name)
    weights = helpers.stored_weights(helpers.model_dir(name))
    prompts = [helpers.random_ids(900 + i, n, cfg["vocab_size"]) for i, n in enumerate([5, 17, 33, 70])]
    n_new = 16
    slack = 1e-4 if dtype == "float32" else 5e-2
    for graphs, depth in ((False, 1), (True, 2), (False, 2)):
        engine = _engine(name, dtype, enable_graphs=graphs, pipeline_depth=depth)
        try:
            results = engine.generate_batch_sync(prompts, max_new_tokens=n_new, temperature=0.0, stop_ids=())
            replays = engine.runner.graph_replays
        finally:
            engine.shutdown_sync()
        assert (replays > 0) == graphs
        for prompt, result in zip(prompts, results):
            assert result.finish_reason == "length" and result.metrics.output_tokens == n_new
            assert len(result.tokens) == n_new
            helpers.assert_greedy_follows(cfg, weights, prompt, result.tokens, slack,
                                          f"tiny {name} {dtype} graphs={graphs} depth={depth}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_generation_after_a_prefix_block(dtype):
    """A block of given embeddings (one BOS id + rows) that sees itself both ways, then text."""
    name = "B"
    cfg = helpers.flat_config(name)
    weights = helpers.stored_weights(helpers.model_dir(name))
    gen = torch.Generator().manual_seed(5)
    rows = torch.randn(cfg["prefix_attn"] - 1, cfg["dim"], generator=gen)
    ids = helpers.random_ids(950, 11, cfg["vocab_size"])
    bos = weights["text.wte"][0].double().unsqueeze(0)
    prefix = torch.cat([bos, rows.double()])
    engine = _engine(name, dtype)
    try:
        result = engine.generate_sync(ids, max_new_tokens=12, prefix_embeds=rows, prefix_ids=[0], stop_ids=())
    finally:
        engine.shutdown_sync()
    assert len(result.tokens) == 12
    helpers.assert_greedy_follows(cfg, weights, ids, result.tokens, 1e-4 if dtype == "float32" else 5e-2,
                                  f"prefix {dtype}", prefix_embeds=prefix)


def test_sampling_is_reproducible_and_independent_of_the_batch():
    cfg = helpers.flat_config("A")
    prompts = [helpers.random_ids(960 + i, 9 + 3 * i, cfg["vocab_size"]) for i in range(4)]
    engine = _engine("A", "float32", seed=11)
    try:
        alone = engine.generate_sync(prompts[2], max_new_tokens=12, temperature=0.8, top_p=0.9, seed=77, stop_ids=())
        futures = [engine.submit_sync(p, max_new_tokens=12, temperature=0.8 if i == 2 else 1.3, top_p=0.9,
                                      seed=77 if i == 2 else i, stop_ids=()) for i, p in enumerate(prompts)]
        mixed = [f.result() for f in futures]
        again = engine.generate_sync(prompts[2], max_new_tokens=12, temperature=0.8, top_p=0.9, seed=78, stop_ids=())
    finally:
        engine.shutdown_sync()
    assert alone.tokens == mixed[2].tokens              # same seed: same tokens, whatever else is in the batch
    assert alone.tokens != again.tokens                 # another seed: another draw
    assert all(0 <= t < cfg["vocab_size"] for r in mixed for t in r.tokens)


@pytest.mark.parametrize("depth,graphs", [(1, False), (2, True)])
def test_sampled_generation_in_portions_beside_decodes_follows_the_plain_model(depth, graphs):
    """Four requests, each a block of 17 positions (one id and 16 given embeddings, which see each
    other both ways) and 3 to 40 ids, 24 tokens each at temperature 0.8 with a seed, under a token
    budget of 24: the block goes in whole, the rest of a prompt in portions beside the decoded tokens
    of the others. (A budget of 8 cannot hold the block, which may not be split; 24 is the nearest
    that does.) Every token must be the one that the request's uniform number for that index picks,
    by inversion in index order, from the plain implementation's softmax(logits / 0.8) after the
    same earlier tokens."""
    from kestrel_amd.ops import core
    from kestrel_amd.sampling import mix_key

    name, temperature, n_new, engine_seed = "B", 0.8, 24, 11
    cfg = helpers.flat_config(name)
    weights = helpers.stored_weights(helpers.model_dir(name))
    bos = weights["text.wte"][0].double().unsqueeze(0)
    requests = []
    for i, n_ids in enumerate((3, 40, 11, 26)):
        rows = torch.randn(cfg["prefix_attn"] - 1, cfg["dim"], generator=torch.Generator().manual_seed(40 + i))
        requests.append((rows, helpers.random_ids(1230 + i, n_ids, cfg["vocab_size"]), 500 + i))
    engine = _engine(name, "float32", max_num_batched_tokens=24, seed=engine_seed, pipeline_depth=depth,
                     enable_graphs=graphs)
    try:
        futures = [engine.submit_sync(ids, max_new_tokens=n_new, temperature=temperature, top_p=1.0, seed=seed,
                                      prefix_embeds=rows, prefix_ids=[0], stop_ids=()) for rows, ids, seed in requests]
        results = [f.result(timeout=120) for f in futures]
        steps = engine.scheduler.steps
    finally:
        engine.shutdown_sync()
    assert steps < 4 * n_new, "the requests were decoded side by side"
    for (rows, ids, seed), result in zip(requests, results):
        assert len(result.tokens) == n_new and result.finish_reason == "length"
        prefix = torch.cat([bos, rows.double()])
        logits = plain.forward(cfg, weights, ids + result.tokens[:-1], prefix)
        first = prefix.shape[0] + len(ids) - 1
        for i, token in enumerate(result.tokens):
            cdf = torch.cumsum(plain.nucleus_probs(logits[first + i], temperature, 1.0), dim=0)
            u = core.uniform(mix_key(engine_seed, seed), i)
            want = int(torch.searchsorted(cdf, torch.tensor(u, dtype=torch.float64), right=True))
            assert token == want or abs(float(cdf[token] - cdf[want])) < 1e-4, \
                f"request with seed {seed}, token {i}: {token}, the plain distribution and u = {u:.6f} give {want}"


@pytest.mark.parametrize("depth", [1, 2])
def test_masks_and_logprobs_through_the_entry_point(depth):
    """Greedy generation with the chosen tokens' log-probabilities, a token that may not come
    first, tokens that may never come and an allow-list, against the plain implementation."""
    name = "A"
    cfg = helpers.flat_config(name)
    weights = helpers.stored_weights(helpers.model_dir(name))
    prompt = helpers.random_ids(975, 11, cfg["vocab_size"])
    tokens, margins = plain.greedy_generate(cfg, weights, prompt, 6)
    engine = _engine(name, "float32", pipeline_depth=depth)
    try:
        scored = engine.generate_sync(prompt, max_new_tokens=6, stop_ids=(), return_logprobs=True)
        barred = engine.generate_sync(prompt, max_new_tokens=3, stop_ids=(), suppress_next_token_ids=[tokens[0]],
                                      return_logprobs=True, temperature=0.7, top_p=1.0, seed=3)
        never = engine.generate_sync(prompt, max_new_tokens=6, stop_ids=(), suppressed_token_ids=tokens[:2])
        only = engine.generate_sync(prompt, max_new_tokens=6, stop_ids=(), allowed_token_ids=[3, 5, 8])
    finally:
        engine.shutdown_sync()
    _assert_greedy(scored.tokens, tokens, margins, 1e-4, "with log-probabilities")
    assert scored.logprobs == [0.0] * len(scored.tokens)            # greedy: the argmax has log-probability 0
    assert barred.tokens[0] != tokens[0]
    # its first token's score under softmax(logits / 0.7) with the barred token at -inf
    logits = plain.forward(cfg, weights, prompt)[-1].clone()
    logits[tokens[0]] = float("-inf")
    expected = torch.log_softmax(logits.double() / 0.7, dim=-1)[barred.tokens[0]]
    assert abs(barred.logprobs[0] - float(expected)) < 1e-3
    assert len(barred.logprobs) == 3 and all(lp <= 0.0 for lp in barred.logprobs)
    assert not set(never.tokens) & set(tokens[:2])
    assert set(only.tokens) <= {3, 5, 8} and only.logprobs is None


def test_stop_ids_max_tokens_and_errors():
    cfg = helpers.flat_config("A")
    weights = helpers.stored_weights(helpers.model_dir("A"))
    prompt = helpers.random_ids(970, 12, cfg["vocab_size"])
    tokens, _ = plain.greedy_generate(cfg, weights, prompt, 8)
    engine = _engine("A", "float32")
    try:
        stopped = engine.generate_sync(prompt, max_new_tokens=8, stop_ids=[tokens[3]])
        first = tokens.index(tokens[3])
        assert stopped.finish_reason == "stop" and stopped.tokens == tokens[:first + 1]
        with pytest.raises(ValueError):
            engine.generate_sync(prompt, max_new_tokens=0)
        with pytest.raises(ValueError):
            engine.generate_sync(prompt, max_new_tokens=4, temperature=-1.0)
        with pytest.raises(ValueError):
            engine.generate_sync([cfg["vocab_size"] + 5] * 200, max_new_tokens=4)      # longer than the context
        # the engine is still alive after refusing requests
        assert engine.generate_sync(prompt, max_new_tokens=2, stop_ids=()).tokens == tokens[:2]
    finally:
        engine.shutdown_sync()


@pytest.mark.parametrize("dtype,depth,graphs", [("float32", 1, False), ("bfloat16", 2, True)])
def test_bad_requests_fail_alone_and_the_engine_goes_on(dtype, depth, graphs):
    """Good and bad requests submitted together: an id beyond the vocabulary, an id of -1 with no
    embedding behind it, the id that stands for "the pending token" inside the engine, embeddings
    one column too wide. Each bad one raises for its caller only; the good ones give the plain
    implementation's tokens; the engine serves a further request and every page and slot is back."""
    name = "D"
    cfg = helpers.flat_config(name)
    weights = helpers.stored_weights(helpers.model_dir(name))
    vocab, dim = cfg["vocab_size"], cfg["dim"]
    good = [helpers.random_ids(1200 + i, n, vocab) for i, n in enumerate((21, 9, 30))]
    slack = 1e-4 if dtype == "float32" else 5e-2
    engine = _engine(name, dtype, pipeline_depth=depth, enable_graphs=graphs)
    try:
        futures = [
            engine.submit_sync(good[0], max_new_tokens=8, stop_ids=()),
            engine.submit_sync(good[1][:4] + [vocab] + good[1][4:], max_new_tokens=8, stop_ids=()),
            engine.submit_sync(good[1][:4] + [-1] + good[1][4:], max_new_tokens=8, stop_ids=()),
            engine.submit_sync([-2] + good[1], max_new_tokens=8, stop_ids=()),
            engine.submit_sync(good[1], max_new_tokens=8, stop_ids=(), prefix_embeds=torch.zeros(5, dim + 1),
                               prefix_ids=[0]),
            engine.submit_sync(good[1], max_new_tokens=8, stop_ids=()),
        ]
        for bad in futures[1:5]:
            with pytest.raises(ValueError):
                bad.result(timeout=60)
        for prompt, future in ((good[0], futures[0]), (good[1], futures[5])):
            result = future.result(timeout=60)
            assert len(result.tokens) == 8 and result.finish_reason == "length"
            helpers.assert_greedy_follows(cfg, weights, prompt, result.tokens, slack, f"beside bad requests, {dtype}")
        later = engine.generate_sync(good[2], max_new_tokens=6, stop_ids=())
        helpers.assert_greedy_follows(cfg, weights, good[2], later.tokens, slack, f"after bad requests, {dtype}")
        assert engine._fatal is None
    finally:
        engine.shutdown_sync()
    cache = engine.runner.cache
    cache.check()
    assert cache.free_slots == cache.max_requests and not engine.runner.held
    assert all(g.pool.free_count == g.pool.n_pages and g.pool.promised_unheld == 0 for g in cache.groups)


@pytest.mark.parametrize("depth", [1, 2])
def test_an_entry_the_step_function_refuses_fails_alone(depth):
    """A request that got past the door (put into the queue by hand) with an id the step function
    refuses: ``ModelRunner.step`` names the entry before it touches the cache, the scheduler fails
    that request and runs the others of the step again without it."""
    from kestrel_amd.engine.types import GenerationRequest, Sequence_

    name = "A"
    cfg = helpers.flat_config(name)
    weights = helpers.stored_weights(helpers.model_dir(name))
    prompts = [helpers.random_ids(1210 + i, n, cfg["vocab_size"]) for i, n in enumerate((13, 40, 7))]
    engine = _engine(name, "float32", pipeline_depth=depth)
    try:
        sched, runner = engine.scheduler, engine.runner
        engine.shutdown_sync()                      # the thread has ended: the scheduler is driven by hand
        sched.enqueue_request(GenerationRequest(0, prompts[0], 6, stop_ids=()))
        sched.advance()
        sched.waiting.append(Sequence_(GenerationRequest(1, prompts[1][:20] + [cfg["vocab_size"] + 3] + prompts[1][20:],
                                                         6, stop_ids=())))
        sched.enqueue_request(GenerationRequest(2, prompts[2], 6, stop_ids=()))
        results = {r.request_id: r for r in sched.run_until_done()}
    finally:
        engine.shutdown_sync()
    assert results[1].finish_reason == "error" and "outside the vocabulary" in results[1].error
    assert sched.failed_steps == 1
    for i in (0, 2):
        expected, margins = plain.greedy_generate(cfg, weights, prompts[i], 6)
        _assert_greedy(results[i].tokens, expected, margins, 1e-4, f"request {i} beside a refused entry")
    runner.cache.check()
    assert runner.cache.free_slots == runner.cache.max_requests and not runner.held
    assert all(g.pool.free_count == g.pool.n_pages and g.pool.promised_unheld == 0 for g in runner.cache.groups)


@pytest.mark.parametrize("temperature", [0.0, 0.9])
def test_a_request_resumed_with_its_generated_tokens_goes_on_as_before(temperature):
    """``_generated_prefix`` (``kestrel/engine/core.py:556-597``): tokens generated before are fed
    after the prompt, count against ``max_tokens`` and head the result. The draw of a token is keyed
    by its index in the request, so a resumed request continues exactly as the unbroken one did."""
    cfg = helpers.flat_config("B")
    prompt = helpers.random_ids(1220, 23, cfg["vocab_size"])
    engine = _engine("B", "float32")
    try:
        whole = engine.generate_sync(prompt, max_new_tokens=10, temperature=temperature, top_p=0.95, seed=5, stop_ids=(),
                                     return_logprobs=True)

        async def resume():
            return await engine.generate(prompt, stop_ids=(), seed=5, settings={
                "temperature": temperature, "top_p": 0.95, "max_tokens": 10, "_logprobs": True,
                "_generated_prefix": {"tokens": whole.tokens[:4], "logprobs": whole.logprobs[:4]}})

        resumed = asyncio.run(resume())
        with pytest.raises(ValueError, match="leaves nothing to generate"):
            engine.generate_sync(prompt, max_new_tokens=4, generated_prefix={"tokens": whole.tokens[:4]})
        with pytest.raises(TypeError, match="takes the keys"):
            engine.generate_sync(prompt, max_new_tokens=8, generated_prefix={"tokens": [1], "scores": [0.0]})
    finally:
        engine.shutdown_sync()
    assert resumed.tokens == whole.tokens and resumed.finish_reason == "length"
    assert resumed.metrics.output_tokens == 6 and resumed.metrics.input_tokens == len(prompt)
    assert resumed.logprobs[:4] == whole.logprobs[:4]
    assert max(abs(a - b) for a, b in zip(resumed.logprobs, whole.logprobs)) < 1e-4


def test_a_request_too_large_for_the_cache_fails_alone():
    cfg = helpers.flat_config("B")
    engine = _engine("B", "float32", kv_cache_pages=4)            # 64 tokens in all
    try:
        big = engine.submit_sync(helpers.random_ids(980, 60, cfg["vocab_size"]), max_new_tokens=30)
        small = engine.submit_sync(helpers.random_ids(981, 10, cfg["vocab_size"]), max_new_tokens=4, stop_ids=())
        assert len(small.result().tokens) == 4
        with pytest.raises(RuntimeError, match="Insufficient KV cache capacity"):
            big.result()
    finally:
        engine.shutdown_sync()


def test_pause_leaves_nothing_in_flight_and_resume_goes_on():
    """``pause`` / ``resume`` (``kestrel/engine/core.py:810-836``): after ``pause`` returns no step is in
    flight and no token arrives, requests keep what they hold, a request submitted meanwhile waits; after
    ``resume`` all of them end with the tokens an undisturbed run gives."""
    import queue
    import time

    cfg = helpers.flat_config("B")
    prompts = [helpers.random_ids(1240 + i, n, cfg["vocab_size"]) for i, n in enumerate([21, 9])]
    late = helpers.random_ids(1243, 12, cfg["vocab_size"])
    options = dict(max_new_tokens=200, temperature=0.8, top_p=0.9, seed=11, stop_ids=())
    engine = _engine("B", "float32", pipeline_depth=2, kv_cache_pages=60)
    try:
        undisturbed = [r.tokens for r in engine.generate_batch_sync(prompts + [late], **options)]
        stream: "queue.Queue" = queue.Queue()
        futures = [engine.submit_sync(prompts[0], _stream=stream, **options), engine.submit_sync(prompts[1], **options)]
        stream.get(timeout=60)                                    # decoding is under way
        assert engine.pause(timeout=60)
        assert len(engine.scheduler._inflight) == 0
        while not stream.empty():
            stream.get_nowait()
        done_before = [f.done() for f in futures]          # (a slow host may let them end before the pause is asked for)
        futures.append(engine.submit_sync(late, **options))
        time.sleep(0.3)
        assert stream.empty() and [f.done() for f in futures[:2]] == done_before and not futures[2].done()
        if not all(done_before):
            held = [g.pool.n_pages - g.pool.free_count for g in engine.runner.cache.groups]
            assert all(n > 0 for n in held)
        engine.resume()
        assert [f.result(timeout=120).tokens for f in futures] == undisturbed
        assert engine.pause(timeout=60)                           # an idle engine pauses too, and shuts down paused
    finally:
        engine.shutdown_sync()


def test_async_entry_point_and_streaming():
    from kestrel_amd import InferenceEngine, RuntimeConfig

    cfg = helpers.flat_config("A")
    prompt = helpers.random_ids(990, 10, cfg["vocab_size"])

    async def run():
        engine = await InferenceEngine.create(RuntimeConfig(model_path=helpers.model_dir("A"), dtype="float32",
                                                            kv_cache_pages=16))
        try:
            whole = await engine.generate(prompt, settings={"temperature": 0.0, "max_tokens": 6}, stop_ids=())
            seen = []
            async for update in engine.submit_streaming(prompt, max_new_tokens=6, stop_ids=()):
                seen.append((update.token_index, update.token))
            both = await asyncio.gather(engine.submit(prompt, max_new_tokens=3, stop_ids=()),
                                        engine.submit(prompt[:5], max_new_tokens=3, stop_ids=()))
        finally:
            await engine.shutdown()
        return whole, seen, both

    whole, seen, both = asyncio.run(run())
    assert len(whole.tokens) == 6 and whole.metrics.input_tokens == 10 and whole.metrics.ttft_ms > 0
    assert seen == list(enumerate(whole.tokens))
    assert both[0].tokens == whole.tokens[:3]


def test_command_line(tmp_path):
    env = dict(os.environ, PYTHONPATH=ROOT)
    config = tmp_path / "cfg.json"
    config.write_text(json.dumps(helpers.TINY_A))
    made = subprocess.run([sys.executable, "-m", "kestrel_amd", "random-weights", "--out", str(tmp_path / "m"),
                           "--config", str(config), "--seed", "0"], capture_output=True, text=True, env=env, cwd=ROOT)
    assert made.returncode == 0, made.stderr
    assert (tmp_path / "m" / "config.json").exists() and (tmp_path / "m" / "model.safetensors").exists()
    cfg = helpers.flat_config("A")
    prompt = helpers.random_ids(995, 7, cfg["vocab_size"])
    done = subprocess.run([sys.executable, "-m", "kestrel_amd", "generate", "--model-path", str(tmp_path / "m"),
                           "--dtype", "float32", "--prompt-ids", ",".join(map(str, prompt)), "--max-tokens", "5",
                           "--temperature", "0", "--kv-cache-pages", "8"], capture_output=True, text=True, env=env,
                          cwd=ROOT, timeout=300)
    assert done.returncode == 0, done.stderr
    record = json.loads(done.stdout.strip().splitlines()[-1])
    # the folder written by the command line holds the same weights as the test's (same seed and recipe)
    tokens, margins = plain.greedy_generate(cfg, helpers.stored_weights(helpers.model_dir("A")), prompt, 5)
    stop = cfg.get("eos_id", 0)
    expected = tokens[:tokens.index(stop) + 1] if stop in tokens else tokens
    _assert_greedy(record["tokens"], expected, margins, 1e-4, "command line")


def test_profile_decode_command(tmp_path):
    """The decode timing command with the reference script's options: one PROFILE line."""
    env = dict(os.environ, PYTHONPATH=ROOT)
    done = subprocess.run([sys.executable, "-m", "kestrel_amd", "profile-decode", "--weights", helpers.model_dir("D"),
                           "--batch-size", "3", "--prompt-len", "20", "--warmup", "2", "--decode-iters", "6",
                           "--profile-iters", "4"], capture_output=True, text=True, env=env, cwd=ROOT, timeout=300)
    assert done.returncode == 0, done.stderr
    line = [l for l in done.stdout.splitlines() if l.startswith("PROFILE:")]
    assert len(line) == 1 and "batch=3, prompt_len=20, profile_iters=4, avg_ms=" in line[0]
    too_long = subprocess.run([sys.executable, "-m", "kestrel_amd", "profile-decode", "--weights", helpers.model_dir("D"),
                               "--prompt-len", "250", "--decode-iters", "50"], capture_output=True, text=True, env=env,
                              cwd=ROOT, timeout=300)
    assert too_long.returncode == 2 and "exceed the model's context" in too_long.stderr


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_everything_is_made_at_start(dtype, caplog):
    """With ``warmup`` (the default) the graph of every bucket of decode rows exists before the first
    request, and a mixed run (prompts cut into portions beside decoded tokens, requests of many lengths,
    sampling with and without temperature) allocates no device memory between its first request's
    end and its last; the logger says what was made, and names a request that is refused."""
    import logging

    from kestrel_amd.engine.step import graph_buckets

    name = "D"
    cfg = helpers.flat_config(name)
    with caplog.at_level(logging.INFO, logger="kestrel_amd"):
        engine = _engine(name, dtype, max_batch_size=6, kv_cache_pages=60, max_num_batched_tokens=64)
    try:
        runner = engine.runner
        assert sorted(runner._graphs) == graph_buckets(6) == [1, 2, 4, 6]
        assert all(state.graph is not None for state in runner._graphs.values())
        assert sorted(runner._mixed) == [(16, 6), (32, 6), (64, 6)]         # steps of any shape, up to the token limit of 64
        assert all(state.graph is not None for state in runner._mixed.values())
        assert not runner.held and runner.cache.free_slots == runner.cache.max_requests
        first = engine.generate_sync(helpers.random_ids(1800, 9, cfg["vocab_size"]), max_new_tokens=4, stop_ids=())
        assert len(first.tokens) == 4
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated()
        prompts = [helpers.random_ids(1801 + i, n, cfg["vocab_size"]) for i, n in enumerate((3, 70, 150, 31, 64, 5, 97, 200, 12))]
        futures = [engine.submit_sync(p, max_new_tokens=5 + 3 * (i % 4), temperature=0.0 if i % 2 else 0.8, top_p=0.9,
                                      seed=i, stop_ids=()) for i, p in enumerate(prompts)]
        results = [f.result(timeout=120) for f in futures]
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == before, "a step of the mixed run allocated device memory"
        assert all(r.finish_reason == "length" for r in results)
        with caplog.at_level(logging.WARNING, logger="kestrel_amd"):
            with pytest.raises(ValueError, match="outside the vocabulary"):
                engine.generate_sync([1, cfg["vocab_size"] + 5], max_new_tokens=2)
    finally:
        engine.shutdown_sync()
    text = caplog.text
    assert "warm-up: 4 decode graphs and 3 graphs of other steps captured" in text and "cache pool: 60 pages" in text and "loaded" in text
    assert "refused at the door" in text and "outside the vocabulary" in text


def test_without_warmup_nothing_is_captured_before_it_is_needed():
    engine = _engine("A", "bfloat16", warmup=False)
    try:
        assert not engine.runner._graphs
        engine.generate_sync([1, 2, 3], max_new_tokens=3, stop_ids=())
        assert sorted(engine.runner._graphs) == [1]
    finally:
        engine.shutdown_sync()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_prompt_with_two_blocks_of_given_embeddings(dtype):
    """Text, a block of given rows, text, another block, text: the positions of each block see each other
    both ways and everything else is causal (``kestrel/models/moondream/text.py:146-157``). The step budget
    of 16 tokens cuts the prompt of 31 into portions that keep each block whole; a second request decodes
    beside them. Every generated token must be the plain implementation's choice."""
    name = "B"
    cfg = helpers.flat_config(name)
    weights = helpers.stored_weights(helpers.model_dir(name))
    gen = torch.Generator().manual_seed(77)
    pieces = [helpers.random_ids(1900, 4, cfg["vocab_size"]), torch.randn(7, cfg["dim"], generator=gen),
              helpers.random_ids(1901, 9, cfg["vocab_size"]), torch.randn(5, cfg["dim"], generator=gen),
              helpers.random_ids(1902, 6, cfg["vocab_size"])]
    ids, rows, blocks, block_of, embedded = [], [], [], [], []
    table = weights["text.wte"].double()
    for piece in pieces:
        if isinstance(piece, torch.Tensor):
            blocks.append((len(ids), len(ids) + piece.shape[0]))
            block_of += [len(blocks) - 1] * piece.shape[0]
            ids += [-1] * piece.shape[0]
            rows.append(piece)
            embedded.append(piece.double())
        else:
            block_of += [-1] * len(piece)
            ids += piece
            embedded.append(table[piece])
    assert blocks == [(4, 11), (20, 25)]
    other = helpers.random_ids(1903, 12, cfg["vocab_size"])
    engine = _engine(name, dtype, max_num_batched_tokens=16)
    try:
        beside = engine.submit_sync(other, max_new_tokens=10, stop_ids=())
        result = engine.generate_sync(ids, max_new_tokens=8, prompt_embeds=torch.cat(rows), blocks=blocks, stop_ids=())
        beside = beside.result(timeout=60)
    finally:
        engine.shutdown_sync()
    slack = 1e-4 if dtype == "float32" else 5e-2
    tokens = result.tokens
    assert len(tokens) == 8
    logits = plain.forward(cfg, weights, tokens[:-1], prefix_embeds=torch.cat(embedded),
                           block_ids=block_of + [-1] * (len(tokens) - 1))
    for i, token in enumerate(tokens):
        row = logits[len(ids) - 1 + i]
        gap = float(row.max() - row[token])
        assert gap <= slack, f"token {i} is {token}, the plain implementation gives {int(row.argmax())} ({gap:.3g} better)"
    # the blocks matter: read causally, the same prompt leads elsewhere
    causal = plain.forward(cfg, weights, [], prefix_embeds=torch.cat(embedded), block_ids=[-1] * len(ids))[-1]
    assert float((causal - logits[len(ids) - 1]).abs().max()) > 1e-3
    helpers.assert_greedy_follows(cfg, weights, other, beside.tokens, slack, f"beside the blocks, {dtype}")


def test_linears_tuned_at_warm_up_give_the_same_tokens():
    """``tune_linears``: the warm-up's prompts time the vendor library's algorithms for every bucket of rows and keep
    the fastest. Whatever it picks, generation stays the plain implementation's (prompts long enough for their
    linears to go through the library: more than 64 rows)."""
    from kestrel_amd.ops import fast

    name = "D"
    cfg = helpers.flat_config(name)
    weights = helpers.stored_weights(helpers.model_dir(name))
    before = fast.library_stats()
    engine = _engine(name, "bfloat16", max_num_batched_tokens=192, kv_cache_pages=64, tune_linears=2)
    try:
        after = fast.library_stats()
        assert after["tuned"] > before["tuned"], (before, after)
        prompts = [helpers.random_ids(2000 + i, n, cfg["vocab_size"]) for i, n in enumerate((150, 70, 9))]
        results = engine.generate_batch_sync(prompts, max_new_tokens=8, stop_ids=())
        assert fast.library_stats()["tuned"] == after["tuned"], "nothing is timed once the warm-up is over"
    finally:
        engine.shutdown_sync()
    for prompt, result in zip(prompts, results):
        helpers.assert_greedy_follows(cfg, weights, prompt, result.tokens, 5e-2, "tuned linears")


@pytest.mark.parametrize("name,dtype", [("D", "bfloat16"), ("B", "float32")])
def test_a_random_stream_of_requests_leaves_nothing_behind(name, dtype):
    """Sixty requests in bursts, drawn at random: prompts of 1 to 150 ids (some behind a block of given
    embeddings), 1 to 20 new tokens, stop ids that occur or do not, greedy or sampled, in a pool so small
    that requests wait for pages, with a token budget of 32 so that prompts go in portions beside the
    decoded tokens of others; every step is a replayed graph. The greedy ones are the plain
    implementation's tokens as far as they go; a stop id ends a request where it first occurs; at the
    end every page and every slot is back."""
    import random
    import time

    cfg = helpers.flat_config(name)
    weights = helpers.stored_weights(helpers.model_dir(name))
    rng = random.Random(2024)
    n_prefix = cfg["prefix_attn"]
    engine = _engine(name, dtype, max_batch_size=4, kv_cache_pages=26, max_num_batched_tokens=32, enable_graphs=True,
                     pipeline_depth=2)
    slack = 1e-4 if dtype == "float32" else 5e-2
    submitted = []
    try:
        for burst in range(4):
            for _ in range(15):
                ids = helpers.random_ids(rng.randrange(10 ** 6), rng.randint(1, 150), cfg["vocab_size"])
                rows = None
                if n_prefix and n_prefix <= 32 and rng.random() < 0.3:
                    rows = torch.randn(n_prefix, cfg["dim"], generator=torch.Generator().manual_seed(rng.randrange(10 ** 6)))
                greedy = rng.random() < 0.6
                stops = tuple(rng.randrange(cfg["vocab_size"]) for _ in range(rng.choice((0, 0, 3, 40))))
                options = dict(max_new_tokens=rng.randint(1, 20), stop_ids=stops)
                if not greedy:
                    options.update(temperature=rng.choice((0.7, 1.3)), top_p=rng.choice((1.0, 0.8)), seed=rng.randrange(1000))
                if rows is not None:
                    options.update(prefix_embeds=rows)
                submitted.append((ids, rows, greedy, stops, options["max_new_tokens"], engine.submit_sync(ids, **options)))
            time.sleep(0.02 * burst)
        results = [entry[-1].result(timeout=180) for entry in submitted]
        runner = engine.runner
        assert runner.mixed_graph_replays > 0 and runner.graph_replays > 0
        assert not runner.held and runner.cache.free_slots == runner.cache.max_requests
        assert all(g.pool.free_count == runner.cache.n_pages for g in runner.cache.groups)
        runner.cache.check()
    finally:
        engine.shutdown_sync()
    checked = 0
    for (ids, rows, greedy, stops, n_new, _future), result in zip(submitted, results):
        assert result.finish_reason in ("stop", "length"), result.finish_reason
        tokens = list(result.tokens)
        assert 1 <= len(tokens) <= n_new and all(0 <= t < cfg["vocab_size"] for t in tokens)
        assert not any(t in stops for t in tokens[:-1]), "a stop id ends the request where it first occurs"
        if result.finish_reason == "stop":
            assert tokens[-1] in stops
        else:
            assert len(tokens) == n_new and tokens[-1] not in stops
        if greedy and checked < 12:
            helpers.assert_greedy_follows(cfg, weights, ids, tokens, slack, f"a random stream, tiny {name} {dtype}",
                                          prefix_embeds=rows)
            checked += 1
    assert checked == 12


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_whole_architecture_registered_in_a_test(dtype, tmp_path, request):
    """Another architecture, made up here and registered under a name of its own: configuration keys of its
    own, blocks that run mixer and feed-forward one after the other from two norms without shifts, attention
    without biases over grouped kv heads with every channel rotated, a ReLU feed-forward, a final norm, a head
    tied to an embedding table that is scaled on the way in, capped logits, and a schedule that runs its middle
    layer twice (each run with a cache of its own). Nothing of the package is edited: the registry, the
    random-weights writer, the loader, the cache manager, the scheduler and the entry point take it from its
    ``config.json``; greedy generation, with graphs and prompts cut into portions, follows a plain computation
    written here."""
    from dataclasses import dataclass

    from kestrel_amd import InferenceEngine, RuntimeConfig
    from kestrel_amd.config.registry import ModelSpec, register
    from kestrel_amd.parts.specs import (AttentionSpec, DenseFeedForwardSpec, LayerSpec, ModelPlan, NormSpec, PositionSpec,
                                         ScheduleEntry)
    from kestrel_amd.weights import InitRecipe, write_random_model

    @dataclass(frozen=True)
    class StackConfig:
        width: int
        depth: int
        heads: int
        kv_heads: int
        head: int
        inner: int
        vocab: int
        positions: int
        theta: float
        eps: float
        cap: float

    def read_config(config):
        keys = ("width", "depth", "heads", "kv_heads", "head", "inner", "vocab", "positions", "theta", "eps", "cap")
        missing = [k for k in keys if k not in config]
        if missing:
            raise ValueError(f"config.json: keys missing: {missing}")
        return StackConfig(**{k: config[k] for k in keys})

    def build_plan(cfg):
        position = PositionSpec("rotary_neox", cfg.head, cfg.theta, cfg.positions)
        layers = []
        for i in range(cfg.depth):
            p = f"stack.{i}."
            layers.append(LayerSpec(
                arrangement="sequential", norm=NormSpec("layernorm", cfg.width, cfg.eps, bias=False),
                norm2=NormSpec("layernorm", cfg.width, cfg.eps, bias=False),
                mixer=AttentionSpec("attention", cfg.width, cfg.heads, cfg.kv_heads, cfg.head, position, bias=False),
                feed_forward=DenseFeedForwardSpec("dense", cfg.width, cfg.inner, "relu", bias=False),
                names={"norm.weight": p + "n1", "norm2.weight": p + "n2", "mixer.qkv.weight": p + "qkv", "mixer.proj.weight": p + "o",
                       "feed_forward.fc1.weight": p + "up", "feed_forward.fc2.weight": p + "down"}))
        order = [0] + [i for i in range(1, cfg.depth - 1) for _ in range(2)] + [cfg.depth - 1]
        return ModelPlan(architecture="toy_stack", vocab_size=cfg.vocab, dim=cfg.width, max_positions=cfg.positions,
                         layers=tuple(layers), schedule=tuple(ScheduleEntry(i) for i in order),
                         final_norm=NormSpec("layernorm", cfg.width, cfg.eps, bias=False), head_bias=False, tied_head=True,
                         names={"embedding": "table", "final_norm.weight": "last_norm"}, eos_token_ids=(1,),
                         embedding_scale=float(cfg.width) ** 0.5, logit_softcap=cfg.cap)

    from kestrel_amd.config import registry

    register(ModelSpec(name="toy_stack", read_config=read_config, build_plan=build_plan))
    request.addfinalizer(lambda: registry._REGISTRY.pop("toy_stack", None))       # (other tests list the registered names)
    config = {"model": "toy_stack", "width": 96, "depth": 3, "heads": 6, "kv_heads": 2, "head": 16, "inner": 136, "vocab": 257,
              "positions": 160, "theta": 777.0, "eps": 1e-4, "cap": 12.0}
    folder = str(tmp_path / "toy_stack")
    write_random_model(folder, config, seed=9, recipe=InitRecipe(std=0.08, gain_std=0.1))
    weights = {k: v.double() for k, v in helpers.stored_weights(folder).items()}
    assert sorted(weights)[:3] == ["last_norm", "stack.0.down", "stack.0.n1"] and "table" in weights

    def logits_of(ids):
        cfg = read_config(config)
        n = len(ids)
        x = weights["table"][torch.tensor(ids)] * cfg.width ** 0.5
        positions = torch.arange(n)
        allowed = plain.visibility(positions, None)
        table = plain.rotary_table(cfg.head, n, cfg.theta)
        zero = torch.zeros(cfg.width, dtype=torch.float64)
        for i in (0, 1, 1, 2):
            p = f"stack.{i}."
            h = plain.layer_norm(x, weights[p + "n1"], zero, cfg.eps)
            q, k, v = plain.linear(h, weights[p + "qkv"], None).split([cfg.heads * cfg.head, cfg.kv_heads * cfg.head, cfg.kv_heads * cfg.head], dim=-1)
            q = plain.apply_rotary(q.reshape(n, cfg.heads, cfg.head), positions, table)
            k = plain.apply_rotary(k.reshape(n, cfg.kv_heads, cfg.head), positions, table)
            mixed = plain.attention_core(q, k, v.reshape(n, cfg.kv_heads, cfg.head), allowed, cfg.head ** -0.5)
            x = x + plain.linear(mixed.reshape(n, -1), weights[p + "o"], None)
            h = plain.layer_norm(x, weights[p + "n2"], zero, cfg.eps)
            x = x + plain.linear(torch.relu(plain.linear(h, weights[p + "up"], None)), weights[p + "down"], None)
        out = plain.linear(plain.layer_norm(x, weights["last_norm"], zero, cfg.eps), weights["table"], None)
        return cfg.cap * torch.tanh(out / cfg.cap)

    engine = InferenceEngine.create_sync(RuntimeConfig(model_path=folder, dtype=dtype, max_batch_size=3, kv_cache_pages=40,
                                                       max_num_batched_tokens=32))
    try:
        assert engine.runner.model.plan.architecture == "toy_stack" and len(engine.runner.layer_caches) == 4
        prompts = [helpers.random_ids(2100 + i, n, 257) for i, n in enumerate((7, 45, 70))]
        results = engine.generate_batch_sync(prompts, max_new_tokens=10, stop_ids=())
        assert engine.runner.mixed_graph_replays > 0 and engine.runner.graph_replays > 0
    finally:
        engine.shutdown_sync()
    slack = 1e-4 if dtype == "float32" else 5e-2
    for prompt, result in zip(prompts, results):
        tokens = list(result.tokens)
        assert len(tokens) == 10
        rows = logits_of(prompt + tokens[:-1])
        for i, token in enumerate(tokens):
            row = rows[len(prompt) - 1 + i]
            gap = float(row.max() - row[token])
            assert gap <= slack, f"toy_stack {dtype}: token {i} is {token}, the plain computation gives {int(row.argmax())} ({gap:.3g} better)"
