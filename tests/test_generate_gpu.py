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
    for i, (got, want) in enumerate(zip(result_tokens, expected)):
        if got != want:
            assert margins[i] < slack, f"{what}: token {i} is {got}, the plain implementation gives {want} (margin {margins[i]:.3g})"
            return                                       # a near tie: later tokens follow another path
    assert len(result_tokens) == len(expected)


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
    expected = [plain.greedy_generate(cfg, weights, p, n_new) for p in prompts]
    slack = 1e-4 if dtype == "float32" else 5e-2
    for graphs, depth in ((False, 1), (True, 2), (False, 2)):
        engine = _engine(name, dtype, enable_graphs=graphs, pipeline_depth=depth)
        try:
            results = engine.generate_batch_sync(prompts, max_new_tokens=n_new, temperature=0.0, stop_ids=())
            replays = engine.runner.graph_replays
        finally:
            engine.shutdown_sync()
        assert (replays > 0) == graphs
        for result, (tokens, margins) in zip(results, expected):
            assert result.finish_reason == "length" and result.metrics.output_tokens == n_new
            _assert_greedy(result.tokens, tokens, margins, slack, f"tiny {name} {dtype} graphs={graphs} depth={depth}")


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
    tokens, margins = plain.greedy_generate(cfg, weights, ids, 12, prefix_embeds=prefix)
    engine = _engine(name, dtype)
    try:
        result = engine.generate_sync(ids, max_new_tokens=12, prefix_embeds=rows, prefix_ids=[0], stop_ids=())
    finally:
        engine.shutdown_sync()
    _assert_greedy(result.tokens, tokens, margins, 1e-4 if dtype == "float32" else 5e-2, f"prefix {dtype}")


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
