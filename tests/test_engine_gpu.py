"""The engine against the plain implementation under every way of cutting the work."""

import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from tests import helpers
from tests.helpers import Request
from tests.plain import moondream_plain as plain

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]
DTYPE_IDS = ["fp32", "bf16"]
NAMES = ["A", "B", "C", "D", "E", "F"]


def _runner(name, dtype, n_pages=64, page_size=16, max_requests=8, graphs=False):
    from kestrel_amd.engine.loading import load_model, make_runner

    net = load_model(helpers.model_dir(name), dtype, torch.device("cuda:0"))
    runner = make_runner(net, page_size, n_pages, max_requests, enable_graphs=graphs)
    helpers.poison_cache(runner)
    return runner


def _expected(name, req: Request):
    folder = helpers.model_dir(name)
    return plain.forward(helpers.flat_config(name), helpers.stored_weights(folder), req.ids, req.prefix)


def _request(name, tag, seed, n_ids, n_prefix=0):
    cfg = helpers.flat_config(name)
    prefix = None
    if n_prefix:
        gen = torch.Generator().manual_seed(1000 + seed)
        prefix = torch.randn(n_prefix, cfg["dim"], generator=gen)
    return Request(tag, helpers.random_ids(seed, n_ids, cfg["vocab_size"]), prefix)


def _check(name, dtype, requests, got):
    for tag, req in requests.items():
        helpers.assert_close(got[tag], _expected(name, req), dtype, f"tiny {name} request {tag}")


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("name", NAMES)
def test_whole_prompt(name, dtype):
    """Each request alone and whole, also the first tokens of a sequence (1, 2, 3 tokens)."""
    runner = _runner(name, dtype)
    for seed, length in enumerate([1, 2, 3, 5, 17, 33, 70, 100]):
        reqs = {"r": _request(name, "r", 100 + seed, length)}
        got = helpers.replay(runner, reqs, [[("r", length)]])
        _check(name, dtype, reqs, got)


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("name", NAMES)
def test_last_32_one_by_one(name, dtype):
    """Most of the request in one step, the last 32 tokens decoded one by one."""
    runner = _runner(name, dtype)
    for seed, length in enumerate([33, 64, 81, 120]):
        reqs = {"r": _request(name, "r", 200 + seed, length)}
        steps = ([[("r", length - 32)]] if length > 32 else []) + [[("r", 1)] for _ in range(32)]
        got = helpers.replay(runner, reqs, steps, poison=True)
        _check(name, dtype, reqs, got)


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("name", NAMES)
def test_portions_of_changing_size(name, dtype):
    """Portions cut anywhere, down to two tokens, over page edges (page size 16)."""
    runner = _runner(name, dtype)
    sizes = [7, 2, 9, 14, 2, 3, 16, 1, 31, 2, 33]
    length = sum(sizes)
    reqs = {"r": _request(name, "r", 300, length)}
    got = helpers.replay(runner, reqs, [[("r", s)] for s in sizes], poison=True)
    _check(name, dtype, reqs, got)


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("name", NAMES)
def test_mixed_batches_with_page_reuse(name, dtype):
    """Up to four live requests, portions of some beside decoded tokens of others, with so
    few pages that later requests run in pages earlier ones gave back."""
    lengths = {"a": 40, "b": 75, "c": 23, "d": 90, "e": 61, "f": 18, "g": 50}
    # 4 live requests of at most 90 tokens: 4 * 6 pages of 16; the pool has 18, so the order
    # below only works because pages come back and are used again.
    runner = _runner(name, dtype, n_pages=18, max_requests=4)
    reqs = {tag: _request(name, tag, 400 + i, n) for i, (tag, n) in enumerate(lengths.items())}
    steps = [
        [("a", 30), ("b", 20)],
        [("a", 1), ("b", 40), ("c", 2)],
        [("a", 1), ("b", 1), ("c", 21)],                      # c ends
        [("a", 8), ("b", 14), ("d", 50)],                     # a, b end
        [("d", 1), ("e", 33), ("f", 17)],
        [("d", 1), ("e", 1), ("f", 1), ("g", 2)],             # f ends
        [("d", 38), ("e", 27), ("g", 47)],                    # d, e end
        [("g", 1)],
    ]
    got = helpers.replay(runner, reqs, steps, poison=True)
    assert all(r.done == r.length for r in reqs.values())
    _check(name, dtype, reqs, got)
    assert runner.cache.groups[0].pool.free_count == 18


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("name", ["D", "F"])
@pytest.mark.parametrize("graphs", [False, True], ids=["eager", "graphs"])
def test_many_requests_decoded_together(name, dtype, graphs):
    """Short prompts fed together in one step, then decoded side by side, one token each a step: 12
    rows (the kernel that cuts K into parts takes the last linears from 9 rows on), 24 and 48 (a
    block's last launch also computes the next block's norm from 17 rows on; replayed in the buckets
    of 32 and 48 rows, with padding rows), 70 and 130 (more rows than the weight-streaming kernels take)."""
    for count in (12, 24, 48, 70, 130):
        runner = _runner(name, dtype, n_pages=2 * count + 8, max_requests=count, graphs=graphs)
        reqs = {f"r{i}": _request(name, f"r{i}", 900 + i, 6 + i % 9) for i in range(count)}
        steps = [[(tag, 3 + int(tag[1:]) % 4) for tag in reqs]]
        while True:
            fed = steps_fed(steps)
            rest = [(tag, 1) for tag, r in reqs.items() if fed.get(tag, 0) < r.length]
            if not rest:
                break
            steps.append(rest)
        got = helpers.replay(runner, reqs, steps)
        _check(name, dtype, reqs, got)


def steps_fed(steps):
    fed = {}
    for step in steps:
        for tag, count in step:
            fed[tag] = fed.get(tag, 0) + count
    return fed


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("name", ["B", "C", "D", "E", "F"])
def test_prefix_embeddings_bidirectional(name, dtype):
    """Given embeddings as one bidirectional block, then text; the block in one portion, the
    rest cut into portions and decoded; two such requests mixed."""
    cfg = helpers.flat_config(name)
    n_prefix = cfg["prefix_attn"]
    runner = _runner(name, dtype)
    reqs = {"p": _request(name, "p", 500, 29, n_prefix), "q": _request(name, "q", 501, 12, n_prefix)}
    steps = [[("p", n_prefix + 4)], [("p", 10), ("q", n_prefix)], [("p", 1), ("q", 5)], [("p", 14), ("q", 7)]]
    got = helpers.replay(runner, reqs, steps, poison=True)
    _check(name, dtype, reqs, got)


def test_split_bidirectional_block_is_refused():
    from kestrel_amd.engine.step import StepEntry

    runner = _runner("B", torch.float32)
    slot = runner.admit()
    embeds = torch.randn(8, helpers.flat_config("B")["dim"])
    with pytest.raises(ValueError, match="must lie inside one portion"):
        runner.step([StepEntry(slot, [-1] * 8, embeds=embeds, bidirectional=[(0, 17)])])


@pytest.mark.parametrize("graphs", [False, True], ids=["eager", "graphs"])
def test_an_odd_entry_is_refused_by_its_index_before_the_cache_is_touched(graphs):
    """No tokens at all, a token that is no integer, wanted places that repeat a row: each is named by
    ``StepRefused.entry_index`` (also where steps are replayed as graphs, whose bucket is looked for
    first), and the request beside it holds what it held."""
    from kestrel_amd.engine.step import StepEntry, StepRefused

    runner = _runner("A", torch.float32, graphs=graphs)
    good, odd = runner.admit(), runner.admit()
    runner.step([StepEntry(good, [5, 6, 7], want=[2]), StepEntry(odd, [9, 10], want=[1])])
    free = [g.pool.free_count for g in runner.cache.groups]
    for tokens, message in (([], "at least one token"), (["x"], "integers"), ([1.5], "integers")):
        with pytest.raises(StepRefused, match=message) as caught:
            runner.step([StepEntry(good, [8], want=[0]), StepEntry(odd, tokens, want=[0] if tokens else [])])
        assert caught.value.entry_index == 1
        assert runner.held == {good: 3, odd: 2} and [g.pool.free_count for g in runner.cache.groups] == free
    logits = runner.step([StepEntry(good, [8], want=[0]), StepEntry(odd, [11], want=[0])])
    assert logits.shape[0] == 2 and bool(torch.isfinite(logits).all())


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
def test_wanted_places_that_number_the_tokens_but_are_not_them(dtype):
    """A decode-only step of three rows that wants three rows of logits, but not one of each: the first
    row's twice, the second's not at all. The head's launch that normalises 'every row, in order'
    itself must not be taken for it."""
    from kestrel_amd.engine.step import StepEntry

    name = "D"
    runner = _runner(name, dtype)
    reqs = [_request(name, f"w{i}", 1700 + i, n) for i, n in enumerate((9, 21, 14))]
    slots = [runner.admit() for _ in reqs]
    runner.step([StepEntry(slot, req.ids[:-1]) for slot, req in zip(slots, reqs)])
    logits = runner.step([StepEntry(slots[0], req_last(reqs[0]), want=[0, 0]), StepEntry(slots[1], req_last(reqs[1])),
                          StepEntry(slots[2], req_last(reqs[2]), want=[0])]).clone()
    expected = [_expected(name, req)[-1] for req in reqs]
    for row, which in enumerate((0, 0, 2)):
        helpers.assert_close(logits[row], expected[which], dtype, f"row {row} of logits is request {which}'s")


def req_last(req: Request):
    return req.ids[-1:]


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("name", ["B", "D", "F"])
def test_long_decoding(name, dtype):
    """A short prompt, then every further token one by one up to the context length."""
    length = helpers.flat_config(name)["max_context"]
    runner = _runner(name, dtype)
    reqs = {"r": _request(name, "r", 600, length)}
    got = helpers.replay(runner, reqs, [[("r", 3)]] + [[("r", 1)] for _ in range(length - 3)])
    _check(name, dtype, reqs, got)


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
def test_a_context_of_thousands(dtype):
    """4,300 tokens: most in two portions, the rest one by one (the decode attention kernel cuts a
    row of more than 4096 keys into parts), beside a short request."""
    name = "G"
    runner = _runner(name, dtype, n_pages=300, max_requests=2)
    reqs = {"long": _request(name, "long", 950, 4300), "short": _request(name, "short", 951, 40)}
    steps = [[("long", 3000)], [("long", 1090), ("short", 30)]] + [[("long", 1), ("short", 1)] for _ in range(10)] \
        + [[("long", 1)] for _ in range(200)]
    got = helpers.replay(runner, reqs, steps)
    _check(name, dtype, reqs, got)


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("name", ["A", "D", "F"])
def test_replayed_graphs_match_the_plain_implementation(name, dtype):
    """Decode steps replayed as HIP graphs, compared logit by logit with the plain implementation:
    one, three and five live requests (buckets of 1, 4 and 8, the last two with padding rows), across
    page edges, with prompt steps (eager) between the replays, a request that ends and whose slot
    and pages another takes, and a return to a bucket captured earlier."""
    lengths = {"r0": 58, "r1": 41, "r2": 37, "r3": 50, "r4": 30, "r5": 44}
    runner = _runner(name, dtype, n_pages=20, max_requests=8, graphs=True)
    reqs = {tag: _request(name, tag, 1300 + i, n) for i, (tag, n) in enumerate(lengths.items())}
    steps = [[("r0", 13)]]
    steps += [[("r0", 1)]] * 5                                           # bucket 1, over the page edge at 16
    steps += [[("r1", 30), ("r0", 1)], [("r2", 9), ("r0", 1), ("r1", 1)]]         # eager: prompts beside decoded tokens
    steps += [[("r0", 1), ("r1", 1), ("r2", 1)]] * 6                     # bucket 4 with a padding row
    steps += [[("r3", 29), ("r4", 15)]]
    steps += [[("r0", 1), ("r1", 1), ("r2", 1), ("r3", 1), ("r4", 1)]] * 4        # bucket 8 with three padding rows; r1 ends
    steps += [[("r5", 17), ("r2", 1)]]                                   # r5 takes r1's slot and pages
    steps += [[("r4", 1), ("r5", 1), ("r0", 1), ("r2", 1), ("r3", 1)]] * 7        # bucket 8, other rows in other places
    steps += [[("r0", 1), ("r3", 1), ("r5", 1)]] * 4                     # back to bucket 4
    steps += [[("r0", 1)]] * 3                                           # and to bucket 1
    fed = steps_fed(steps)
    for tag, req in reqs.items():                                        # whatever is left, request by request (bucket 1)
        steps += [[(tag, 1)]] * (req.length - fed[tag])
    got = helpers.replay(runner, reqs, steps, poison=True)
    assert all(r.done == r.length for r in reqs.values())
    assert sorted(runner._graphs) == [1, 4, 8]
    assert runner.graph_replays == sum(1 for step in steps if all(count == 1 for _tag, count in step))
    _check(name, dtype, reqs, got)
    assert runner.cache.groups[0].pool.free_count == 20


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
def test_replayed_graphs_over_a_long_context(dtype):
    """A model whose context is longer than what one workgroup of the decode attention kernel takes
    (4096 keys): a captured step is cut for the longest context there can be, so every replay goes
    through the kernel that splits a row's keys and the one that merges the parts, with padding rows
    that have no keys at all. A request is decoded across the 4096-key edge beside shorter ones."""
    name = "G"
    runner = _runner(name, dtype, n_pages=290, max_requests=3, graphs=True)
    reqs = {"long": _request(name, "long", 1350, 4110), "mid": _request(name, "mid", 1351, 70),
            "short": _request(name, "short", 1352, 21)}
    steps = [[("long", 2500)], [("long", 1590), ("mid", 60)]]
    steps += [[("long", 1), ("mid", 1)]] * 10                            # bucket 2: 4090 .. 4099
    steps += [[("short", 12)]]
    steps += [[("short", 1), ("long", 1)]] * 9                           # bucket 2, other rows
    steps += [[("long", 1)]]                                             # bucket 1: the long one ends
    got = helpers.replay(runner, reqs, steps)
    assert sorted(runner._graphs) == [1, 2] and runner.graph_replays == 20
    _check(name, dtype, reqs, got)


@pytest.mark.parametrize("page_size", [1, 4, 64])
def test_other_page_sizes(page_size):
    runner = _runner("A", torch.float32, n_pages=512 // page_size, page_size=page_size)
    reqs = {"r": _request("A", "r", 700, 77)}
    got = helpers.replay(runner, reqs, [[("r", 40)], [("r", 5)]] + [[("r", 1)] for _ in range(32)])
    _check("A", torch.float32, reqs, got)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(tmp_path, dtype):
    """bin/trace_run as a user runs it: JSON lines in, <step>.f32 files and 'done' lines out."""
    name = "A"
    cfg = helpers.flat_config(name)
    ids_a = helpers.random_ids(800, 50, cfg["vocab_size"])
    ids_b = helpers.random_ids(801, 37, cfg["vocab_size"])
    lines = [
        {"step": 0, "entries": [{"id": "a", "tokens": ids_a[:18], "want": [0, 17]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": ids_a[18:48], "want": []},
                                {"id": "b", "tokens": ids_b[:2], "want": [1]}], "end": []},
        {"step": 2, "entries": [{"id": "b", "tokens": ids_b[2:37], "want": [34]}], "end": ["b"]},
        {"step": 3, "entries": [{"id": "a", "tokens": ids_a[48:49], "want": []}], "end": []},
        {"step": 4, "entries": [{"id": "a", "tokens": ids_a[49:50], "want": [0]}], "end": ["a"]},
    ]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = tmp_path / "out"
    done = subprocess.run(
        [sys.executable, os.path.join(root, "bin", "trace_run"), "--model", helpers.model_dir(name), "--dtype", dtype,
         "--out", str(out), "--max-tokens", "128"],
        input="\n".join(json.dumps(l) for l in lines) + "\n", capture_output=True, text=True, timeout=300)
    assert done.returncode == 0, done.stderr
    assert [l for l in done.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(5)]
    assert sorted(f.name for f in out.iterdir()) == ["0.f32", "1.f32", "2.f32", "4.f32"]     # step 3 wanted nothing
    weights = helpers.stored_weights(helpers.model_dir(name))
    exp_a = plain.forward(cfg, weights, ids_a)
    exp_b = plain.forward(cfg, weights, ids_b)
    tdtype = torch.float32 if dtype == "float32" else torch.bfloat16

    def load(step, rows):
        data = np.fromfile(out / f"{step}.f32", dtype="<f4")
        return torch.from_numpy(data.reshape(rows, cfg["vocab_size"]))

    helpers.assert_close(load(0, 2), exp_a[[0, 17]], tdtype, "step 0")
    helpers.assert_close(load(1, 1), exp_b[[1]], tdtype, "step 1")
    helpers.assert_close(load(2, 1), exp_b[[36]], tdtype, "step 2")
    helpers.assert_close(load(4, 1), exp_a[[49]], tdtype, "step 4")


def _random_configuration(rng):
    """A small configuration drawn at random: head sizes in steps of 16 (in steps of 32 above 128),
    grouped heads, widths and vocabularies that are no power of two, every rotary width."""
    while True:
        hd = rng.choice([16, 32, 48, 64, 80, 96, 112, 128, 160, 192, 256])
        hkv = rng.choice([1, 2, 3])
        heads = hkv * rng.choice([1, 2, 3])
        if heads * hd <= 640:
            break
    explicit = rng.random() < 0.5
    cfg = {"dim": rng.choice([40, 72, 100, 136, 200, 264]) if explicit else heads * hd,
           "ff_dim": rng.choice([24, 56, 136, 200, 320]), "n_layers": rng.choice([1, 2, 3]),
           "vocab_size": rng.choice([97, 300, 777, 1000]), "max_context": 512, "n_heads": heads, "n_kv_heads": hkv,
           "rope_theta": rng.choice([100.0, 5000.0, 10000.0, 1.5e6]), "prefix_attn": 0,
           "layer_norm_eps": rng.choice([1e-5, 1e-6, 3e-4])}
    if explicit:
        cfg["head_dim"] = hd
    rotary = rng.choice([None, None, hd, 2, max(hd // 2 - 2, 2), 0])
    if rotary is not None:
        cfg["rotary_dim"] = rotary - rotary % 2
    return cfg


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("seed", range(8))
def test_configurations_drawn_at_random(seed, dtype, tmp_path):
    """Six requests of a random configuration, up to four live, cut at random into portions and
    single tokens, some with a block of given embeddings, in a pool that makes pages come back."""
    import random

    from kestrel_amd.engine.loading import load_model, make_runner
    from kestrel_amd.weights import InitRecipe, write_random_model

    rng = random.Random(1000 + seed)
    cfg = _random_configuration(rng)
    folder = str(tmp_path / "model")
    write_random_model(folder, {"text": cfg}, seed, InitRecipe(std=0.04, bias_std=0.04, gain_std=0.1, shift_std=0.05))
    weights = helpers.stored_weights(folder)
    net = load_model(folder, dtype, torch.device("cuda:0"))
    lengths = [rng.choice([3, 17, 33, 64, 65, 130, 257]) for _ in range(6)]
    pages = sum(sorted(-(-n // 16) for n in lengths)[-4:]) + 2
    runner = make_runner(net, 16, pages, 4)
    helpers.poison_cache(runner)
    reqs = {}
    for i, n in enumerate(lengths):
        n_prefix = rng.choice([0, 0, 5, 17]) if n > 20 else 0
        prefix = torch.randn(n_prefix, cfg["dim"], generator=torch.Generator().manual_seed(seed * 100 + i)) if n_prefix else None
        reqs[f"r{i}"] = Request(f"r{i}", helpers.random_ids(seed * 10 + i, n - n_prefix, cfg["vocab_size"]), prefix)
    waiting, live, steps, fed = list(reqs), [], [], {tag: 0 for tag in reqs}
    while waiting or live:
        while waiting and len(live) < 4 and (not live or rng.random() < 0.7):
            live.append(waiting.pop(0))
        step = []
        for tag in list(live):
            if rng.random() < 0.2 and len(live) > 1:
                continue                                   # left out of this step
            req = reqs[tag]
            count = rng.choice([1, 1, 2, 3, 7, 16, 31, 64, 100, 1000])
            if fed[tag] == 0 and req.n_prefix:
                count = max(count, req.n_prefix)
            count = min(count, req.length - fed[tag])
            fed[tag] += count
            step.append((tag, count))
            if fed[tag] == req.length:
                live.remove(tag)
        if step:
            steps.append(step)
    got = helpers.replay(runner, reqs, steps, poison=True)
    for tag, req in reqs.items():
        helpers.assert_close(got[tag], plain.forward(cfg, weights, req.ids, req.prefix), dtype, f"{cfg} request {tag}")
