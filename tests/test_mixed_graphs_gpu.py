"""Steps of any shape (prompt portions, alone or beside decoded tokens) replayed as HIP graphs,
against the plain implementation and against the same steps launched kernel by kernel."""

from typing import Dict, List

import pytest
import torch

from tests import helpers
from tests.helpers import Request
from tests.plain import moondream_plain as plain

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]
DTYPE_IDS = ["fp32", "bf16"]


def _runner(name, dtype, n_pages=64, max_requests=8, graphs=True, max_tokens_per_step=4096):
    from kestrel_amd.engine.loading import load_model, make_runner

    net = load_model(helpers.model_dir(name), dtype, torch.device("cuda:0"))
    runner = make_runner(net, 16, n_pages, max_requests, enable_graphs=graphs, max_tokens_per_step=max_tokens_per_step)
    helpers.poison_cache(runner)
    return runner


def _request(name, tag, seed, n_ids, n_prefix=0):
    cfg = helpers.flat_config(name)
    prefix = None
    if n_prefix:
        prefix = torch.randn(n_prefix, cfg["dim"], generator=torch.Generator().manual_seed(1000 + seed))
    return Request(tag, helpers.random_ids(seed, n_ids, cfg["vocab_size"]), prefix)


def replay_last_places(runner, requests: Dict[str, Request], steps, wanted=1, poison=True):
    """Run ``steps`` = lists of (request name, number of tokens); of every portion only the last
    ``wanted`` places are wanted (as a scheduler asks). Returns per request ``{position: logits}``."""
    from kestrel_amd.engine.step import StepEntry

    rows: Dict[str, Dict[int, torch.Tensor]] = {name: {} for name in requests}
    for step in steps:
        entries, order = [], []
        for name, count in step:
            req = requests[name]
            if req.slot is None:
                req.slot = runner.admit()
            tokens, embeds, bidir, lo = req.take(count)
            want = list(range(max(0, len(tokens) - wanted), len(tokens)))
            entries.append(StepEntry(req.slot, tokens, want=want, embeds=None if embeds is None else embeds.to("cuda:0"),
                                     bidirectional=bidir))
            order.append((name, [lo + w for w in want]))
        logits = runner.step(entries).clone()
        at = 0
        for name, places in order:
            for place in places:
                rows[name][place] = logits[at]
                at += 1
        assert at == logits.shape[0]
        for name, _ in order:
            req = requests[name]
            if req.done == req.length:
                pages = [[p for p in runner.cache.block_table(g, req.slot) if p >= 0] for g in range(len(runner.cache.groups))]
                runner.release(req.slot)
                req.slot = None
                if poison:
                    for g, group in enumerate(runner.cache.groups):
                        if pages[g]:
                            for tensor in group.tensors.values():
                                tensor[:, torch.tensor(pages[g], device=tensor.device)] = float("nan")
        runner.cache.check()
    return rows


def _check(name, dtype, requests, got):
    folder = helpers.model_dir(name)
    cfg, weights = helpers.flat_config(name), helpers.stored_weights(folder)
    for tag, req in requests.items():
        expected = plain.forward(cfg, weights, req.ids, req.prefix)
        places = sorted(got[tag])
        assert places, f"request {tag} has no logits"
        helpers.assert_close(torch.stack([got[tag][p] for p in places]), expected[places], dtype, f"tiny {name} request {tag}")


def _mixed_steps():
    lengths = {"a": 40, "b": 75, "c": 23, "d": 90, "e": 61, "f": 18, "g": 50}
    steps = [
        [("a", 30), ("b", 20)],                               # 50 tokens: the bucket of 64
        [("a", 1), ("b", 40), ("c", 2)],                      # a decoded token beside two portions
        [("a", 1), ("b", 1), ("c", 21)],                      # c ends; 23 tokens: the bucket of 32
        [("a", 1), ("b", 1)],                                 # a decode step between (its own graph)
        [("a", 7), ("b", 13), ("d", 50)],                     # a, b end; 70 tokens: the bucket of 128
        [("d", 1), ("e", 33), ("f", 17)],
        [("d", 1), ("e", 1), ("f", 1), ("g", 2)],             # f ends; 5 tokens: the bucket of 16
        [("d", 38), ("e", 27), ("g", 47)],                    # d, e end; 112 tokens
        [("g", 1)],
    ]
    return lengths, steps


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("name", ["A", "C", "D", "F"])
def test_replayed_steps_of_any_shape_match_the_plain_implementation(name, dtype):
    """Up to four live requests, portions of some beside decoded tokens of others, in pages that
    earlier requests gave back (and that hold NaN since): every step is a replay, of the decode graphs
    or of the graph of its bucket of tokens, several of them more than once with other steps between."""
    lengths, steps = _mixed_steps()
    runner = _runner(name, dtype, n_pages=18, max_requests=4)
    assert runner.mixed_graphs
    reqs = {tag: _request(name, tag, 400 + i, n) for i, (tag, n) in enumerate(lengths.items())}
    got = replay_last_places(runner, reqs, steps, wanted=1)
    assert all(r.done == r.length for r in reqs.values())
    decode_steps = sum(1 for step in steps if all(count == 1 for _tag, count in step))
    assert runner.graph_replays == decode_steps and runner.mixed_graph_replays == len(steps) - decode_steps
    assert sorted(runner._mixed) == [(16, 4), (32, 4), (64, 4), (128, 4)]
    # the graphs run one after the other and share their scratch tensors
    assert all(state.workspace is runner._mixed_workspace for state in runner._mixed.values())
    _check(name, dtype, reqs, got)
    assert runner.cache.groups[0].pool.free_count == 18


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("name", ["B", "E"])
def test_replayed_steps_with_given_embeddings(name, dtype):
    """Blocks of given embeddings (bidirectional) at the front of two requests, fed through replayed
    steps, the second while the first decodes; then a request without any, through the same graph."""
    n_prefix = helpers.flat_config(name)["prefix_attn"]
    runner = _runner(name, dtype)
    reqs = {"p": _request(name, "p", 500, 29, n_prefix), "q": _request(name, "q", 501, 12, n_prefix),
            "t": _request(name, "t", 502, n_prefix + 9)}
    steps = [[("p", n_prefix + 4)], [("p", 10), ("q", n_prefix)], [("p", 1), ("q", 5)], [("p", 14), ("q", 7)],
             [("t", n_prefix + 4)], [("t", 5)]]
    got = replay_last_places(runner, reqs, steps, wanted=2)
    assert runner.mixed_graph_replays == len(steps)
    _check(name, dtype, reqs, got)


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
def test_replayed_and_launched_steps_agree(dtype):
    """The same steps through a runner that replays and one that launches kernel by kernel: the same
    kernels run on the same rows (the buckets of tokens here all take the kernels of few rows, which
    treat every row alike), so the logits agree closely; wanted places in the middle of a portion."""
    from kestrel_amd.engine.step import StepEntry

    name = "D"
    results = []
    for graphs in (True, False):
        runner = _runner(name, dtype, graphs=graphs)
        reqs = [_request(name, f"r{i}", 700 + i, 44) for i in range(3)]
        slots = [runner.admit() for _ in reqs]
        out = []
        for lo, hi in ((0, 20), (20, 23), (23, 44)):
            entries = [StepEntry(slot, req.ids[lo:hi], want=[0, (hi - lo) // 2]) for slot, req in zip(slots, reqs)]
            out.append(runner.step(entries).clone())
        assert (runner.mixed_graph_replays == 3) == graphs
        results.append(torch.cat(out))
    tol = 2e-5 if dtype == torch.float32 else 3e-2
    assert torch.isfinite(results[0]).all()
    assert (results[0] - results[1]).abs().max().item() <= tol * max(1.0, results[1].abs().max().item())


def test_what_does_not_fit_a_captured_layout_is_launched():
    """More tokens than the largest bucket, or more wanted places than rows: launched kernel by kernel,
    with the same result as ever; a step that is refused makes no graph."""
    from kestrel_amd.engine.step import MIXED_GRAPH_MAX_TOKENS, StepEntry, StepRefused, mixed_graph_buckets, mixed_graph_rows

    assert mixed_graph_buckets(4096)[-1] == MIXED_GRAPH_MAX_TOKENS and mixed_graph_buckets(100) == [16, 32, 64, 100]
    assert mixed_graph_rows(4) == [4] and mixed_graph_rows(300) == [8, 64, 300]
    name, dtype = "A", torch.float32
    runner = _runner(name, dtype, max_tokens_per_step=48)
    assert runner._mixed_tokens == [16, 32, 48]
    req = _request(name, "r", 800, 40)
    slot = runner.admit()
    logits = runner.step([StepEntry(slot, req.ids[:20], want=list(range(20)))]).clone()     # 20 wanted places, 8 rows
    assert runner.mixed_graph_replays == 0 and not runner._mixed
    with pytest.raises(StepRefused):
        runner.step([StepEntry(slot, req.ids[20:30], want=[3], start=5)])
    assert not runner._mixed
    last = runner.step([StepEntry(slot, req.ids[20:40], want=[19])]).clone()
    assert runner.mixed_graph_replays == 1 and sorted(runner._mixed) == [(32, 8)]
    expected = plain.forward(helpers.flat_config(name), helpers.stored_weights(helpers.model_dir(name)), req.ids, None)
    helpers.assert_close(torch.cat([logits, last]), expected[list(range(20)) + [39]], dtype, "launched, then replayed")
