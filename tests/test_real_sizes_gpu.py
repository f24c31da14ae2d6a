"""The engine at real layer sizes against the plain implementation.

Two layers (named as such: the full models have 24 and 32) at the widths of Moondream 2 (dim 2048,
feed-forward 8192, 32 heads of 64, rotary 32, vocabulary 51200, a bidirectional block of 730 given
embeddings) and of Phi-2 (dim 2560, feed-forward 10240, 32 heads of 80, rotary 32, no block), random
weights N(0, 0.02). What only these widths reach is checked end to end here: the tile choices of the
prompt GEMMs, K cut into parts at 512-token portions, the wide weight-streaming kernel at 17 to 64
rows, the LayerNorm prologue at 2048 and 2560, the vocabulary-wide head. Logits are compared at
places spread over every step; the plain model runs in float64 on the CPU.
"""

import functools
import tempfile

import pytest
import torch

from kestrel_amd.weights import InitRecipe, write_random_model
from tests import helpers
from tests.helpers import Request
from tests.plain import moondream_plain as plain

pytestmark = pytest.mark.gpu

N_LAYERS = 2
SIZES = {
    "moondream2": {"dim": 2048, "ff_dim": 8192, "n_layers": N_LAYERS, "vocab_size": 51200, "max_context": 2048,
                   "n_heads": 32, "n_kv_heads": 32, "rope_theta": 10000.0, "prefix_attn": 730, "layer_norm_eps": 1e-5},
    "phi2": {"dim": 2560, "ff_dim": 10240, "n_layers": N_LAYERS, "vocab_size": 51200, "max_context": 2048,
             "n_heads": 32, "n_kv_heads": 32, "head_dim": 80, "rotary_dim": 32, "rope_theta": 10000.0, "prefix_attn": 0,
             "layer_norm_eps": 1e-5},
}
N_SMALL = 40           # short requests that decode beside the portions of a long prompt


@functools.lru_cache(maxsize=None)
def _folder(sizes: str) -> str:
    folder = tempfile.mkdtemp(prefix=f"kestrel_amd_real_{sizes}_")
    write_random_model(folder, {"text": SIZES[sizes]}, seed=2 if sizes == "moondream2" else 3, recipe=InitRecipe(std=0.02))
    return folder


def _workload(sizes: str):
    """Requests and steps: a 1,024-position prompt in one step (with the block of given embeddings
    where the sizes have one), short prompts packed into one step, portions of 512 of a long prompt
    beside 8, then 40 decoding requests, then 16 steps of one token per request: the first four
    with all 42 rows, the rest with the 10 that are left."""
    cfg = SIZES[sizes]
    vocab, n_prefix = cfg["vocab_size"], cfg["prefix_attn"]
    prefix = torch.randn(n_prefix, cfg["dim"], generator=torch.Generator().manual_seed(77)) if n_prefix else None
    reqs = {"p": Request("p", helpers.random_ids(1400, 1040 - n_prefix, vocab), prefix),
            "m": Request("m", helpers.random_ids(1401, 1116, vocab))}
    for i in range(N_SMALL):
        reqs[f"d{i}"] = Request(f"d{i}", helpers.random_ids(1410 + i, (12 + (5 * i) % 19) + (19 if i < 8 else 6), vocab))
    small = [f"d{i}" for i in range(N_SMALL)]
    prompt = lambda tag: reqs[tag].length - (19 if int(tag[1:]) < 8 else 6)      # what is left is decoded
    steps = [[("p", 1024)]]
    steps += [[(tag, prompt(tag)) for tag in small[:8]]]
    steps += [[("m", 512)] + [(tag, 1) for tag in small[:8]]]                    # 520 tokens
    steps += [[(tag, prompt(tag)) for tag in small[8:]]]
    steps += [[("m", 512)] + [(tag, 1) for tag in small]]                        # 552 tokens
    steps += [[("m", 76)] + [(tag, 1) for tag in small]]
    steps += [[("p", 1), ("m", 1)] + [(tag, 1) for tag in small]] * 4            # 42 rows; d8.. end here
    steps += [[("p", 1), ("m", 1)] + [(tag, 1) for tag in small[:8]]] * 12       # 10 rows
    return reqs, steps


@functools.lru_cache(maxsize=None)
def _expected(sizes: str):
    """float64 logits of every request at every position, request by request."""
    cfg = SIZES[sizes]
    weights = {k: v.double() for k, v in helpers.stored_weights(_folder(sizes)).items()}
    reqs, _ = _workload(sizes)
    return {tag: plain.forward(cfg, weights, req.ids, req.prefix).float() for tag, req in reqs.items()}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("sizes", ["moondream2", "phi2"])
def test_real_layer_sizes_against_the_plain_implementation(sizes, dtype):
    from kestrel_amd.engine.loading import load_model, make_runner

    reqs, steps = _workload(sizes)
    fed = {}
    for step in steps:
        for tag, count in step:
            fed[tag] = fed.get(tag, 0) + count
    assert all(fed[tag] == req.length for tag, req in reqs.items())
    net = load_model(_folder(sizes), dtype, torch.device("cuda:0"))
    pages = sum(-(-req.length // 16) for req in reqs.values()) + 4
    runner = make_runner(net, 16, pages, len(reqs), max_tokens_per_step=1024)
    helpers.poison_cache(runner)
    got = helpers.replay(runner, reqs, steps)
    expected = _expected(sizes)
    for tag, req in reqs.items():
        helpers.assert_close(got[tag], expected[tag], dtype, f"{sizes} sizes, {N_LAYERS} layers, request {tag}")


# ----------------------------------------------------------------------------------------------------
# the decode path that serving and the benchmark run: steps replayed as HIP graphs
# ----------------------------------------------------------------------------------------------------
N_GRAPH = 64
SAMPLED = ("g1", "g9")     # their tokens after the prompt are the engine's own greedy choices, fed as PENDING_TOKEN


def _graph_workload(sizes: str):
    """64 short requests and one long one (1,030 places: past 1,024 keys a row's tiles do not divide over
    the waves of the decode attention kernel), their prompts in eager steps, then decode-only steps of
    1, 2, 4, 5, 8 and 64 rows, a request that ends and another that takes its slot and pages over,
    and returns to buckets captured earlier. Returns the requests, the prompt steps and the decode steps."""
    cfg = SIZES[sizes]
    vocab, n_prefix = cfg["vocab_size"], cfg["prefix_attn"]
    prefix = torch.randn(n_prefix, cfg["dim"], generator=torch.Generator().manual_seed(78)) if n_prefix else None
    tags = [f"g{i}" for i in range(N_GRAPH)]
    every = ["g0", "g1", "g2", "g3", "n0"] + tags[5:]
    decode = [["g0"], ["g0", "g1"], ["g0", "g1", "g2", "g3"], ["g0", "g1", "g2", "g3", "g4"],
              "g4 ends, n0 joins",
              ["g0", "g1", "g2", "g3", "n0", "g5", "g6", "g7"], every, ["g1"], every, ["g0", "g1"], ["g9", "g1", "g0", "g12"]]
    counts = {}
    for step in decode:
        if isinstance(step, list):
            for tag in step:
                counts[tag] = counts.get(tag, 0) + 1
    prompt_len = {tag: 6 + (11 * i) % 17 for i, tag in enumerate(tags)}
    prompt_len["g0"] = 1030
    prompt_len["n0"] = 21
    reqs = {}
    for i, tag in enumerate(tags + ["n0"]):
        n_ids = prompt_len[tag] + (0 if tag in SAMPLED else counts[tag])
        if tag == "g0":
            reqs[tag] = Request(tag, helpers.random_ids(1500, n_ids - n_prefix, vocab), prefix)
        else:
            reqs[tag] = Request(tag, helpers.random_ids(1500 + i, n_ids, vocab))
    prompts = [[("g0", prompt_len["g0"])], [(tag, prompt_len[tag]) for tag in tags[1:]]]
    return reqs, prompt_len, prompts, decode


def _step_graph_workload(runner, sampler, reqs, prompt_len, entries_of):
    """One step: ``entries_of`` = [(tag, count)]. Only the last place of each entry is wanted; every row of
    logits is sampled greedily into the device table of pending tokens (as the scheduler does), and the
    requests in SAMPLED take their next token from there. Returns {tag: logits row}."""
    from kestrel_amd.engine.step import PENDING_TOKEN, StepEntry

    entries = []
    for tag, count in entries_of:
        req = reqs[tag]
        if req.slot is None:
            req.slot = runner.admit()
        if tag in SAMPLED and req.done >= prompt_len[tag]:
            assert count == 1 and req.done == len(req.ids) - 1
            entries.append(StepEntry(req.slot, [PENDING_TOKEN], want=[0]))
            req.done += 1
        else:
            tokens, embeds, bidir, _lo = req.take(count)
            entries.append(StepEntry(req.slot, tokens, want=[len(tokens) - 1], embeds=embeds, bidirectional=bidir))
    logits = runner.step(entries)
    ids = sampler.greedy(logits, slots=runner.logit_slots).tolist()
    rows = logits.clone()
    out = {}
    for row, (tag, _count) in enumerate(entries_of):
        out[tag] = rows[row]
        if tag in SAMPLED:
            reqs[tag].ids.append(int(ids[row]))          # what the next step's PENDING_TOKEN stands for
            reqs[tag].length += 1
    return out


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("sizes", ["moondream2", "phi2"])
def test_replayed_decode_graphs_at_real_layer_sizes(sizes, dtype, monkeypatch):
    """What serving runs when it decodes: graphs on, buckets of 1, 2, 4, 8 and 64 rows captured on padding rows
    and replayed (with padding rows at 5 of 8), ids taken from the device table that sampling filled, a
    slot and its pages taken over between replays, the head's launch that normalises the rows itself; at
    Moondream 2's widths in bf16 the steps of 1, 2 and 4 rows run the feed-forward's first linear inside the
    attention launch. Every row of logits against the plain implementation."""
    from kestrel_amd.engine.loading import load_model, make_runner
    from kestrel_amd.ops import fast
    from kestrel_amd.sampling import Sampler

    reqs, prompt_len, prompts, decode = _graph_workload(sizes)
    net = load_model(_folder(sizes), dtype, torch.device("cuda:0"))
    pages = sum(-(-(req.length + 12) // 16) for tag, req in reqs.items() if tag != "n0") + 1
    runner = make_runner(net, 16, pages, N_GRAPH, max_tokens_per_step=2048, enable_graphs=True)
    helpers.poison_cache(runner)
    sampler = Sampler(net.device, pending=runner.pending)
    launches = []
    plain_decode = fast.attention_decode_bf16

    def watched(*args, **kwargs):
        done = plain_decode(*args, **kwargs)
        if done:
            launches.append((args[0].shape[0], kwargs.get("beside") is not None))
        return done

    monkeypatch.setattr(fast, "attention_decode_bf16", watched)
    got = {tag: {} for tag in reqs}            # request -> {position: logits row}
    n_replays = 0
    for step in prompts:
        for tag, row in _step_graph_workload(runner, sampler, reqs, prompt_len, step).items():
            got[tag][reqs[tag].done - 1] = row
    assert runner.graph_replays == 0
    for step in decode:
        if not isinstance(step, list):
            gone = reqs["g4"]
            assert gone.done == gone.length
            slot = gone.slot
            runner.release(slot)
            gone.slot = None
            for tag, row in _step_graph_workload(runner, sampler, reqs, prompt_len, [("n0", prompt_len["n0"])]).items():
                got[tag][reqs[tag].done - 1] = row
            assert reqs["n0"].slot == slot, "the request that joins takes the slot that was given back"
            continue
        for tag, row in _step_graph_workload(runner, sampler, reqs, prompt_len, [(tag, 1) for tag in step]).items():
            got[tag][reqs[tag].done - 1] = row
        n_replays += 1
        runner.cache.check()
    assert runner.graph_replays == n_replays
    assert sorted(runner._graphs) == [1, 2, 4, 8, 64]
    if dtype == torch.bfloat16:
        rows_with_linear = {n for n, beside in launches if beside}
        assert {n for n, _ in launches} >= {1, 2, 4, 8, 64}
        # head size 64 and K = 2048: the attention of 1 to 4 rows takes the linear layer along; not so at head size 80
        assert rows_with_linear == ({1, 2, 4} if sizes == "moondream2" else set()), rows_with_linear
    cfg = SIZES[sizes]
    weights = {k: v.double() for k, v in helpers.stored_weights(_folder(sizes)).items()}
    for tag, req in reqs.items():
        fed = req.done
        expected = plain.forward(cfg, weights, req.ids[:fed - req.n_prefix], req.prefix).float()
        places = sorted(got[tag])
        assert places and places[-1] == fed - 1
        actual = torch.stack([got[tag][p] for p in places])
        helpers.assert_close(actual, expected[places], dtype, f"{sizes} sizes, graphs, request {tag}")


# ----------------------------------------------------------------------------------------------------
# prompt portions replayed as HIP graphs, the vendor library's kernels among the captured
# ----------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("sizes", ["moondream2", "phi2"])
def test_replayed_prompt_portions_at_real_layer_sizes(sizes):
    """What serving runs on short prompts and on portions beside decoded tokens: the graph of a bucket of
    tokens, whose linears of more than 64 rows are the vendor library's kernels. Each graph here is replayed
    three to five times on other tokens, with replays of other graphs and decode steps between them, and every
    replay's logits are compared with the plain implementation (a node that a replay would run differently
    from the capture shows as a replay that is wrong)."""
    from kestrel_amd.engine.loading import load_model, make_runner
    from tests.test_mixed_graphs_gpu import replay_last_places

    cfg = SIZES[sizes]
    vocab = cfg["vocab_size"]
    lengths = {"a": 700, "b": 610, "c": 333, "d": 129}
    reqs = {tag: Request(tag, helpers.random_ids(1600 + i, n, vocab)) for i, (tag, n) in enumerate(lengths.items())}
    steps = [
        [("a", 200)],                                   # 256
        [("a", 1), ("b", 180)],                         # 256, a decoded token beside
        [("a", 1), ("b", 1)],                           # a decode step
        [("a", 100), ("b", 1), ("c", 20)],              # 128
        [("a", 190), ("b", 60)],                        # 256
        [("a", 1), ("b", 1), ("c", 1)],
        [("a", 90), ("b", 30), ("c", 2)],               # 128
        [("a", 117), ("b", 120), ("c", 10)],            # 256
        [("b", 100), ("c", 15), ("d", 3)],              # 128
        [("b", 117), ("c", 130)],                       # 256
        [("c", 100), ("d", 26)],                        # 128
        [("c", 55), ("d", 100)],                        # 192
    ]
    fed = {}
    for step in steps:
        for tag, count in step:
            fed[tag] = fed.get(tag, 0) + count
    assert fed == lengths
    net = load_model(_folder(sizes), torch.bfloat16, torch.device("cuda:0"))
    pages = sum(-(-n // 16) for n in lengths.values()) + 2
    runner = make_runner(net, 16, pages, 4, max_tokens_per_step=512, enable_graphs=True)
    helpers.poison_cache(runner)
    got = replay_last_places(runner, reqs, steps, wanted=1)
    assert runner.graph_replays == 2 and runner.mixed_graph_replays == len(steps) - 2
    assert sorted(runner._mixed) == [(128, 4), (192, 4), (256, 4)]
    weights = {k: v.double() for k, v in helpers.stored_weights(_folder(sizes)).items()}
    for tag, req in reqs.items():
        expected = plain.forward(cfg, weights, req.ids, None).float()
        places = sorted(got[tag])
        helpers.assert_close(torch.stack([got[tag][p] for p in places]), expected[places], torch.bfloat16,
                             f"{sizes} sizes, replayed portions, request {tag}")


def test_a_whole_prompt_replayed_three_times_at_real_layer_sizes():
    """The graph of the largest bucket (2,048 tokens), in which the vendor library runs its kernels for many rows
    (among them one that cuts the work of all tiles evenly over the compute units and sums the pieces through
    scratch memory): three prompts of about 2,000 tokens, the first with a block of given embeddings, each a
    replay of that one graph, decode steps between them; the last place of each against the plain implementation."""
    from kestrel_amd.engine.loading import load_model, make_runner
    from tests.test_mixed_graphs_gpu import replay_last_places

    sizes = "moondream2"
    cfg = SIZES[sizes]
    vocab, n_prefix = cfg["vocab_size"], cfg["prefix_attn"]
    prefix = torch.randn(n_prefix, cfg["dim"], generator=torch.Generator().manual_seed(79))
    reqs = {"a": Request("a", helpers.random_ids(1700, 1955 - n_prefix, vocab), prefix),
            "b": Request("b", helpers.random_ids(1701, 1993, vocab)),
            "c": Request("c", helpers.random_ids(1702, 2043, vocab))}
    steps = [[("a", 1950)], [("a", 1)], [("b", 1990), ("a", 1)], [("a", 1), ("b", 1)], [("c", 2040), ("a", 1), ("b", 1)],
             [("a", 1), ("b", 1), ("c", 1)], [("c", 1)], [("c", 1)]]
    net = load_model(_folder(sizes), torch.bfloat16, torch.device("cuda:0"))
    runner = make_runner(net, 16, 3 * 129, 4, max_tokens_per_step=2048, enable_graphs=True)
    helpers.poison_cache(runner)
    got = replay_last_places(runner, reqs, steps, wanted=1, poison=False)
    assert all(r.done == r.length for r in reqs.values())
    assert sorted(runner._mixed) == [(2048, 4)] and runner.mixed_graph_replays == 3 and runner.graph_replays == 5
    weights = {k: v.double() for k, v in helpers.stored_weights(_folder(sizes)).items()}
    for tag, req in reqs.items():
        expected = plain.forward(cfg, weights, req.ids, req.prefix).float()
        places = sorted(got[tag])
        helpers.assert_close(torch.stack([got[tag][p] for p in places]), expected[places], torch.bfloat16,
                             f"{sizes} sizes, a whole prompt replayed, request {tag}")
