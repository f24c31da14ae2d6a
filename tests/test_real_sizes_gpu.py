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
