"""The engine against the plain implementation under every way of cutting the work."""

import pytest
import torch

from tests import helpers
from tests.plain import moondream_plain as plain

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


def _runner(name, dtype, n_pages=64, page_size=16, max_requests=8):
    from kestrel_amd.engine.loading import load_model, make_runner

    net = load_model(helpers.model_dir(name), dtype, torch.device("cuda:0"))
    return make_runner(net, page_size, n_pages, max_requests)


def _expected(name, ids):
    folder = helpers.model_dir(name)
    return plain.forward(helpers.flat_config(name), helpers.stored_weights(folder), ids)


@pytest.mark.parametrize("dtype", DTYPES, ids=["fp32", "bf16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_whole_prompt(name, dtype):
    from kestrel_amd.engine.step import StepEntry

    runner = _runner(name, dtype)
    vocab = helpers.flat_config(name)["vocab_size"]
    for seed, length in enumerate([5, 17, 33, 70]):
        ids = helpers.random_ids(100 + seed, length, vocab)
        slot = runner.admit()
        logits = runner.step([StepEntry(slot, ids, want=list(range(length)))]).clone()
        runner.release(slot)
        helpers.assert_close(logits, _expected(name, ids), dtype, f"tiny {name} length {length}")
    runner.cache.check()
