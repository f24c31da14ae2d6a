"""The scheduler's decisions, against a runner that only keeps books (no GPU)."""

from types import SimpleNamespace

import pytest
import torch

from kestrel_amd.cache import CacheManager
from kestrel_amd.engine.scheduler import GenerationScheduler
from kestrel_amd.engine.types import GenerationRequest
from kestrel_amd.parts.specs import CacheSpec


class FakeRunner:
    """Implements what the scheduler uses of ``ModelRunner``; records every step."""

    def __init__(self, n_pages=16, page_size=4, max_requests=4, max_positions=64, vocab=64):
        self.cache = CacheManager([(CacheSpec(1, 8, None), None, None)], page_size, n_pages, max_requests)
        self.model = SimpleNamespace(plan=SimpleNamespace(max_positions=max_positions, vocab_size=vocab, dim=8))
        self.held = {}
        self.steps = []
        self.tokens = []
        self.vocab = vocab
        self.refuse_token = None        # a step with this token in an entry is refused for that entry
        self.break_at_step = None       # the step with this number fails as a whole
        self.broken = []

    def admit(self, reserve_length=0, portion=1):
        slot = self.cache.admit(reserve_length, portion)
        self.held[slot] = 0
        return slot

    def release(self, slot):
        self.cache.release(slot)
        del self.held[slot]

    def step(self, entries):
        from kestrel_amd.engine.step import StepRefused

        record = []
        wanted = 0
        for i, e in enumerate(entries):            # refusals come before anything changes, as in ModelRunner
            if self.refuse_token in list(e.tokens):
                raise StepRefused(i, f"slot {e.slot}: token {self.refuse_token} is refused by this fake")
        if self.break_at_step == len(self.steps) + len(self.broken):
            self.broken.append([e.slot for e in entries])
            raise RuntimeError("the device said no")
        for e in entries:
            start = self.held[e.slot] if e.start is None else e.start
            assert start == self.held[e.slot], "portions must follow each other"
            self.cache.ensure(e.slot, start + len(e.tokens))
            self.held[e.slot] = start + len(e.tokens)
            for lo, hi in e.bidirectional:
                assert start <= lo and hi <= start + len(e.tokens), "a block was split"
            record.append((e.slot, start, len(e.tokens), list(e.want)))
            wanted += len(e.want)
        self.steps.append(record)
        self.tokens.append([list(e.tokens) for e in entries])
        self.cache.check()
        return torch.zeros(wanted, self.vocab)


class FakeSampler:
    """Token = 10 + index of the token in its request; request seed 99 emits the stop id 0 at index 2."""

    def __init__(self):
        self.calls = []

    def sample_step(self, logits, temps, tops, seeds, indices, slots=None, suppress=(), allowed=None, logprobs=False):
        self.calls.append(dict(suppress=list(suppress), allowed=allowed, logprobs=logprobs, indices=list(indices)))
        ids = self.sample(logits, temps, tops, seeds, indices, slots)
        return ids, (torch.tensor([-0.5 * (i + 1) for i in indices]) if logprobs else None)

    def sample(self, logits, temps, tops, seeds, indices, slots=None):
        assert logits.shape[0] == len(temps) == len(indices)
        assert slots is None or len(slots) == len(indices)
        return torch.tensor([0 if (s == 99 and i == 2) else 10 + i for s, i in zip(seeds, indices)], dtype=torch.int32)


def _scheduler(runner=None, max_batch_size=4, budget=16, pipeline_depth=1, **kw):
    runner = runner or FakeRunner(**kw)
    return GenerationScheduler(runner, FakeSampler(), max_batch_size, budget, eos_token_ids=(0,),
                               pipeline_depth=pipeline_depth), runner


def _req(i, n_prompt, n_new, **kw):
    return GenerationRequest(i, list(range(1, n_prompt + 1)), n_new, **kw)


def test_prompt_is_cut_under_the_token_budget_and_then_decoded():
    sched, runner = _scheduler(budget=16)
    sched.enqueue_request(_req(0, 40, 3))
    results = sched.run_until_done()
    sizes = [[(n, want) for _s, _p, n, want in step] for step in runner.steps]
    assert sizes[:3] == [[(16, [])], [(16, [])], [(8, [7])]]          # portions of 16, 16, 8; logits only at the end
    assert sizes[3:] == [[(1, [0])], [(1, [0])]]                       # then one token a step
    assert results[0].tokens == [10, 11, 12] and results[0].finish_reason == "length"
    assert runner.cache.groups[0].pool.free_count == 16 and runner.cache.free_slots == 4


def test_portions_end_on_page_boundaries():
    """A portion that does not finish its prompt is cut back to a page boundary (pages of 4 here),
    so that the next one starts on a fresh page; the last portion takes what is left."""
    sched, runner = _scheduler(budget=10)
    sched.enqueue_request(_req(0, 23, 1))
    sched.run_until_done()
    portions = [(p, n) for step in runner.steps for _s, p, n, _w in step if n > 1]
    assert portions == [(0, 8), (8, 8), (16, 7)]
    # a budget smaller than a page still makes progress
    sched, runner = _scheduler(budget=3)
    sched.enqueue_request(_req(0, 9, 1))
    sched.run_until_done()
    assert [(p, n) for step in runner.steps for _s, p, n, _w in step][:4] == [(0, 3), (3, 1), (4, 3), (7, 2)]


def test_decodes_ride_beside_prompt_portions():
    sched, runner = _scheduler(budget=8)
    sched.enqueue_request(_req(0, 4, 6))
    sched.advance()                                                     # request 0 prefilled, first token
    sched.enqueue_request(_req(1, 20, 2))
    sched.advance()
    step = runner.steps[-1]
    # the decoding request has its token first, the prompt gets the rest of the budget, cut down to a
    # page boundary (pages of 4: 4 of the 7 places left); in the packed batch the portion stands first
    assert [(n, want) for _s, _p, n, want in step] == [(4, []), (1, [0])]
    sched.advance()
    assert [(p, n) for _s, p, n, _w in runner.steps[-1]][0] == (4, 4)      # the next portion starts on that boundary
    results = sched.run_until_done()
    assert sorted(r.request_id for r in results) == [0, 1]


def test_stop_token_and_length_finish():
    sched, runner = _scheduler()
    sched.enqueue_request(_req(0, 3, 10, seed=99))
    sched.enqueue_request(_req(1, 3, 2))
    results = {r.request_id: r for r in sched.run_until_done()}
    assert results[0].tokens == [10, 11, 0] and results[0].finish_reason == "stop"
    assert results[1].tokens == [10, 11] and results[1].finish_reason == "length"
    # the context length ends a request too
    sched, runner = _scheduler(max_positions=12)
    sched.enqueue_request(_req(2, 8, 100))
    (result,) = sched.run_until_done()
    assert result.finish_reason == "length" and len(result.tokens) == 4     # 8 + 4 = 12 positions
    assert result.metrics.prompt_tokens == 8 and result.metrics.decode_tokens == 4


def test_at_most_max_batch_size_requests_are_live():
    sched, runner = _scheduler(max_batch_size=2, budget=64, n_pages=64)
    for i in range(5):
        sched.enqueue_request(_req(i, 5, 3))
    sched.advance()
    assert len(runner.steps[-1]) == 2 and len(sched.waiting) == 3
    results = sched.run_until_done()
    assert len(results) == 5
    assert max(len(step) for step in runner.steps) <= 2


def test_a_request_waits_for_pages_and_a_smaller_one_may_pass():
    # 8 pages of 4 = 32 tokens. Request 0 takes 6 pages (24); request 1 needs 5 and must wait;
    # request 2 needs 2 and passes; request 1 runs once request 0 has given its pages back.
    sched, runner = _scheduler(n_pages=8, budget=32)
    sched.enqueue_request(_req(0, 20, 4))
    sched.enqueue_request(_req(1, 16, 4))
    sched.enqueue_request(_req(2, 4, 4))
    sched.advance()
    assert [s.request.request_id for s in sched.running] == [0, 2]
    assert [s.request.request_id for s in sched.waiting] == [1]
    results = sched.run_until_done()
    assert [r.request_id for r in results] == [0, 2, 1]
    assert all(r.finish_reason == "length" for r in results)
    assert runner.cache.groups[0].pool.free_count == 8


def test_a_request_that_can_never_fit_fails_alone():
    sched, runner = _scheduler(n_pages=4, budget=32)      # 16 tokens in all
    sched.enqueue_request(_req(0, 20, 10))
    sched.enqueue_request(_req(1, 4, 2))
    results = {r.request_id: r for r in sched.run_until_done()}
    assert results[1].finish_reason == "length"
    assert results[0].finish_reason == "error"
    assert results[0].error == "Insufficient KV cache capacity for request 0 (needs 30 tokens)."


def test_a_bidirectional_block_goes_in_one_portion():
    sched, runner = _scheduler(budget=12, n_pages=32)
    embeds = torch.zeros(7, 8)
    sched.enqueue_request(_req(0, 9, 2))
    sched.advance()
    sched.enqueue_request(GenerationRequest(1, [5, 6, 7, 8, 9, 10], 2, prefix_embeds=embeds, prefix_ids=[0]))
    sched.advance()
    step = runner.steps[-1]
    # 1 decode + 11 budget: block of 8 (BOS + 7 rows) and 3 text tokens, cut back to the page boundary at 8
    assert [(n, w) for _s, _p, n, w in step] == [(8, []), (1, [0])]
    sched.run_until_done()
    # a block larger than what is left of the budget waits for a step with room; it is never split
    sched, runner = _scheduler(budget=9, n_pages=32)
    sched.enqueue_request(_req(0, 5, 2))
    sched.enqueue_request(GenerationRequest(1, [5, 6], 1, prefix_embeds=embeds, prefix_ids=[0]))
    sched.advance()
    assert [n for _s, _p, n, _w in runner.steps[-1]] == [5]
    sched.run_until_done()
    assert any(n == 8 or n == 9 or n == 10 for step in runner.steps for _s, _p, n, _w in step)
    with pytest.raises(ValueError, match="does not fit in one step"):
        sched.enqueue_request(GenerationRequest(2, [1], 1, prefix_embeds=torch.zeros(20, 8)))


def test_several_blocks_in_one_request_are_each_kept_whole():
    """A prompt with two blocks of given embeddings between text: ids with -1 where rows of ``prompt_embeds``
    stand, ``blocks`` naming the ranges. Portions are cut so that no block is split: a portion that would end
    inside a block ends at the block's start, whatever the page boundary says."""
    ids = [1, 2, 3] + [-1] * 6 + [4, 5, 6, 7, 8] + [-1] * 5 + [9, 10]           # blocks [3, 9) and [14, 19)
    rows = torch.arange(11 * 8, dtype=torch.float32).reshape(11, 8)
    sched, runner = _scheduler(budget=8, n_pages=32)
    sched.enqueue_request(GenerationRequest(0, ids, 2, prompt_embeds=rows, blocks=[(14, 19), (3, 9)]))
    seen = []
    step_entry = runner.step

    def watching(entries):
        seen.extend((e.start, len(e.tokens), list(e.bidirectional), None if e.embeds is None else e.embeds.clone())
                    for e in entries if len(e.tokens) > 1)
        return step_entry(entries)

    runner.step = watching
    (result,) = sched.run_until_done()
    assert result.finish_reason == "length" and len(result.tokens) == 2
    # budget 8, pages of 4: [0, 8) would split the first block -> [0, 3); [3, 11) is not cut back to the page
    # boundary at 8, which lies inside the block; [11, 19) ends with the second block; the rest follows
    assert [(start, n) for start, n, _b, _e in seen] == [(0, 3), (3, 8), (11, 8), (19, 2)]
    assert [b for _s, _n, b, _e in seen] == [[], [(3, 9)], [(14, 19)], []]
    assert torch.equal(seen[1][3], rows[:6]) and torch.equal(seen[2][3], rows[6:])
    assert seen[0][3] is None and seen[3][3] is None
    for bad, message in ((dict(blocks=[(3, 9), (8, 12)]), "not overlap"), (dict(blocks=[(20, 30)]), "inside the prompt"),
                         (dict(blocks=[(4, 4)]), "at least one position"),
                         (dict(prompt_embeds=rows[:10]), "10 rows for 11 places")):
        options = dict(prompt_embeds=rows, blocks=[(3, 9)])
        options.update(bad)
        with pytest.raises(ValueError, match=message):
            sched.enqueue_request(GenerationRequest(1, ids, 2, **options))
    with pytest.raises(ValueError, match="does not fit in one step"):
        sched.enqueue_request(GenerationRequest(2, ids, 2, prompt_embeds=rows, blocks=[(0, 12)]))


def test_bad_requests_are_refused():
    sched, _ = _scheduler()
    for bad in (dict(max_new_tokens=0), dict(temperature=-1.0), dict(top_p=0.0), dict(top_p=1.5)):
        kwargs = dict(max_new_tokens=2)
        kwargs.update(bad)
        with pytest.raises(ValueError):
            sched.enqueue_request(GenerationRequest(0, [1, 2], **kwargs))
    with pytest.raises(ValueError, match="at least one"):
        sched.enqueue_request(GenerationRequest(0, [], 2))
    with pytest.raises(ValueError, match="leaves no room"):
        sched.enqueue_request(_req(0, 64, 2))


def test_what_the_step_function_would_refuse_is_refused_at_the_door():
    sched, _ = _scheduler()
    bad = [
        (dict(prompt_ids=[1, 64]), "token id 64 outside the vocabulary"),
        (dict(prompt_ids=[1, -1]), "token id -1 outside"),
        (dict(prompt_ids=[-2, 3]), "token id -2 outside"),          # would otherwise read as "the pending token"
        (dict(prompt_ids=[1], prefix_ids=[70], prefix_embeds=torch.zeros(2, 8)), "prefix_ids: token id 70"),
        (dict(prompt_ids=[1], prefix_embeds=torch.zeros(2, 9)), "prefix_embeds"),
        (dict(prompt_ids=[1], prefix_embeds=torch.zeros(2, 8, dtype=torch.int32)), "prefix_embeds"),
        (dict(prompt_ids=[1], prefix_embeds=torch.zeros(16)), "prefix_embeds"),
        (dict(prompt_ids=[1], suppressed_token_ids=(99,)), "suppressed_token_ids"),
        (dict(prompt_ids=[1], suppress_next_token_ids=(-5,)), "suppress_next_token_ids"),
        (dict(prompt_ids=[1], allowed_token_ids=(3, 64)), "allowed_token_ids"),
        (dict(prompt_ids=[1.5, 2.0]), "integer token ids"),
        (dict(prompt_ids=[[1, 2]]), "flat sequence"),
    ]
    for kwargs, message in bad:
        with pytest.raises(ValueError, match=message):
            sched.enqueue_request(GenerationRequest(0, max_new_tokens=2, **kwargs))
    assert not sched.has_pending_work()


@pytest.mark.parametrize("depth", [1, 2])
def test_a_request_the_step_function_refuses_fails_alone(depth):
    """Token 31 is inside the vocabulary, so the door lets it in; the (fake) step function refuses
    the entry that holds it. The others of that step are planned again and finish as if it had
    never been there."""
    expected = {}
    for with_bad in (False, True):
        sched, runner = _scheduler(pipeline_depth=depth, budget=16, n_pages=32)
        runner.refuse_token = 31
        sched.enqueue_request(_req(0, 5, 4))
        sched.advance()                                           # request 0 decodes when the bad one arrives
        if with_bad:
            sched.enqueue_request(GenerationRequest(1, [4, 31, 6], 3))
        sched.enqueue_request(_req(2, 6, 3))
        results = {r.request_id: r for r in sched.run_until_done()}
        good = {i: (r.tokens, r.finish_reason) for i, r in results.items() if i != 1}
        assert good == {0: ([10, 11, 12, 13], "length"), 2: ([10, 11, 12], "length")}
        if with_bad:
            assert results[1].finish_reason == "error" and "refused" in results[1].error
            assert sched.failed_steps == 1
        expected[with_bad] = good
        runner.cache.check()
        assert runner.cache.groups[0].pool.free_count == 32 and runner.cache.free_slots == 4 and not runner.held
    assert expected[False] == expected[True]


@pytest.mark.parametrize("depth", [1, 2])
def test_a_step_that_breaks_takes_its_requests_only(depth):
    """Step 2 raises something that names no entry: every request of that step fails, the ones
    that wait are served afterwards, and every page and slot comes back."""
    sched, runner = _scheduler(pipeline_depth=depth, budget=16, max_batch_size=2, n_pages=32)
    runner.break_at_step = 2
    for i in range(4):
        sched.enqueue_request(_req(i, 5, 4))
    results = {r.request_id: r for r in sched.run_until_done()}
    assert len(runner.broken) == 1 and len(runner.broken[0]) == 2
    failed = sorted(i for i, r in results.items() if r.finish_reason == "error")
    assert failed == [0, 1] and all("the device said no" in results[i].error for i in failed)
    assert all(results[i].tokens == [10, 11, 12, 13] and results[i].finish_reason == "length" for i in (2, 3))
    runner.cache.check()
    assert runner.cache.groups[0].pool.free_count == 32 and runner.cache.free_slots == 4 and not runner.held


# ---------------------------------------------------------------------- tokens generated before
def test_a_generated_prefix_is_fed_counted_and_returned():
    """``kestrel/scheduler/types.py:215-263``; result and metrics as in the reference's
    ``tests/scheduler/test_logprobs.py:177-202`` (tokens and logprobs keep the prefix at their head,
    ``decode_tokens`` counts only what was decoded now)."""
    from kestrel_amd.engine.types import GeneratedPrefix

    sched, runner = _scheduler(budget=16)
    request = GenerationRequest(7, [1], 4, return_logprobs=True, suppress_next_token_ids=(9,),
                                generated_prefix=GeneratedPrefix((20, 21), (-0.1, -0.2)))
    assert request.prompt_length == 1 and request.generated_prefix_length == 2 and request.prefill_length == 3
    sched.enqueue_request(request)
    (result,) = sched.run_until_done()
    # fed: the prompt and the two old tokens in one portion; then one decode; 2 + 2 = max_new_tokens
    assert runner.tokens[0] == [[1, 20, 21]] and [n for step in runner.steps for _s, _p, n, _w in step] == [3, 1]
    assert result.tokens == [20, 21, 12, 13] and result.finish_reason == "length"
    assert result.logprobs == [-0.1, -0.2, -1.5, -2.0]           # the fake sampler: -0.5 * (index + 1)
    assert result.metrics.decode_tokens == 2 and result.metrics.prompt_tokens == 1
    # the one-shot suppression applies to the first token after the prefix (index 2), not later
    calls = sched.sampler.calls
    assert calls[0]["indices"] == [2] and calls[0]["suppress"] == [(0, 9)] and calls[1]["suppress"] == []
    assert runner.cache.groups[0].pool.free_count == 16


def test_a_generated_prefix_is_checked():
    from kestrel_amd.engine.types import GeneratedPrefix

    with pytest.raises(ValueError, match="leaves nothing to generate"):
        GenerationRequest(7, [1], 2, generated_prefix=GeneratedPrefix((10, 11)))
    with pytest.raises(ValueError, match="one per token"):
        GenerationRequest(7, [1], 4, generated_prefix=GeneratedPrefix((10,), ()))
    with pytest.raises(ValueError, match="must bring those of the tokens"):
        GenerationRequest(7, [1], 4, return_logprobs=True, generated_prefix=GeneratedPrefix((10,)))
    sched, _ = _scheduler()
    with pytest.raises(ValueError, match="generated_prefix.tokens: token id 70"):
        sched.enqueue_request(GenerationRequest(7, [1], 4, generated_prefix=GeneratedPrefix((70,))))


def test_a_generated_prefix_is_cut_like_a_prompt():
    from kestrel_amd.engine.types import GeneratedPrefix

    sched, runner = _scheduler(budget=4)
    sched.enqueue_request(GenerationRequest(0, [1, 2, 3], 6, generated_prefix=GeneratedPrefix((20, 21, 22))))
    (result,) = sched.run_until_done()
    assert runner.tokens[0] == [[1, 2, 3, 20]] and runner.tokens[1] == [[21, 22]]
    assert runner.steps[0][0][3] == [] and runner.steps[1][0][3] == [1]
    assert result.tokens == [20, 21, 22, 13, 14, 15]


def test_tokens_are_streamed_as_they_are_committed():
    sched, _ = _scheduler()
    seen = []
    sched.enqueue_request(_req(0, 3, 3, on_token=lambda tok, i: seen.append((tok, i))))
    sched.run_until_done()
    assert seen == [(10, 0), (11, 1), (12, 2)]


# ---------------------------------------------------------------------- two steps in flight
def _mixed_requests():
    return [_req(0, 3, 10, seed=99), _req(1, 3, 2), _req(2, 21, 5), _req(3, 7, 1), _req(4, 5, 6, seed=99)]


def test_pipelined_scheduling_gives_the_same_results():
    outcomes = []
    for depth in (1, 2):
        sched, runner = _scheduler(pipeline_depth=depth, budget=16, max_batch_size=3, n_pages=24)
        for request in _mixed_requests():
            sched.enqueue_request(request)
        results = {r.request_id: (r.tokens, r.finish_reason) for r in sched.run_until_done()}
        assert runner.cache.groups[0].pool.free_count == 24 and runner.cache.free_slots == 4
        assert not runner.held
        outcomes.append(results)
    assert outcomes[0] == outcomes[1]
    assert outcomes[0][0] == ([10, 11, 0], "stop") and outcomes[0][3] == ([10], "length")


def test_a_step_is_launched_before_the_last_one_is_read():
    from kestrel_amd.engine.step import PENDING_TOKEN

    sched, runner = _scheduler(pipeline_depth=2)
    seen = []
    sched.enqueue_request(_req(0, 3, 4, on_token=lambda tok, i: seen.append(i)))
    sched.advance()                                    # the prompt is launched; nothing read yet
    assert seen == [] and len(runner.steps) == 1
    assert sched.running and sched.running[0].launched == 1 and sched.running[0].tokens == []
    sched.advance()                                    # first decode launched with a token the host has not seen
    assert runner.tokens[-1] == [[PENDING_TOKEN]] and seen == [0]
    sched.run_until_done()
    assert seen == [0, 1, 2, 3]
    # the length limit is known without the token: prompt + 3 decode steps, none beyond
    assert [n for step in runner.steps for _s, _p, n, _w in step] == [3, 1, 1, 1]
    assert all(tokens == [[PENDING_TOKEN]] for tokens in runner.tokens[1:])


def test_a_request_that_stopped_runs_one_step_too_many_and_is_freed_after_it():
    sched, runner = _scheduler(pipeline_depth=2)
    sched.enqueue_request(_req(0, 3, 10, seed=99))     # stops with its third token
    done = []
    while sched.has_pending_work():
        sched.advance()
        finished = sched.pop_completed()
        if finished:
            done.append((len(runner.steps), finished[0], dict(runner.held)))
    (steps_then, result, held_then), = done
    assert result.tokens == [10, 11, 0] and result.finish_reason == "stop"
    # prompt, two decodes that count and one more that was already launched when the stop was read
    assert len(runner.steps) == 4 and steps_then == 4
    assert held_then, "the slot is still held while the extra step is in flight"
    assert not runner.held and runner.cache.groups[0].pool.free_count == 16 and runner.cache.free_slots == 4


def test_a_finished_request_makes_room_one_step_later_when_pipelined():
    sched, runner = _scheduler(pipeline_depth=2, max_batch_size=1, n_pages=64, budget=64)
    sched.enqueue_request(_req(0, 4, 2))
    sched.enqueue_request(_req(1, 4, 2))
    results = sched.run_until_done()
    assert [r.request_id for r in results] == [0, 1] and all(r.tokens == [10, 11] for r in results)
    assert max(len(step) for step in runner.steps) == 1


# ---------------------------------------------------------------------- masks and scores
@pytest.mark.parametrize("depth", [1, 2])
def test_masks_and_logprobs_reach_the_sampler(depth):
    sched, runner = _scheduler(pipeline_depth=depth)
    sched.enqueue_request(_req(0, 3, 3, return_logprobs=True, suppress_next_token_ids=(7, 8), suppressed_token_ids=(5,)))
    sched.enqueue_request(_req(1, 4, 2, allowed_token_ids=(10, 11, 12)))
    sched.enqueue_request(_req(2, 2, 2))
    results = {r.request_id: r for r in sched.run_until_done()}
    calls = sched.sampler.calls
    # first step: all three prompts end; request 0 is row 0 and suppresses 5 always and 7, 8 for its first token
    assert sorted(calls[0]["suppress"]) == [(0, 5), (0, 7), (0, 8)]
    assert calls[0]["allowed"] == [None, (10, 11, 12), None] and calls[0]["logprobs"] is True
    # afterwards only the lasting suppression is left
    assert all(sorted(c["suppress"]) == [(0, 5)] for c in calls[1:] if c["suppress"])
    assert results[0].logprobs == [-0.5, -1.0, -1.5] and len(results[0].tokens) == 3
    assert results[1].logprobs is None and results[2].logprobs is None
    with pytest.raises(ValueError, match="allow-list"):
        sched.enqueue_request(_req(3, 2, 2, allowed_token_ids=()))


# ---------------------------------------------------------------------- graph buckets
def test_graph_buckets_follow_the_reference_rule():
    """1, 2, 4, 8, every multiple of 16, and the largest batch itself: the reference's vectors
    (``tests/test_decode_graph_manager.py:77-81``) and two sizes at which powers of two would differ."""
    from kestrel_amd.engine.step import graph_buckets

    assert graph_buckets(1) == [1]
    assert graph_buckets(3) == [1, 2, 3]
    assert graph_buckets(16) == [1, 2, 4, 8, 16]
    assert graph_buckets(33) == [1, 2, 4, 8, 16, 32, 33]
    assert graph_buckets(64) == [1, 2, 4, 8, 16, 32, 48, 64]
    assert graph_buckets(100) == [1, 2, 4, 8, 16, 32, 48, 64, 80, 96, 100]


def test_buckets_of_steps_of_any_shape():
    """Token counts and numbers of rows that steps other than decode steps are captured for: fine where a step is
    short, in steps of 128 further up, never beyond the step's token limit or 2,048 tokens."""
    from kestrel_amd.engine.step import MIXED_GRAPH_MAX_TOKENS, mixed_graph_buckets, mixed_graph_rows

    assert MIXED_GRAPH_MAX_TOKENS == 2048
    assert mixed_graph_buckets(1) == [1] and mixed_graph_buckets(16) == [16] and mixed_graph_buckets(40) == [16, 32, 40]
    assert mixed_graph_buckets(512) == [16, 32, 64, 128, 192, 256, 320, 384, 448, 512]
    assert mixed_graph_buckets(700) == [16, 32, 64, 128, 192, 256, 320, 384, 448, 512, 640, 700]
    top = mixed_graph_buckets(10 ** 6)
    assert top == mixed_graph_buckets(2048) and top[-1] == 2048 and top[-3:] == [1792, 1920, 2048]
    for tokens in range(1, 2049):
        bucket = next(b for b in top if b >= tokens)
        # never more than 127 tokens that fill a step up, and from 16 tokens on fewer than the step's own
        assert bucket - tokens < 128 and (tokens < 16 or bucket < 2 * tokens), (tokens, bucket)
    assert mixed_graph_rows(1) == [1] and mixed_graph_rows(6) == [6] and mixed_graph_rows(8) == [8]
    assert mixed_graph_rows(64) == [8, 64] and mixed_graph_rows(300) == [8, 64, 300]
