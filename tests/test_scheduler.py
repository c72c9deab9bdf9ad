"""The scheduler's decisions, on the CPU, above a stand-in for the step function that does
the cache bookkeeping of the real engine and returns made-up logits."""

import random
from collections import Counter
from types import SimpleNamespace

import pytest
import torch

from pagedserve_amd.cache import CacheGroupSpec, CacheManager
from pagedserve_amd.engine.engine import StepOutput
from pagedserve_amd.engine.scheduler import (ORCA_STRATEGY, SARATHI_STRATEGY,
                                             ContinuousBatchScheduler)
from pagedserve_amd.sampling import SamplingParams, uniform_for

VOCAB = 50


class FakeEngine:
    """Cache bookkeeping as in Engine.step; logits put all mass on a token that depends on
    the request's whole history, so outputs tell whether every token arrived in order."""

    def __init__(self, pages=64, page_size=4, max_requests=8, max_step_tokens=64, max_positions=128,
                 window=0):
        self.spec = SimpleNamespace(vocab_size=VOCAB, max_positions=max_positions)
        groups = [CacheGroupSpec((0,), 1, 16, 0)]
        if window:
            groups.append(CacheGroupSpec((1,), 1, 16, window))
        self.cache = CacheManager(groups, pages, page_size, max_requests, torch.float32, "cpu",
                                  max_positions=max_positions, allocate_pools=False)
        self.max_requests = max_requests
        self.max_step_tokens = max_step_tokens
        self.history = {}
        self.steps = []
        self.fail_next = False

    def step(self, entries, greedy=False):
        if self.fail_next:
            self.fail_next = False
            raise RuntimeError("injected failure")
        assert sum(len(e.tokens) for e in entries) <= self.max_step_tokens
        assert len({e.request_id for e in entries}) == len(entries)
        rows = []
        for entry in entries:
            if entry.request_id not in self.cache.requests:
                self.cache.admit(entry.request_id)
                self.history[entry.request_id] = []
            start = self.cache.length(entry.request_id)
            self.cache.grow(entry.request_id, start + len(entry.tokens))
        for entry in entries:
            start = self.cache.length(entry.request_id)
            self.history[entry.request_id].extend(entry.tokens)
            self.cache.commit(entry.request_id, start + len(entry.tokens))
            for place in entry.want:
                assert place == len(entry.tokens) - 1
                seen = self.history[entry.request_id]
                row = torch.zeros(VOCAB)
                row[(sum(seen) * 7 + len(seen)) % (VOCAB - 1)] = 5.0   # never VOCAB-1 (the end token)
                rows.append(row)
        self.steps.append([(e.request_id, list(e.tokens), list(e.want)) for e in entries])
        self.cache.check_invariants()
        logits = torch.stack(rows) if rows else torch.zeros((0, VOCAB))
        return StepOutput(logits=logits, rows=[])

    def finish(self, request_id):
        self.cache.release(request_id)
        del self.history[request_id]


class ArgmaxSampler:
    def sample(self, logits, params, keys, indices, seeds):
        return logits.argmax(-1).tolist()


def expected_tokens(prompt, count):
    seen, out = list(prompt), []
    for _ in range(count):
        token = (sum(seen) * 7 + len(seen)) % (VOCAB - 1)
        out.append(token)
        seen.append(token)
    return out


def make(strategy=ORCA_STRATEGY, engine=None, **kwargs):
    engine = engine or FakeEngine()
    kwargs.setdefault("max_batch_size", engine.max_requests)
    return ContinuousBatchScheduler(engine, ArgmaxSampler(), tokenizer=None,
                                    scheduling_strategy=strategy, **kwargs), engine


def test_orca_runs_whole_prompts_together():
    # testing/test_project.py:940-988: two prompts of different length in one step,
    # finished after two tokens, nothing reserved, nothing left in the manager
    scheduler, engine = make(max_batch_size=4)
    a = scheduler.add_token_request([1, 2, 3], max_new_tokens=2)
    b = scheduler.add_token_request([4, 5, 6, 7, 8], max_new_tokens=2)
    first = scheduler.step()
    assert set(first) == {a, b}
    assert engine.steps[0] == [(a, [1, 2, 3], [2]), (b, [4, 5, 6, 7, 8], [4])]
    second = scheduler.step()
    assert set(second) == {a, b} and not scheduler.has_work()
    assert engine.steps[1] == [(a, [first[a]], [0]), (b, [first[b]], [0])]
    assert scheduler.reserved_blocks == [0] and not engine.cache.requests
    assert scheduler.finished[a].generated_token_ids == expected_tokens([1, 2, 3], 2)
    assert scheduler.finished[b].finish_reason == "length"
    assert scheduler.step() == {}


def test_sarathi_chunks_and_piggybacks():
    # testing/test_project.py:991-1051: chunk 2 -> {}, {}, {A}; B's first portion rides with A's decode
    scheduler, engine = make(SARATHI_STRATEGY, prefill_chunk_size=2, max_batch_size=4)
    a = scheduler.add_token_request([1, 2, 3, 4, 5], max_new_tokens=3)
    assert scheduler.step() == {} and scheduler.waiting[0].prefill_cursor == 2
    assert scheduler.step() == {} and scheduler.waiting[0].prefill_cursor == 4
    assert engine.cache.length(a) == 4
    emitted = scheduler.step()
    assert set(emitted) == {a} and not scheduler.waiting and a in scheduler.active
    assert [step[0][2] for step in engine.steps] == [[], [], [0]]
    b = scheduler.add_token_request([9, 8, 7], max_new_tokens=1)
    emitted = scheduler.step()
    assert set(emitted) == {a}
    assert engine.steps[-1] == [(a, [scheduler.active[a].generated_token_ids[0]], [0]), (b, [9, 8], [])]
    assert engine.cache.length(a) == 6 and engine.cache.length(b) == 2
    emitted = scheduler.step()
    assert set(emitted) == {a, b}
    assert not scheduler.has_work()
    assert scheduler.finished[a].generated_token_ids == expected_tokens([1, 2, 3, 4, 5], 3)
    assert scheduler.finished[b].generated_token_ids == expected_tokens([9, 8, 7], 1)


def test_token_budget_cuts_prompts_in_both_strategies():
    for strategy in (ORCA_STRATEGY, SARATHI_STRATEGY):
        scheduler, engine = make(strategy, max_num_batched_tokens=6, prefill_chunk_size=4,
                                 max_prefill_requests=8)
        a = scheduler.add_token_request(list(range(1, 11)), max_new_tokens=2)
        b = scheduler.add_token_request([3, 3, 3], max_new_tokens=2)
        scheduler.run_until_complete()
        assert all(sum(len(tokens) for _, tokens, _ in step) <= 6 for step in engine.steps)
        assert scheduler.finished[a].generated_token_ids == expected_tokens(list(range(1, 11)), 2)
        assert scheduler.finished[b].generated_token_ids == expected_tokens([3, 3, 3], 2)
        portions = [len(tokens) for step in engine.steps for rid, tokens, _ in step if rid == a and len(tokens) > 1]
        assert sum(portions) == 10 and max(portions) <= (6 if strategy == ORCA_STRATEGY else 4)


def test_results_do_not_depend_on_strategy_chunk_or_batch_limit():
    prompts = [[(i * 5 + j) % VOCAB for j in range(3 + 4 * i)] for i in range(6)]
    outputs = []
    for strategy, kwargs in ((ORCA_STRATEGY, {}), (ORCA_STRATEGY, {"max_batch_size": 2}),
                             (SARATHI_STRATEGY, {"prefill_chunk_size": 2}),
                             (SARATHI_STRATEGY, {"prefill_chunk_size": 5, "max_prefill_requests": 3}),
                             (ORCA_STRATEGY, {"max_num_batched_tokens": 7})):
        scheduler, _ = make(strategy, **kwargs)
        ids = [scheduler.add_token_request(p, max_new_tokens=4 + i) for i, p in enumerate(prompts)]
        scheduler.run_until_complete()
        outputs.append([scheduler.finished[i].generated_token_ids for i in ids])
        assert all(len(tokens) == 4 + i for i, tokens in enumerate(outputs[-1]))
    assert all(out == outputs[0] for out in outputs)
    assert outputs[0] == [expected_tokens(p, 4 + i) for i, p in enumerate(prompts)]


def test_when_pages_run_out_requests_wait_in_order():
    # 6 pages of 4 tokens.  Each request reserves ceil((6 + 6) / 4) = 3 pages: two fit.
    engine = FakeEngine(pages=6, page_size=4)
    scheduler, _ = make(engine=engine, max_batch_size=8)
    ids = [scheduler.add_token_request([i + 1] * 6, max_new_tokens=6) for i in range(4)]
    scheduler.step()
    assert scheduler.reserved_blocks == [6]
    assert [rid for rid, _, _ in engine.steps[0]] == ids[:2]       # the third waits, and so does the fourth
    assert [r.request_id for r in scheduler.waiting] == ids[2:]
    small = scheduler.add_token_request([7], max_new_tokens=1)     # would fit, but may not overtake
    order = []
    while scheduler.has_work():
        before = set(scheduler.finished)
        scheduler.step()
        order.extend(sorted(set(scheduler.finished) - before))
        assert scheduler.reserved_blocks[0] <= 6
        engine.cache.check_invariants()
    assert order.index(small) > order.index(ids[2])
    assert scheduler.reserved_blocks == [0] and engine.cache.pools[0].num_free == 6
    for i, rid in enumerate(ids):
        assert scheduler.finished[rid].generated_token_ids == expected_tokens([i + 1] * 6, 6)
    # sarathi: the head of the queue waits likewise while decodes go on
    engine = FakeEngine(pages=6, page_size=4)
    scheduler, _ = make(SARATHI_STRATEGY, engine=engine, prefill_chunk_size=8)
    ids = [scheduler.add_token_request([i + 1] * 6, max_new_tokens=6) for i in range(3)]
    scheduler.run_until_complete()
    assert all(len(scheduler.finished[rid].generated_token_ids) == 6 for rid in ids)


def test_request_that_can_never_fit_is_refused_at_once():
    engine = FakeEngine(pages=3, page_size=4)
    scheduler, _ = make(engine=engine)
    with pytest.raises(ValueError, match="never be scheduled"):
        scheduler.add_token_request([1] * 10, max_new_tokens=5)
    assert not scheduler.waiting
    scheduler.add_token_request([1] * 6, max_new_tokens=6)          # exactly 3 pages
    scheduler.run_until_complete()


def test_request_validation():
    scheduler, _ = make()
    for bad in ([], [1, VOCAB], [-1], [1.5], [True]):
        with pytest.raises(ValueError):
            scheduler.add_token_request(bad, max_new_tokens=1)
    with pytest.raises(ValueError):
        scheduler.add_token_request([1], max_new_tokens=0)
    with pytest.raises(ValueError, match="context limit"):
        scheduler.add_token_request([1] * 100, max_new_tokens=29)   # 129 > 128
    scheduler.add_token_request([1] * 100, max_new_tokens=28)
    with pytest.raises(ValueError, match="tokenizer"):
        scheduler.add_request("hello")
    with pytest.raises(ValueError, match="strategy"):
        make("fifo")
    with pytest.raises(ValueError):
        make(max_batch_size=0)
    with pytest.raises(ValueError):
        make(max_batch_size=100)
    with pytest.raises(ValueError):
        make(max_num_batched_tokens=10 ** 6)


def test_end_token_stops_unless_ignored():
    class EosSampler:
        def sample(self, logits, params, keys, indices, seeds):
            return [VOCAB - 1 if index == 1 else 3 for index in indices]

    engine = FakeEngine()
    scheduler = ContinuousBatchScheduler(engine, EosSampler(), eos_token_id=VOCAB - 1, max_batch_size=8)
    a = scheduler.add_token_request([1, 2], max_new_tokens=5)
    b = scheduler.add_token_request([1, 2], max_new_tokens=5, sampling=SamplingParams(ignore_eos=True, max_new_tokens=5))
    scheduler.run_until_complete()
    assert scheduler.finished[a].generated_token_ids == [3, VOCAB - 1]
    assert scheduler.finished[a].finish_reason == "stop"
    assert len(scheduler.finished[b].generated_token_ids) == 5 and scheduler.finished[b].finish_reason == "length"
    assert not engine.cache.requests


def test_failed_step_unreserves_new_requests():
    scheduler, engine = make()
    a = scheduler.add_token_request([1, 2, 3], max_new_tokens=2)
    engine.fail_next = True
    with pytest.raises(RuntimeError, match="injected"):
        scheduler.step()
    # src/scheduler/orca_scheduler.py:243-247
    assert scheduler.reserved_blocks == [0] and scheduler.waiting[0].reserved_blocks == []
    scheduler.run_until_complete()
    assert scheduler.finished[a].generated_token_ids == expected_tokens([1, 2, 3], 2)


def test_window_group_reserves_less():
    engine = FakeEngine(pages=[40, 6], page_size=4, window=8, max_step_tokens=8)
    scheduler, _ = make(SARATHI_STRATEGY, engine=engine, prefill_chunk_size=8)
    rid = scheduler.add_token_request([2] * 60, max_new_tokens=20)
    assert scheduler._required_blocks(scheduler.waiting[0]) == [20, 5]
    scheduler.run_until_complete()
    assert len(scheduler.finished[rid].generated_token_ids) == 20
    assert engine.cache.pools[1].peak_allocated <= 5


@pytest.mark.parametrize("seed", range(5))
def test_random_arrivals_finish_with_exact_outputs(seed):
    rng = random.Random(seed)
    strategy = rng.choice([ORCA_STRATEGY, SARATHI_STRATEGY])
    engine = FakeEngine(pages=rng.choice([12, 20, 64]), page_size=4, max_requests=6, max_step_tokens=32)
    scheduler, _ = make(strategy, engine=engine, max_batch_size=rng.choice([2, 4, 6]),
                        prefill_chunk_size=rng.choice([1, 3, 8]), max_num_batched_tokens=rng.choice([8, 32]))
    expected = {}
    pending = 25
    while pending or scheduler.has_work():
        if pending and rng.random() < 0.5:
            prompt = [rng.randrange(VOCAB) for _ in range(rng.randint(1, 20))]
            count = rng.randint(1, 12)
            expected[scheduler.add_token_request(prompt, max_new_tokens=count)] = expected_tokens(prompt, count)
            pending -= 1
        if scheduler.has_work():
            scheduler.step()
    assert {rid: r.generated_token_ids for rid, r in scheduler.finished.items()} == expected
    assert scheduler.reserved_blocks == [0] and not engine.cache.requests


def test_uniform_numbers_are_a_function_of_seed_request_and_index():
    a = uniform_for(7, 3, 0)
    assert a == uniform_for(7, 3, 0) and 0.0 <= a < 1.0
    assert len({uniform_for(7, 3, i) for i in range(100)}) == 100
    assert uniform_for(7, 4, 0) != a and uniform_for(8, 3, 0) != a
    values = [uniform_for(1, r, i) for r in range(50) for i in range(200)]
    assert abs(sum(values) / len(values) - 0.5) < 0.01
    assert float(torch.tensor(values, dtype=torch.float32).max()) < 1.0
    with pytest.raises(ValueError):
        SamplingParams(temperature=-1)


class ChoosingEngine(FakeEngine):
    """The stand-in with what running ahead needs: it chooses tokens itself, hands them over
    only when asked (as a copy that is "on its way"), and resolves entries that carry on a
    row of the last step instead of a token id."""

    supports_draws = True

    def __init__(self, **kwargs):
        super().__init__(**kwargs)
        self.last_tokens = []
        self.outstanding = 0      # steps whose tokens nobody has read yet
        self.most_outstanding = 0

    def step(self, entries, greedy=False, draws=None):
        wanted = sum(len(entry.want) for entry in entries)
        assert greedy or draws is not None or not wanted
        for entry in entries:
            if entry.carry is not None:
                assert len(entry.tokens) == 1 and 0 <= entry.carry < len(self.last_tokens)
                entry.tokens = [self.last_tokens[entry.carry]]
        output = super().step(entries)
        if not wanted:
            self.last_tokens = []       # as the engine: nothing to carry on from this step
            return output
        tokens = output.logits.argmax(-1)
        self.last_tokens = tokens.tolist()
        self.outstanding += 1
        self.most_outstanding = max(self.most_outstanding, self.outstanding)
        engine = self

        class Ready:
            def synchronize(self_inner):
                engine.outstanding -= 1

        output.tokens = tokens
        output.host_tokens = tokens.clone()
        output.ready = Ready()
        return output


@pytest.mark.parametrize("run_ahead", [False, True])
def test_running_ahead_decisions(run_ahead):
    """The next iteration is launched before the last one's tokens are read: requests that end
    by length are left out of it, one that meets the end token gets its extra token dropped, a
    newcomer's prompt runs beside the tokens that are carried on.  Tokens and finish reasons
    are those of the step-by-step run."""
    end_token = expected_tokens([3, 1, 4], 9)[5]
    prompts = {"a": [3, 1, 4], "b": [2, 7], "c": [9, 9, 9, 9], "late": [5, 6]}
    budgets = {"a": 9, "b": 4, "c": 12, "late": 6}
    engine = ChoosingEngine()
    scheduler = ContinuousBatchScheduler(engine, ArgmaxSampler(), tokenizer=None, max_batch_size=8,
                                         eos_token_id=end_token, run_ahead=run_ahead)
    ids = {name: scheduler.add_token_request(prompts[name], budgets[name]) for name in ("a", "b", "c")}
    streamed = {}
    steps = 0
    while scheduler.has_work():
        if steps == 6:
            ids["late"] = scheduler.add_token_request(prompts["late"], budgets["late"])
        for rid, token in scheduler.step().items():
            streamed.setdefault(rid, []).append(token)
        steps += 1
    for name, rid in ids.items():
        free_run = expected_tokens(prompts[name], budgets[name])
        cut = free_run.index(end_token) + 1 if end_token in free_run else len(free_run)
        request = scheduler.finished[rid]
        assert request.generated_token_ids == free_run[:cut], name
        assert streamed[rid] == free_run[:cut]
        assert request.finish_reason == ("stop" if cut < len(free_run) or free_run[-1] == end_token else "length")
    assert scheduler.finished[ids["a"]].finish_reason == "stop"      # the end token really came
    assert not engine.cache.requests and scheduler.reserved_blocks == [0]
    if run_ahead:
        assert scheduler.steps_run_ahead >= 5 and engine.most_outstanding == 2
        # no step carried a request on after its last token by length
        for step in engine.steps:
            assert len(step) <= 4
    else:
        assert scheduler.steps_run_ahead == 0 and engine.most_outstanding == 1


def _burst(run_ahead, strategy, seed, end_token=None):
    """A burst of requests on so few pages that newcomers wait for others to end, fewer turns
    than decoding requests, prompts cut into portions: (scheduler, engine, expected tokens)."""
    rng = random.Random(seed)
    engine = ChoosingEngine(pages=rng.choice([14, 24]), page_size=4, max_requests=6, max_step_tokens=32)
    scheduler = ContinuousBatchScheduler(
        engine, ArgmaxSampler(), tokenizer=None, scheduling_strategy=strategy,
        max_batch_size=rng.choice([3, 6]), prefill_chunk_size=rng.choice([2, 5, 16]),
        max_num_batched_tokens=rng.choice([8, 32]), max_prefill_requests=rng.choice([1, 3]),
        eos_token_id=end_token, run_ahead=run_ahead)
    expected = {}
    for _ in range(14):
        prompt = [rng.randrange(VOCAB - 1) for _ in range(rng.randint(1, 20))]
        count = rng.randint(1, 12)
        free_run = expected_tokens(prompt, count)
        cut = free_run.index(end_token) + 1 if end_token in free_run else count
        expected[scheduler.add_token_request(prompt, max_new_tokens=count)] = free_run[:cut]
    return scheduler, engine, expected


@pytest.mark.parametrize("strategy", [ORCA_STRATEGY, SARATHI_STRATEGY])
@pytest.mark.parametrize("seed", range(6))
def test_running_ahead_changes_no_iteration(strategy, seed):
    """With nothing ending at an end token, everything that decides an iteration's work is
    known before the tokens of the one before it are: launched ahead or not, the engine sees
    the same steps with the same tokens (prompt portions, turns, newcomers that take the
    pages of requests that have just ended by length), and every step but the first is
    launched while its predecessor's tokens are still on their way."""
    runs = {}
    for run_ahead in (False, True):
        scheduler, engine, expected = _burst(run_ahead, strategy, seed)
        streamed = {}
        while scheduler.has_work():
            for rid, token in scheduler.step().items():
                streamed.setdefault(rid, []).append(token)
            engine.cache.check_invariants()
        assert streamed == expected
        assert {rid: r.generated_token_ids for rid, r in scheduler.finished.items()} == expected
        assert all(r.finish_reason == "length" for r in scheduler.finished.values())
        assert scheduler.reserved_blocks == [0] and not engine.cache.requests
        runs[run_ahead] = (engine.steps, scheduler.iterations)
        if run_ahead:
            assert scheduler.steps_run_ahead == len(engine.steps) - 1
            assert engine.most_outstanding == 2
        else:
            assert scheduler.steps_run_ahead == 0 and engine.most_outstanding == 1
    assert runs[True] == runs[False]
    assert any(len(tokens) > 1 for step in runs[True][0][1:] for _, tokens, _ in step)   # prompts ran ahead too


@pytest.mark.parametrize("strategy", [ORCA_STRATEGY, SARATHI_STRATEGY])
@pytest.mark.parametrize("seed", range(6))
def test_running_ahead_with_end_tokens(strategy, seed):
    """A request that meets the end token is known to have ended one iteration late: the
    token computed for it meanwhile is dropped, its pages go back then, and every request
    still receives exactly the tokens of the step-by-step run."""
    free_runs = _burst(False, strategy, seed)[2]
    # the token that cuts the most requests short
    end_token = Counter(token for run in free_runs.values() for token in set(run[:-1])).most_common(1)[0][0]
    ended_early = 0
    for run_ahead in (False, True):
        scheduler, engine, expected = _burst(run_ahead, strategy, seed, end_token=end_token)
        streamed = {}
        while scheduler.has_work():
            for rid, token in scheduler.step().items():
                streamed.setdefault(rid, []).append(token)
            engine.cache.check_invariants()
        assert streamed == expected
        assert {rid: r.generated_token_ids for rid, r in scheduler.finished.items()} == expected
        for rid, request in scheduler.finished.items():
            stopped = expected[rid][-1] == end_token
            assert request.finish_reason == ("stop" if stopped else "length")
            ended_early += stopped and len(expected[rid]) < request.max_new_tokens
        assert scheduler.reserved_blocks == [0] and not engine.cache.requests
    assert ended_early >= 2


def test_arrivals_while_running_ahead():
    """Requests that arrive between iterations join the next one that is chosen, beside tokens
    that are carried on; outputs are exact."""
    for seed in range(5):
        rng = random.Random(100 + seed)
        engine = ChoosingEngine(pages=rng.choice([12, 20, 64]), page_size=4, max_requests=6, max_step_tokens=32)
        scheduler = ContinuousBatchScheduler(
            engine, ArgmaxSampler(), tokenizer=None,
            scheduling_strategy=rng.choice([ORCA_STRATEGY, SARATHI_STRATEGY]),
            max_batch_size=rng.choice([2, 4, 6]), prefill_chunk_size=rng.choice([1, 3, 8]),
            max_num_batched_tokens=rng.choice([8, 32]), eos_token_id=None)
        expected = {}
        pending = 25
        while pending or scheduler.has_work():
            if pending and rng.random() < 0.5:
                prompt = [rng.randrange(VOCAB) for _ in range(rng.randint(1, 20))]
                count = rng.randint(1, 12)
                expected[scheduler.add_token_request(prompt, max_new_tokens=count)] = expected_tokens(prompt, count)
                pending -= 1
            if scheduler.has_work():
                scheduler.step()
        assert {rid: r.generated_token_ids for rid, r in scheduler.finished.items()} == expected
        assert scheduler.reserved_blocks == [0] and not engine.cache.requests
        assert scheduler.steps_run_ahead > scheduler.iterations // 2 and engine.most_outstanding == 2


@pytest.mark.parametrize("strategy", [ORCA_STRATEGY, SARATHI_STRATEGY])
def test_decoding_requests_beyond_the_limit_take_turns(strategy):
    """Six decoding requests, four per iteration: each is served in two of every three
    iterations, none waits for another to finish (the reference always takes the lowest ids,
    src/scheduler/orca_scheduler.py:165-166)."""
    engine = FakeEngine(max_requests=8)
    scheduler, _ = make(strategy, engine=engine, max_batch_size=6, prefill_chunk_size=8,
                        max_prefill_requests=6)
    ids = [scheduler.add_token_request([i + 1, i + 2], max_new_tokens=13) for i in range(6)]
    while scheduler.waiting:
        scheduler.step()
    scheduler.max_batch_size = 4
    served = {rid: 0 for rid in ids}
    for _ in range(9):
        step_ids = list(scheduler.step())
        assert len(step_ids) == 4
        for rid in step_ids:
            served[rid] += 1
        # entries stay in arrival order
        assert [rid for rid, _, _ in engine.steps[-1]] == sorted(step_ids)
    assert set(served.values()) == {6}
    scheduler.run_until_complete()
    for i, rid in enumerate(ids):
        assert scheduler.finished[rid].generated_token_ids == expected_tokens([i + 1, i + 2], 13)


def test_no_end_token_can_be_said():
    """``eos_token_id=None`` means that no token ends a request, whatever the tokenizer's end
    token is; leaving the argument out takes the tokenizer's."""
    class EndSampler:
        def sample(self, logits, params, keys, indices, seeds):
            return [VOCAB - 1 for _ in indices]

    tokenizer = SimpleNamespace(eos_token_id=VOCAB - 1, encode=lambda text: [1], decode=lambda ids: "")
    scheduler = ContinuousBatchScheduler(FakeEngine(), EndSampler(), tokenizer=tokenizer,
                                         eos_token_id=None, max_batch_size=8)
    rid = scheduler.add_token_request([1, 2], max_new_tokens=4)
    scheduler.run_until_complete()
    assert scheduler.finished[rid].generated_token_ids == [VOCAB - 1] * 4
    assert scheduler.finished[rid].finish_reason == "length"
    scheduler = ContinuousBatchScheduler(FakeEngine(), EndSampler(), tokenizer=tokenizer, max_batch_size=8)
    rid = scheduler.add_token_request([1, 2], max_new_tokens=4)
    scheduler.run_until_complete()
    assert scheduler.finished[rid].finish_reason == "stop"
    assert scheduler.finished[rid].generated_token_ids == [VOCAB - 1]


def test_arrival_trace_runner_times_requests_by_its_clock():
    """Requests are submitted when their time has come (not before), every token gets the time
    at which its iteration ended, and TTFT / TPOT follow comparison_benchmark.py:444-472."""
    from pagedserve_amd.engine.workload import (TraceRequest, arrival_times, percentile,
                                                 run_arrival_trace, summarize)

    offsets = arrival_times(5, 4.0, "poisson", seed=3)
    assert offsets[0] == 0.0 and offsets == sorted(offsets) and len(offsets) == 5
    assert offsets == arrival_times(5, 4.0, "poisson", seed=3) != arrival_times(5, 4.0, "poisson", seed=4)
    # the mean gap of many draws is 1 / rate
    many = arrival_times(4001, 50.0, "poisson", seed=1)
    assert abs(many[-1] / 4000 - 1 / 50.0) < 0.002
    assert arrival_times(3, 2.0, "even") == [0.0, 0.5, 1.0]
    assert arrival_times(3, float("inf")) == [0.0, 0.0, 0.0] == arrival_times(3, process="burst")
    assert arrival_times(0, 1.0) == []
    with pytest.raises(ValueError):
        arrival_times(3, 0.0)
    with pytest.raises(ValueError):
        arrival_times(3, 1.0, "bursty")
    assert percentile([1, 2, 3, 4], 50) == 2.5 and percentile([5], 99) == 5
    spread = summarize(range(101))
    assert (spread["p50"], spread["p95"], spread["p99"], spread["max"]) == (50, 95, 99, 100)

    class Clock:
        now = 0.0

        def __call__(self):
            return self.now

    clock = Clock()
    scheduler, engine = make(max_batch_size=8)
    plain_step = scheduler.step

    def timed_step():
        clock.now += 0.25          # every iteration takes a quarter of a second
        return plain_step()

    scheduler.step = timed_step

    def idle(seconds):
        clock.now += max(seconds, 1e-3)

    requests = [TraceRequest([1, 2, 3], 3), TraceRequest([4, 5], 2), TraceRequest([6], 4)]
    offsets = [0.0, 0.6, 5.0]
    summary = run_arrival_trace(scheduler, requests, offsets, clock=clock, idle=idle)
    records = summary["records"]
    assert summary["completed"] == 3 and summary["output_tokens"] == 9 and summary["prompt_tokens"] == 6
    # the first request: tokens at 0.25, 0.5, 0.75
    assert records[0].token_times == pytest.approx([0.25, 0.5, 0.75])
    assert records[0].metrics()["ttft"] == pytest.approx(0.25) and records[0].metrics()["tpot"] == pytest.approx(0.25)
    # the second arrives at 0.6, is seen at 0.75, its first token comes at 1.0
    assert records[1].submitted_at == pytest.approx(0.75)
    assert records[1].metrics()["ttft"] == pytest.approx(1.0 - 0.6)
    assert records[1].metrics()["queue_delay"] == pytest.approx(0.15)
    # the third waits for its time while nothing runs
    assert 5.0 <= records[2].submitted_at < 5.01 and len(records[2].token_times) == 4
    assert summary["wall_seconds"] == pytest.approx(records[2].token_times[-1])
    assert summary["ttft_seconds"]["max"] == pytest.approx(0.4)
    for index, request in enumerate(requests):
        assert scheduler.finished[records[index].request_id].generated_token_ids == \
            expected_tokens(list(request.prompt_token_ids), request.max_new_tokens)


def test_command_line_takes_the_reference_options(capsys):
    """Option names of the reference's main.py:257-342; its two backend options are accepted as
    far as they mean something here."""
    import os
    import sys

    sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    import main

    args = main.parse_args(["--model", "reference", "--strategy", "sarathi", "--prefill-chunk-size", "32",
                            "--max-batch-size", "4", "--kv-cache-memory-mb", "64",
                            "--kv-cache-memory-utilization", "0.5", "--kv-cache-safety-mb", "128",
                            "--dtype", "bfloat16", "--decode-attention-backend", "hip",
                            "--kv-cache-dtype", "model", "--disable-cuda-graphs"])
    assert args.strategy == "sarathi" and args.prefill_chunk_size == 32 and args.max_batch_size == 4
    assert args.kv_cache_memory_mb == 64 and args.disable_hip_graphs and args.dtype == "bfloat16"
    # a backend that is not built is an error that names the one that is, not a silent alias
    with pytest.raises(SystemExit):
        main.parse_args(["--decode-attention-backend", "triton"])
    assert "'hip'" in capsys.readouterr().err
    with pytest.raises(SystemExit):
        main.parse_args(["--kv-cache-dtype", "int8"])
    assert "quantized caches are not built" in capsys.readouterr().err
    with pytest.raises(SystemExit):
        main.parse_args(["--decode-attention-backend", "flash"])


def test_python_entry_takes_the_reference_keyword_names():
    """build_scheduler(model_name=..., enable_cuda_graphs=..., decode_attention_backend=...,
    kv_cache_dtype=...) of the reference's main.py:136-150; what cannot be had is refused
    before anything is loaded."""
    from pagedserve_amd.engine.llm import build_scheduler

    with pytest.raises(ValueError, match="quantized caches are not built"):
        build_scheduler(model_name="reference", kv_cache_dtype="int8")
    for backend in ("flash", "torch", "triton"):
        with pytest.raises(ValueError, match="Unknown decode attention backend.*'hip'"):
            build_scheduler(model_name="reference", decode_attention_backend=backend)


def test_a_failing_step_ahead_loses_no_tokens():
    """The iteration that is launched ahead fails with an error that is no refusal (a kernel's,
    say): the iteration that was already running still lands, its tokens reach the caller, the
    error comes out of the next call, and the loop goes on from there as if nothing had been
    launched ahead."""

    class BreaksOnce(ChoosingEngine):
        def __init__(self):
            super().__init__()
            self.broken = False

        def step(self, entries, greedy=False, draws=None):
            if not self.broken and any(entry.carry is not None for entry in entries):
                self.broken = True
                raise RuntimeError("a launch failed")
            return super().step(entries, greedy=greedy, draws=draws)

    engine = BreaksOnce()
    scheduler = ContinuousBatchScheduler(engine, ArgmaxSampler(), tokenizer=None, max_batch_size=4,
                                         eos_token_id=None)
    first = scheduler.add_token_request([3, 1, 4], 6)
    second = scheduler.add_token_request([2, 7], 6)
    streamed = {first: [], second: []}
    raised = 0
    while scheduler.has_work():
        try:
            for rid, token in scheduler.step().items():
                streamed[rid].append(token)
        except RuntimeError as error:
            assert "a launch failed" in str(error)
            raised += 1
    assert raised == 1 and engine.broken
    assert streamed[first] == expected_tokens([3, 1, 4], 6) == scheduler.finished[first].generated_token_ids
    assert streamed[second] == expected_tokens([2, 7], 6) == scheduler.finished[second].generated_token_ids
    assert not engine.cache.requests
