"""Generation through the entry points, long decoding, the first tokens of a sequence,
sampling, and the command line."""

import os
import subprocess
import sys

import pytest
import torch

import helpers
import plain_gpt2

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    base = tmp_path_factory.mktemp("gen_models")
    return {which: helpers.tiny_folder(base, which) for which in ("A", "B")}


# the tiny workloads: A: prompts 5, 17, 31 -> 16 tokens; B: 1, 9, 40, 64, 100 -> 24 tokens,
# portions of 32, mixed batches
WORKLOADS = {"A": ([5, 17, 31], 16, dict(scheduling_strategy="orca")),
             "B": ([1, 9, 40, 64, 100], 24, dict(scheduling_strategy="sarathi", prefill_chunk_size=32,
                                                max_prefill_requests=2))}


@pytest.mark.parametrize("which", ["A", "B"])
def test_greedy_generation_matches_plain(folders, which):
    from pagedserve_amd.engine.llm import LLM
    from pagedserve_amd.sampling import SamplingParams

    folder, config, page_size = folders[which]
    lengths, new_tokens, options = WORKLOADS[which]
    prompts = [helpers.random_tokens(n, config["vocab_size"], 300 + i) for i, n in enumerate(lengths)]
    raw, weights = plain_gpt2.read_model_folder(folder)
    expected = [plain_gpt2.greedy_generate(raw, weights, prompt, new_tokens) for prompt in prompts]
    llm = LLM(folder, dtype="float32", block_size=page_size, num_kv_pages=40, max_batch_size=4,
              eos_token_id=None, **options)
    outputs = llm.generate(prompts, SamplingParams(max_new_tokens=new_tokens))
    assert [o.token_ids for o in outputs] == expected
    assert all(o.finish_reason == "length" for o in outputs)
    llm.engine.cache.check_invariants()
    assert not llm.engine.cache.requests
    # bfloat16 runs the same workload; its tokens follow the rounded model closely
    llm16 = LLM(folder, dtype="bfloat16", block_size=page_size, num_kv_pages=40, max_batch_size=4,
                eos_token_id=None, **options)
    outputs16 = llm16.generate(prompts, SamplingParams(max_new_tokens=new_tokens))
    first = [o.token_ids[0] for o in outputs16]
    assert sum(a == e[0] for a, e in zip(first, expected)) >= len(prompts) - 1


def test_running_ahead_gives_the_same_tokens_and_stops_at_the_end_token(folders):
    """Iterations launched before the last one's tokens reached the host change nothing: with
    an end token that some requests meet on the way and different lengths, every request gets
    the tokens of the step-by-step run, and the extra token computed for a request that has
    just ended is dropped."""
    from pagedserve_amd.engine import ContinuousBatchScheduler, Engine
    from pagedserve_amd.model import load_model
    from pagedserve_amd.sampling import Sampler, SamplingParams

    folder, config, page_size = folders["A"]
    prompts = [helpers.random_tokens(n, config["vocab_size"], 900 + i) for i, n in enumerate([5, 9, 17, 3])]
    budgets = [40, 23, 31, 12]
    raw, weights = plain_gpt2.read_model_folder(folder)
    free_run = [plain_gpt2.greedy_generate(raw, weights, prompt, budget) for prompt, budget in zip(prompts, budgets)]
    # an end token that the first request produces somewhere in the middle
    end_token = free_run[0][len(free_run[0]) // 2]
    expected = []
    for tokens in free_run:
        cut = tokens.index(end_token) + 1 if end_token in tokens else len(tokens)
        expected.append(tokens[:cut])
    assert any(len(e) < len(f) for e, f in zip(expected, free_run))
    model, _ = load_model(folder, dtype="float32")
    results = {}
    for run_ahead in (False, True):
        engine = Engine(model, num_pages=64, page_size=page_size, max_requests=4, max_step_tokens=64)
        scheduler = ContinuousBatchScheduler(engine, Sampler(engine.device, 4), max_batch_size=4,
                                             eos_token_id=end_token, run_ahead=run_ahead)
        ids = [scheduler.add_token_request(prompt, budget, sampling=SamplingParams(max_new_tokens=budget))
               for prompt, budget in zip(prompts, budgets)]
        streamed = {rid: [] for rid in ids}
        while scheduler.has_work():
            for rid, token in scheduler.step().items():
                streamed[rid].append(token)
        got = [scheduler.finished[rid].generated_token_ids for rid in ids]
        assert got == expected, run_ahead
        assert [streamed[rid] for rid in ids] == expected
        reasons = [scheduler.finished[rid].finish_reason for rid in ids]
        assert reasons == ["stop" if e[-1] == end_token else "length" for e in expected]
        engine.cache.check_invariants()
        assert not engine.cache.requests and scheduler.reserved_blocks == [0]
        results[run_ahead] = scheduler.steps_run_ahead
    assert results[False] == 0 and results[True] > 10


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_running_ahead_beside_prompt_portions(folders, dtype):
    """Iterations that hold prompt portions are launched ahead too: decoded tokens are carried
    on from the device beside the portions, requests that end by length give their pages to
    newcomers before their last token has reached the host (so few pages that newcomers wait
    for them), late arrivals join.  Every request gets the plain implementation's greedy tokens
    (32-bit), and the tokens of the step-by-step run (both)."""
    from pagedserve_amd.engine import ContinuousBatchScheduler, Engine
    from pagedserve_amd.model import load_model
    from pagedserve_amd.sampling import Sampler, SamplingParams

    folder, config, page_size = folders["A"]
    lengths = [33, 5, 50, 17, 40, 9, 26]
    budgets = [20, 35, 12, 28, 16, 30, 1]
    prompts = [helpers.random_tokens(n, config["vocab_size"], 700 + i) for i, n in enumerate(lengths)]
    model, _ = load_model(folder, dtype=dtype)
    results = {}
    for run_ahead in (False, True):
        engine = Engine(model, num_pages=22, page_size=page_size, max_requests=4, max_step_tokens=32)
        scheduler = ContinuousBatchScheduler(engine, Sampler(engine.device, 4), max_batch_size=4,
                                             eos_token_id=None, run_ahead=run_ahead,
                                             scheduling_strategy="sarathi", prefill_chunk_size=11,
                                             max_num_batched_tokens=24, max_prefill_requests=2)
        ids = []
        steps = 0
        while len(ids) < len(prompts) or scheduler.has_work():
            # 32-bit: four at once, then one every fifth iteration; bfloat16: all at once, so
            # that both runs make the same iterations and rounding cannot tell them apart
            while len(ids) < len(prompts) and (dtype == "bfloat16" or len(ids) < 4
                                               or steps >= 5 * (len(ids) - 3)):
                ids.append(scheduler.add_token_request(
                    prompts[len(ids)], budgets[len(ids)],
                    sampling=SamplingParams(max_new_tokens=budgets[len(ids)])))
            scheduler.step()
            steps += 1
            engine.cache.check_invariants()
        results[run_ahead] = [scheduler.finished[rid].generated_token_ids for rid in ids]
        assert [len(tokens) for tokens in results[run_ahead]] == budgets
        assert not engine.cache.requests and scheduler.reserved_blocks == [0]
        if run_ahead:
            # all but the iterations after which nothing was left to choose
            assert scheduler.steps_run_ahead > 0.9 * scheduler.iterations
        else:
            assert scheduler.steps_run_ahead == 0
    assert results[True] == results[False]
    if dtype == "float32":
        raw, weights = plain_gpt2.read_model_folder(folder)
        for prompt, budget, tokens in zip(prompts, budgets, results[True]):
            assert tokens == plain_gpt2.greedy_generate(raw, weights, prompt, budget)


def test_running_ahead_with_temperature_draws_the_same_tokens(folders):
    """Drawn tokens (seeded) are the same whether the host's sampler picks them from the
    logits after each step, the step picks them on the device, or steps run ahead, under
    Orca's whole prompts as under Sarathi's portions beside decoded tokens."""
    from pagedserve_amd.engine import ContinuousBatchScheduler, Engine
    from pagedserve_amd.model import load_model
    from pagedserve_amd.sampling import Sampler, SamplingParams

    folder, config, page_size = folders["B"]
    prompts = [helpers.random_tokens(n, config["vocab_size"], 950 + i) for i, n in enumerate([4, 21, 9])]
    budgets = [30, 18, 25]
    temperatures = [6.0, 0.0, 12.0]
    model, _ = load_model(folder, dtype="float32")
    results = []
    for on_device, run_ahead, strategy in ((False, False, "orca"), (True, False, "orca"), (True, True, "orca"),
                                          (True, True, "sarathi"), (False, False, "sarathi")):
        engine = Engine(model, num_pages=32, page_size=page_size, max_requests=4, max_step_tokens=64)
        engine.supports_draws = on_device
        scheduler = ContinuousBatchScheduler(engine, Sampler(engine.device, 4), max_batch_size=4,
                                             eos_token_id=None, run_ahead=run_ahead,
                                             scheduling_strategy=strategy, prefill_chunk_size=5,
                                             max_prefill_requests=2)
        ids = [scheduler.add_token_request(prompt, budget, sampling=SamplingParams(
                   max_new_tokens=budget, temperature=temperature, seed=11 + i))
               for i, (prompt, budget, temperature) in enumerate(zip(prompts, budgets, temperatures))]
        scheduler.run_until_complete()
        results.append([scheduler.finished[rid].generated_token_ids for rid in ids])
        assert [len(tokens) for tokens in results[-1]] == budgets
        if run_ahead:
            assert scheduler.steps_run_ahead > 10
        engine.cache.check_invariants()
    assert all(result == results[0] for result in results)
    # the draws are no argmax in disguise
    raw, weights = plain_gpt2.read_model_folder(folder)
    assert results[0][0] != plain_gpt2.greedy_generate(raw, weights, prompts[0], budgets[0])
    assert results[0][1] == plain_gpt2.greedy_generate(raw, weights, prompts[1], budgets[1])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(folders, dtype):
    """Two prompt tokens, then 250 tokens decoded one by one up to the last position."""
    from pagedserve_amd.engine import Engine, StepEntry
    from pagedserve_amd.model import load_model

    folder, config, page_size = folders["B"]
    tokens = helpers.random_tokens(config["n_positions"], config["vocab_size"], 400)
    reference = helpers.plain_logits(folder, tokens, bfloat16=dtype == "bfloat16")
    model, _ = load_model(folder, dtype=dtype)
    engine = Engine(model, num_pages=config["n_positions"] // page_size, page_size=page_size,
                    max_requests=2, max_step_tokens=64)
    rows = {}
    out = engine.step([StepEntry("r", tokens[:2], [0, 1])])
    rows[0], rows[1] = out.logits[0].double().cpu(), out.logits[1].double().cpu()
    for position in range(2, len(tokens)):
        out = engine.step([StepEntry("r", [tokens[position]], [0])])
        rows[position] = out.logits[0].double().cpu()
    error = max(float((rows[p] - reference[p]).abs().max()) for p in rows)
    scale = float(reference.abs().max())
    assert error <= helpers.TOLERANCE[dtype] * scale, (error, scale)
    from pagedserve_amd.engine import StepError
    with pytest.raises(StepError, match="position"):
        engine.step([StepEntry("r", [1], [0])])          # the position table is exhausted


LONG = {
    "architectures": ["GPT2LMHeadModel"], "model_type": "gpt2",
    "n_layer": 2, "n_embd": 128, "n_head": 2, "n_inner": 192, "vocab_size": 97,
    "n_positions": 3072, "layer_norm_epsilon": 1e-5, "activation_function": "gelu_new",
    "scale_attn_by_inverse_layer_idx": False, "tie_word_embeddings": True, "eos_token_id": None,
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decoding_over_long_contexts(tmp_path, dtype, monkeypatch):
    """Contexts of 2,900 and 1,500 tokens (heads of 64): prompts in portions, then tokens
    decoded one by one, first for one request, then for both together.  With so many keys per
    request the decode kernel cuts them into more than twenty ranges, which in bfloat16 the
    output projection merges with the ranges of a row shared among its lanes."""
    from pagedserve_amd.engine import Engine, StepEntry
    from pagedserve_amd.model import load_model
    from pagedserve_amd.ops import kernels

    merged = []
    merge = kernels.attention_merge_linear

    def recording(partial, count, heads, head_dim, splits, *args, **kwargs):
        merged.append((count, splits))
        return merge(partial, count, heads, head_dim, splits, *args, **kwargs)

    monkeypatch.setattr(kernels, "attention_merge_linear", recording)
    folder = helpers.write_folder(os.path.join(str(tmp_path), "long"), LONG, helpers.lively_tensors(LONG, 9))
    lengths = {"far": 2900, "near": 1500}
    decoded = 24
    tokens = {name: helpers.random_tokens(n + decoded, LONG["vocab_size"], 520 + i)
              for i, (name, n) in enumerate(lengths.items())}
    reference = {name: helpers.plain_logits(folder, tokens[name], bfloat16=dtype == "bfloat16") for name in tokens}
    model, _ = load_model(folder, dtype=dtype)
    engine = Engine(model, num_pages=(2900 + 1500 + 2 * decoded) // 16 + 4, page_size=16, max_requests=2,
                    max_step_tokens=1024)
    worst = 0.0

    def check(out, places):
        nonlocal worst
        values = out.logits.double().cpu()
        for row, (name, position) in enumerate(places):
            worst = max(worst, float((values[row] - reference[name][position]).abs().max()))

    for name, length in lengths.items():
        for begin in range(0, length, 1024):
            part = tokens[name][begin:min(begin + 1024, length)]
            last = begin + len(part) == length
            out = engine.step([StepEntry(name, part, [len(part) - 1] if last else [])])
            if last:
                check(out, [(name, length - 1)])
    held = dict(lengths)
    for step in range(decoded):
        names = ["far"] if step < 8 else ["far", "near"]
        out = engine.step([StepEntry(name, [tokens[name][held[name]]], [0]) for name in names])
        check(out, [(name, held[name]) for name in names])
        for name in names:
            held[name] += 1
    scale = max(float(reference[name].abs().max()) for name in reference)
    assert worst <= helpers.TOLERANCE[dtype] * scale, (worst, scale)
    engine.cache.check_invariants()
    if dtype == "bfloat16":
        # (launches that were recorded into graphs are counted once)
        assert {count for count, _ in merged} == {1, 2} and min(splits for _, splits in merged) > 8, merged
    else:
        assert not merged


MANY_HEADS = {
    "architectures": ["GPT2LMHeadModel"], "model_type": "gpt2",
    "n_layer": 1, "n_embd": 96, "n_head": 12, "n_inner": 160, "vocab_size": 83,
    "n_positions": 2200, "layer_norm_epsilon": 1e-5, "activation_function": "gelu_new",
    "scale_attn_by_inverse_layer_idx": False, "tie_word_embeddings": True, "eos_token_id": None,
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("live,shortest,cut", [(20, 530, False), (24, 530, True), (30, 530, True), (34, 530, False),
                                               (34, 2060, True)])
def test_decoding_many_requests_over_hundreds_of_keys(tmp_path, dtype, live, shortest, cut, monkeypatch):
    """20 to 34 requests of 12 heads decode together at contexts of 530 to 600 tokens: between
    one and one and a half (token, head) pairs per compute unit the decode kernel cuts every
    request's keys into ranges (blocks of 4 waves) and a second launch merges them; below and
    above it does not, unless the contexts are long (2,060 to 2,130 tokens here).  The weights
    make attention far from uniform, so a range that is skipped or merged with a wrong weight
    shows in the logits."""
    from pagedserve_amd.engine import Engine, StepEntry
    from pagedserve_amd.model import load_model
    from pagedserve_amd.ops import kernels

    launches = []
    real = kernels.attention_decode

    def recording(*args, **kwargs):
        launches.append((int(args[9]), kwargs.get("waves", 4)))
        return real(*args, **kwargs)

    monkeypatch.setattr(kernels, "attention_decode", recording)
    folder = helpers.write_folder(os.path.join(str(tmp_path), "many"), MANY_HEADS,
                                  helpers.lively_tensors(MANY_HEADS, 31))
    decoded = 3
    lengths = {f"q{i}": shortest + (7 * i) % 70 for i in range(live)}
    tokens = {name: helpers.random_tokens(n + decoded, MANY_HEADS["vocab_size"], 900 + i)
              for i, (name, n) in enumerate(lengths.items())}
    checked = list(lengths)[:3] + list(lengths)[-2:]
    reference = {name: helpers.plain_logits(folder, tokens[name], bfloat16=dtype == "bfloat16") for name in checked}
    model, _ = load_model(folder, dtype=dtype)
    pages = sum(-(-(n + decoded) // 16) for n in lengths.values()) + 2
    engine = Engine(model, num_pages=pages, page_size=16, max_requests=live, max_step_tokens=2200)
    for name, length in lengths.items():
        engine.step([StepEntry(name, tokens[name][:length], [])])
    worst = 0.0
    held = dict(lengths)
    for step in range(decoded):
        out = engine.step([StepEntry(name, [tokens[name][held[name]]], [0]) for name in lengths])
        values = out.logits.double().cpu()
        for row, name in enumerate(lengths):
            if name in reference:
                worst = max(worst, float((values[row] - reference[name][held[name]]).abs().max()))
            held[name] += 1
    scale = max(float(reference[name].abs().max()) for name in reference)
    assert worst <= helpers.TOLERANCE[dtype] * scale, (worst, scale)
    engine.cache.check_invariants()
    assert kernels.compute_units() == 256, "the cases above are chosen for 256 compute units"
    assert {splits > 1 for splits, _ in launches} == {cut}, launches


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_first_tokens_of_a_sequence(folders, dtype):
    """Positions 0, 1, 2 in every arrangement: alone, one by one, and beside another request."""
    from pagedserve_amd.engine import Engine, StepEntry
    from pagedserve_amd.model import load_model

    folder, config, page_size = folders["A"]
    tokens = helpers.random_tokens(3, config["vocab_size"], 410)
    other = helpers.random_tokens(11, config["vocab_size"], 411)
    reference = helpers.plain_logits(folder, tokens, bfloat16=dtype == "bfloat16")
    model, _ = load_model(folder, dtype=dtype)
    engine = Engine(model, num_pages=8, page_size=page_size, max_requests=4, max_step_tokens=32)
    tolerance = helpers.TOLERANCE[dtype] * float(reference.abs().max())
    whole = engine.step([StepEntry("a", tokens, [0, 1, 2])]).logits.double().cpu()
    assert float((whole - reference).abs().max()) <= tolerance
    for position in range(3):
        entries = [StepEntry("b", [tokens[position]], [0])]
        if position == 1:
            entries.insert(0, StepEntry("c", other, [10]))
        got = engine.step(entries).logits[-1].double().cpu()
        assert float((got - reference[position]).abs().max()) <= tolerance
    single = engine.step([StepEntry("d", tokens[:1], [0])]).logits[0].double().cpu()
    assert float((single - reference[0]).abs().max()) <= tolerance


def test_step_refuses_what_it_cannot_run(folders):
    from pagedserve_amd.cache import CacheFull
    from pagedserve_amd.engine import Engine, StepEntry, StepError
    from pagedserve_amd.model import load_model

    folder, config, page_size = folders["A"]
    model, _ = load_model(folder, dtype="float32")
    engine = Engine(model, num_pages=4, page_size=page_size, max_requests=2, max_step_tokens=16)
    with pytest.raises(StepError, match="at least one"):
        engine.step([])
    with pytest.raises(StepError, match="twice"):
        engine.step([StepEntry("a", [1], []), StepEntry("a", [2], [])])
    with pytest.raises(StepError, match="vocabulary"):
        engine.step([StepEntry("a", [config["vocab_size"]], [])])
    with pytest.raises(StepError, match="place"):
        engine.step([StepEntry("a", [1, 2], [2])])
    with pytest.raises(StepError, match="max_step_tokens"):
        engine.step([StepEntry("a", [1] * 17, [])])
    with pytest.raises(StepError, match="live requests"):
        engine.step([StepEntry("a", [1], []), StepEntry("b", [1], []), StepEntry("c", [1], [])])
    engine.step([StepEntry("a", [1] * 16, [])])
    engine.step([StepEntry("a", [1] * 16, [])])
    with pytest.raises(CacheFull):
        engine.step([StepEntry("b", [1], [0])])            # all four pages are held by "a"
    assert not engine.is_live("b")                          # a refused newcomer leaves no trace
    engine.cache.check_invariants()
    engine.finish("a")
    assert engine.step([StepEntry("b", [1], [0])]).logits.shape == (1, config["vocab_size"])


def test_temperature_sampling_is_reproducible_and_batch_independent(folders):
    from pagedserve_amd.engine.llm import LLM
    from pagedserve_amd.sampling import SamplingParams, uniform_for

    folder, config, page_size = folders["A"]
    prompts = [helpers.random_tokens(n, config["vocab_size"], 500 + n) for n in (4, 9, 13)]
    params = SamplingParams(temperature=0.8, seed=7, max_new_tokens=12)
    kwargs = dict(dtype="float32", block_size=page_size, num_kv_pages=32, max_batch_size=4, eos_token_id=None)
    together = [o.token_ids for o in LLM(folder, **kwargs).generate(prompts, params)]
    again = [o.token_ids for o in LLM(folder, **kwargs).generate(prompts, params)]
    assert together == again
    # request ids are part of the key: the same prompts alone, as request 0, 1, 2 of their own engines
    alone = LLM(folder, scheduling_strategy="sarathi", prefill_chunk_size=3, **kwargs)
    assert [o.token_ids for o in alone.generate(prompts, params)] == together
    other_seed = [o.token_ids for o in LLM(folder, **kwargs).generate(
        prompts, SamplingParams(temperature=0.8, seed=8, max_new_tokens=12))]
    assert other_seed != together
    # each drawn token is the inverse-CDF point of the plain model's distribution at the same uniform number
    raw, weights = plain_gpt2.read_model_folder(folder)
    checked = 0
    for request, (prompt, tokens) in enumerate(zip(prompts, together)):
        sequence = list(prompt)
        for index, token in enumerate(tokens):
            logits = plain_gpt2.forward_logits(raw, weights, sequence)[-1]
            cdf = torch.softmax(logits / 0.8, dim=-1).cumsum(-1)
            u = uniform_for(7, request, index)
            upper = float(cdf[token])
            lower = float(cdf[token - 1]) if token > 0 else 0.0
            assert lower - 1e-4 <= u <= upper + 1e-4, (request, index, token, u, lower, upper)
            sequence.append(token)
            checked += 1
    assert checked == 36


def test_command_line(folders):
    """main.py as a user runs it: the built-in random model with the byte tokenizer, and a folder."""
    run = subprocess.run([sys.executable, os.path.join(ROOT, "main.py"), "--dtype", "bfloat16",
                          "--strategy", "sarathi", "--prefill-chunk-size", "4", "--max-batch-size", "4",
                          "--kv-cache-memory-mb", "8"], capture_output=True, text=True, timeout=600)
    assert run.returncode == 0, run.stderr[-2000:]
    lines = [line for line in run.stdout.splitlines() if line.startswith("request ")]
    assert len(lines) == 2 and lines[0].startswith("request 0:")
    folder, config, page_size = folders["A"]
    prompt = helpers.random_tokens(6, config["vocab_size"], 600)
    run = subprocess.run([sys.executable, os.path.join(ROOT, "main.py"), "--model", folder,
                          "--prompt-ids", ",".join(map(str, prompt)), "--max-new-tokens", "5",
                          "--block-size", str(page_size), "--num-kv-pages", "16", "--ignore-eos"],
                         capture_output=True, text=True, timeout=600)
    assert run.returncode == 0, run.stderr[-2000:]
    raw, weights = plain_gpt2.read_model_folder(folder)
    expected = plain_gpt2.greedy_generate(raw, weights, prompt, 5)
    assert f"tokens={expected}" in run.stdout


def test_smoke_entry():
    sys.path.insert(0, ROOT)
    import __graft_entry__

    __graft_entry__.smoke()


@pytest.mark.parametrize("strategy", ["orca", "sarathi"])
def test_many_requests_under_page_pressure_match_plain(folders, strategy):
    """Twenty requests of random lengths through the scheduler with pages for a few of them
    at a time: requests wait, run, end and give their pages to the next ones; every output
    equals the plain implementation's greedy continuation, and nothing is left behind."""
    from pagedserve_amd.engine.llm import LLM
    from pagedserve_amd.sampling import SamplingParams

    folder, config, page_size = folders["A"]
    g = torch.Generator().manual_seed(23)
    lengths = [int(torch.randint(1, 60, (1,), generator=g)) for _ in range(20)]
    budgets = [int(torch.randint(2, 14, (1,), generator=g)) for _ in range(20)]
    prompts = [helpers.random_tokens(n, config["vocab_size"], 800 + i) for i, n in enumerate(lengths)]
    raw, weights = plain_gpt2.read_model_folder(folder)
    expected = [plain_gpt2.greedy_generate(raw, weights, prompt, budget) for prompt, budget in zip(prompts, budgets)]
    options = dict(scheduling_strategy=strategy)
    if strategy == "sarathi":
        options.update(prefill_chunk_size=16, max_prefill_requests=2)
    # 30 pages of 8 tokens: the longest request needs 10 of them, so three to six run at a time
    llm = LLM(folder, dtype="float32", block_size=page_size, num_kv_pages=30, max_batch_size=6,
              eos_token_id=None, **options)
    outputs = llm.generate(prompts, [SamplingParams(max_new_tokens=budget) for budget in budgets])
    assert [o.token_ids for o in outputs] == expected
    llm.engine.cache.check_invariants()
    assert not llm.engine.cache.requests
    assert llm.scheduler.iterations > 20       # they did not all fit at once


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_random_schedules_match_plain(tmp_path, seed):
    """Random sets of requests under random schedules (strategy, portion size, batch limit,
    token budget, page size, few or many pages, recorded steps or not), greedy, in 32-bit:
    every output equals the plain implementation's continuation, whatever the schedule, and
    the cache's books are right afterwards.  The weights are lively and the head is untied, so
    that the tokens change from place to place."""
    import random

    from pagedserve_amd.engine.llm import LLM
    from pagedserve_amd.sampling import SamplingParams

    rng = random.Random(seed)
    config = {"architectures": ["GPT2LMHeadModel"], "model_type": "gpt2", "n_layer": 2, "n_embd": 64,
              "n_head": 4, "n_inner": 256, "vocab_size": 512, "n_positions": 160,
              "layer_norm_epsilon": 1e-5, "activation_function": "gelu_new",
              "tie_word_embeddings": False, "eos_token_id": None}
    folder = helpers.write_folder(str(tmp_path / "model"), config, helpers.lively_tensors(config, 900 + seed))
    raw, weights = plain_gpt2.read_model_folder(folder)
    for trial in range(8):
        count = rng.randint(1, 14)
        prompts = [helpers.random_tokens(rng.randint(1, 70), 512, seed * 10000 + trial * 100 + i)
                   for i in range(count)]
        news = [rng.randint(1, 40) for _ in range(count)]
        strategy = rng.choice(["orca", "sarathi"])
        chunk = rng.choice([1, 2, 3, 5, 8, 16, 33, 64])
        batch = rng.randint(1, 8)
        block = rng.choice([1, 2, 4, 8, 16])
        need = max(-(-(len(p) + n) // block) for p, n in zip(prompts, news))
        pages = need + rng.randint(0, 3 * need) + 1
        budget = rng.choice([None, None, batch + 1, 16, 64])
        graphs = rng.random() < 0.7
        case = (f"trial {trial}: {count} requests, {strategy}, portions of {chunk}, {batch} at a time, "
                f"pages of {block}, {pages} pages, budget {budget}, recorded steps {graphs}")
        llm = LLM(folder, dtype="float32", num_kv_pages=pages, block_size=block, max_batch_size=batch,
                  scheduling_strategy=strategy, prefill_chunk_size=chunk, max_num_batched_tokens=budget,
                  enable_hip_graphs=graphs, eos_token_id=None)
        outputs = llm.generate(prompts, [SamplingParams(max_new_tokens=n) for n in news])
        expected = [plain_gpt2.greedy_generate(raw, weights, prompt, n) for prompt, n in zip(prompts, news)]
        assert [list(o.token_ids) for o in outputs] == expected, case
        llm.engine.cache.check_invariants()
        assert not llm.engine.cache.requests, case
