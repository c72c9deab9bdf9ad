"""Decode and prefill throughput of the engine on one MI355X, bfloat16, random weights.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one decode step of the scheduler loop that serving runs: the engine's step
function over a batch of single tokens, token selection on the GPU and the copy of the
chosen tokens to the host.  The default run decodes a batch of 8 requests at GPT-2 small
shape whose contexts end at the model's context length, with uniform-random prompt ids.
One JSON line is printed:

* ``value``: decoded tokens a second of those K steps; ``roofline``: the step against the HBM
  roofline; ``prefill``: the step of 2 x 1,024 prompt tokens;
* ``points`` / ``points_roofline``: decode at batch 1 and 64 with contexts that end at the
  context length, and the benchmark configuration's own decode points (prompts of 128 and 512
  tokens, 128 output tokens, batch 1, 8 and 64), tokens a second and fraction of the roofline;
* ``points_fp32``: decode at batch 8 and the prefill step in true 32-bit;
* ``points_long``: a configuration of the same layer sizes with 8,192 positions: decode at
  batch 8 and 32 over contexts of 4,096 and 8,192, prefill of 2 x 4,096 tokens;
* ``workloads``: the other two sizes of the benchmark, each in its own workload.
  ``medium``: GPT-2 medium shape, 256 requests with prompts of 32-896 and outputs of 16-128
  tokens through the continuous-batching scheduler with prompt portions of 512, arriving as
  Poisson streams of three rates and as one burst; output tokens a second, time to first
  token, time per output token and end-to-end time (mean, p50, p95, p99), the share of
  iterations replayed from graphs, the flops of the stream against the peak, and one mixed
  step's time on the host and on the GPU.  ``small_stream``: the same stream at GPT-2 small
  shape, where the host has a third of the time per step.  ``xl``: GPT-2 XL shape, 64
  requests of 768 + 256 tokens at temperature 0.8, seed 7: decoded tokens a second against the
  roofline, prompt tokens a second.

    python bench.py --workload medium|small_stream|xl     one workload alone, one JSON line
    python bench.py --prefill-only --steps K [--prefill-length L]   the prefill step of 2 x L tokens alone (for profiles)
    python bench.py --kernels [--shape small|medium|xl|all] [--only name,name]

``--kernels`` times every kernel of a decode step (1, 8 and 64 requests over 1,024 keys), of
the prefill step (2 x 1,024 tokens) and of a mixed step (32 decoded tokens beside a portion of
512) alone, on weights that no cache holds (a graph of launches
that rotate over copies of them, at least 25 launches untimed and 100 timed), and prints a
table (to standard error) and one JSON line: microseconds, bytes, flops, and both as fractions
of the published peaks and of two measured ones (a device copy and the library's 4096-cubed
product).
"""

import argparse
import json
import sys
import time

# MI355X published peaks
HBM_GBPS = 8000.0
PEAK_TFLOPS = {"bf16": 2500.0, "fp16": 2500.0, "fp8": 5000.0, "fp32": 157.3}

# GPT-2 small: the layer sizes of the benchmark configuration
SMALL = {
    "architectures": ["GPT2LMHeadModel"], "model_type": "gpt2", "n_layer": 12, "n_embd": 768,
    "n_head": 12, "n_inner": 3072, "vocab_size": 50257, "n_positions": 1024,
    "layer_norm_epsilon": 1e-5, "activation_function": "gelu_new", "tie_word_embeddings": True,
    "eos_token_id": None,
}
MEDIUM = dict(SMALL, n_layer=24, n_embd=1024, n_head=16, n_inner=4096)
XL = dict(SMALL, n_layer=48, n_embd=1600, n_head=25, n_inner=6400)
LONG = dict(SMALL, n_positions=8192)
SHAPES = {"small": SMALL, "medium": MEDIUM, "xl": XL}
PAGE_SIZE = 16
PREFILL_TOKENS = 2048


def _random_prompt(generator, length, vocab):
    import torch

    # (an int64 array, as the scheduler hands long prompt portions to the step function)
    return torch.randint(0, vocab, (length,), generator=generator).numpy()


def _build(dtype, max_requests, max_step_tokens, layers=None, shape=SMALL, pages=None):
    """An engine over a model of ``shape`` with random weights (drawn on the GPU: the XL
    shape's 1.5 billion take a second there), and what the weights occupy."""
    import torch

    from pagedserve_amd.engine import Engine, hostgc
    from pagedserve_amd.model import random_model
    from pagedserve_amd.sampling.sampler import Sampler

    raw = dict(shape)
    if layers is not None:
        raw["n_layer"] = layers
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    model, config = random_model(raw, seed=0, dtype=dtype, device="cuda", draw_on="cuda")
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    resident = torch.cuda.memory_allocated() - before
    if pages is None:
        pages = max_requests * (config.n_positions // PAGE_SIZE) + 8
    engine = Engine(model, num_pages=pages, page_size=PAGE_SIZE, max_requests=max_requests,
                    max_step_tokens=max_step_tokens)
    engine.weights_resident_bytes = resident
    # (as the entry points do once an engine stands: the collector does not walk the model and
    # the modules again in the middle of a timed step)
    hostgc.settle()
    return engine, Sampler("cuda", max_requests), config


def decode_run(engine, sampler, config, batch, context_end, steps, warmup, seed=0):
    """Seconds for ``steps`` decode steps of ``batch`` requests whose contexts end at
    ``context_end``; prompts are prefilled (untimed) in portions."""
    import torch

    from pagedserve_amd.engine import ContinuousBatchScheduler
    from pagedserve_amd.sampling import SamplingParams

    generator = torch.Generator().manual_seed(seed)
    # Prompts are prefilled a few per iteration while the requests that are through decode
    # on: the first request is that many tokens ahead of the last.  Every request gets room
    # for it, so that none ends (and the batch stays whole) inside the timed steps; the first
    # one's context ends at ``context_end``, the last one's that many tokens earlier.
    ahead = -(-batch * context_end // engine.max_step_tokens)
    new_tokens = steps + warmup + 1 + ahead
    prompt_len = context_end - new_tokens
    if prompt_len < 1:
        raise ValueError("steps + warmup leave no room for a prompt")
    scheduler = ContinuousBatchScheduler(engine, sampler, max_batch_size=batch,
                                         scheduling_strategy="orca", eos_token_id=None)
    params = SamplingParams(max_new_tokens=new_tokens, ignore_eos=True)
    for _ in range(batch):
        scheduler.add_token_request(_random_prompt(generator, prompt_len, config.vocab_size),
                                    new_tokens, sampling=params)
    while scheduler.waiting:
        scheduler.step()
    for _ in range(warmup):
        scheduler.step()
    torch.cuda.synchronize()
    started = time.perf_counter()
    for _ in range(steps):
        scheduler.step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - started
    mean_context = context_end - 1 - (steps - 1) / 2.0 - ahead / 2.0
    while scheduler.has_work():
        scheduler.step()
    return elapsed, mean_context


def decode_point(engine, sampler, config, batch, prompt_len, output_tokens, warmup=8, seed=0):
    """Seconds for ``output_tokens`` decode steps of ``batch`` requests with prompts of
    ``prompt_len`` tokens (the steps after the prompts are in and ``warmup`` further steps
    have run), and the mean context length during them."""
    import torch

    from pagedserve_amd.engine import ContinuousBatchScheduler
    from pagedserve_amd.sampling import SamplingParams

    generator = torch.Generator().manual_seed(seed)
    ahead = -(-batch * prompt_len // engine.max_step_tokens)
    new_tokens = output_tokens + warmup + 1 + ahead
    scheduler = ContinuousBatchScheduler(engine, sampler, max_batch_size=batch,
                                         scheduling_strategy="orca", eos_token_id=None)
    params = SamplingParams(max_new_tokens=new_tokens, ignore_eos=True)
    for _ in range(batch):
        scheduler.add_token_request(_random_prompt(generator, prompt_len, config.vocab_size),
                                    new_tokens, sampling=params)
    while scheduler.waiting:
        scheduler.step()
    for _ in range(warmup):
        scheduler.step()
    torch.cuda.synchronize()
    started = time.perf_counter()
    for _ in range(output_tokens):
        scheduler.step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - started
    mean_context = prompt_len + warmup + ahead / 2.0 + (output_tokens + 1) / 2.0
    while scheduler.has_work():
        scheduler.step()
    return elapsed, mean_context


def prefill_run(engine, config, reps=8, warmup=None, seed=1, prompts=2, length=PREFILL_TOKENS // 2):
    """Seconds per step of ``prompts`` x ``length`` prompt tokens (logits at each prompt's last
    token), in the steady state: the warm-up covers the steps that allocate buffers and record
    the layout's graph."""
    import torch

    from pagedserve_amd.engine import StepEntry

    generator = torch.Generator().manual_seed(seed)
    times = []
    # (a layout with a prompt portion is recorded once it has come back ``record_after`` times)
    warmup = max(warmup or 0, engine.record_after + 2 if engine.use_graphs else 3)
    for rep in range(reps + warmup):
        entries = [StepEntry(f"p{rep}_{i}", _random_prompt(generator, length, config.vocab_size),
                             [length - 1]) for i in range(prompts)]
        torch.cuda.synchronize()
        started = time.perf_counter()
        # on the engine's own stream, as the scheduler issues its steps: a caller on another
        # stream pays for the hand-over between the two (60 us a step here)
        with torch.cuda.stream(engine.stream):
            engine.step(entries)
        torch.cuda.synchronize()
        if rep >= warmup:
            times.append(time.perf_counter() - started)
        for entry in entries:
            engine.finish(entry.request_id)
    return sum(times) / len(times)


def step_flops(config, tokens_per_request, logits_rows):
    """Multiply-add flops of one step: matrix products of every token, causal attention of
    each request over its own tokens, and the head for the wanted rows."""
    d, inner, layers = config.n_embd, config.n_inner, config.n_layer
    tokens = sum(tokens_per_request)
    linear = 2 * tokens * layers * (3 * d * d + d * d + 2 * d * inner)
    attention = sum(2 * 2 * layers * d * (t * (t + 1) // 2) for t in tokens_per_request)
    head = 2 * logits_rows * d * config.vocab_size
    return linear + attention + head


def decode_bytes(config, element_size, batch, mean_context):
    """Bytes one decode step has to read: every weight it uses once and the cache of the
    live requests."""
    d, inner, layers = config.n_embd, config.n_inner, config.n_layer
    matrices = layers * (3 * d * d + d * d + 2 * d * inner) + config.vocab_size * d
    vectors = layers * (3 * d + d + inner + d + 4 * d) + 2 * d
    cache = batch * mean_context * 2 * layers * d * element_size
    return matrices * element_size + vectors * 4 + cache


def _fraction(config, element, batch, mean_context, seconds_per_step):
    return round(decode_bytes(config, element, batch, mean_context) / seconds_per_step / 1e9 / HBM_GBPS, 4)


def _ms(group):
    return {key: (None if value is None else round(value * 1e3, 3)) for key, value in group.items()}


def _shape_keys(config, shape):
    return {"n_layer": config.n_layer, "n_layer_of_config": shape["n_layer"], "n_embd": config.n_embd,
            "n_head": config.n_head, "n_inner": config.n_inner, "vocab_size": config.vocab_size,
            "n_positions": config.n_positions, "page_size": PAGE_SIZE}


# --------------------------------------------------------------------------------- streams
def stream_requests(config, count, seed=0):
    """``count`` requests with uniform-random prompt lengths 32-896 and output lengths 16-128."""
    import random

    import torch

    from pagedserve_amd.engine.workload import TraceRequest
    from pagedserve_amd.sampling import SamplingParams

    lengths = random.Random(seed)
    generator = torch.Generator().manual_seed(seed)
    requests = []
    for _ in range(count):
        prompt, output = lengths.randint(32, 896), lengths.randint(16, 128)
        requests.append(TraceRequest(_random_prompt(generator, prompt, config.vocab_size), output,
                                     SamplingParams(max_new_tokens=output, ignore_eos=True)))
    return requests


def stream_run(engine, sampler, config, requests, rate, process, short, prompts_per_iteration=1):
    """One pass of the requests through the continuous-batching scheduler (prompt portions of
    512, up to 64 requests an iteration) with the given arrivals; a compact summary."""
    import torch

    from pagedserve_amd.engine import ContinuousBatchScheduler
    from pagedserve_amd.engine.workload import arrival_times, run_arrival_trace

    # an iteration's token budget: one portion of 512 beside up to 64 decoded tokens; with
    # several prompts an iteration, the prompts share that budget
    scheduler = ContinuousBatchScheduler(engine, sampler, max_batch_size=64, eos_token_id=None,
                                         scheduling_strategy="sarathi", prefill_chunk_size=512,
                                         max_prefill_requests=prompts_per_iteration,
                                         max_num_batched_tokens=512 + 64)
    before = engine.graph_summary()
    offsets = arrival_times(len(requests), rate, process, seed=1234)
    summary = run_arrival_trace(scheduler, requests, offsets, synchronize=torch.cuda.synchronize)
    engine.cache.check_invariants()
    after = engine.graph_summary()
    flops = 0
    for request, record in zip(requests, summary["records"]):
        tokens = len(request.prompt_token_ids) + len(record.token_times)
        flops += step_flops(config, [tokens], len(record.token_times))
    iterations = max(summary["iterations"], 1)
    return {
        "output_tok_s": round(summary["output_tokens_per_second"], 1),
        "total_tok_s": round(summary["total_tokens_per_second"], 1),
        "wall_s": round(summary["wall_seconds"], 3), "iterations": summary["iterations"],
        "replayed": round((after["graph_replays"] - before["graph_replays"]) / iterations, 3),
        "captures": after["captures"] - before["captures"], "evicted": after["evicted"] - before["evicted"],
        "capture_ms": round((after["capture_seconds"] - before["capture_seconds"]) * 1e3, 1),
        "steps_run_ahead": scheduler.steps_run_ahead,
        "of_peak_flops": round(flops / summary["wall_seconds"] / (PEAK_TFLOPS[short] * 1e12), 4),
        "ttft_ms": _ms(summary["ttft_seconds"]), "tpot_ms": _ms(summary["tpot_seconds"]),
        "e2e_ms": _ms(summary["e2e_seconds"]),
    }


def mixed_step_times(engine, config, decodes=32, portion=512, context=300, reps=5):
    """One mixed step (``decodes`` decoded tokens beside a prompt portion) issued kernel by
    kernel and replayed from its graph: milliseconds that the host needs to issue it, and
    milliseconds until the GPU is through with it."""
    import torch

    from pagedserve_amd.engine import StepEntry

    generator = torch.Generator().manual_seed(5)
    names = [f"mixed_d{i}" for i in range(decodes)]
    for name in names:
        engine.step([StepEntry(name, _random_prompt(generator, context, config.vocab_size), [context - 1])])
    prompt = _random_prompt(generator, portion, config.vocab_size)

    def one(rep):
        entries = [StepEntry(name, [5], [0]) for name in names] + [StepEntry(f"mixed_p{rep}", prompt, [])]
        torch.cuda.synchronize()
        started = time.perf_counter()
        with torch.cuda.stream(engine.stream):
            engine.step(entries, greedy=True)
        host = time.perf_counter() - started
        torch.cuda.synchronize()
        wall = time.perf_counter() - started
        engine.finish(f"mixed_p{rep}")
        return host, wall

    graphs = engine.use_graphs
    engine.use_graphs = False
    direct = [one(rep) for rep in range(reps + 2)][2:]
    engine.use_graphs = graphs
    # (the layout is recorded once it has come back ``record_after`` times)
    replayed = [one(rep) for rep in range(reps + 2, 2 * reps + 4 + engine.record_after)][-reps:]
    for name in names:
        engine.finish(name)

    def mean(values):
        return round(sum(values) / len(values) * 1e3, 3)

    return {"tokens": decodes + portion, "decoded": decodes,
            "direct_host_ms": mean([h for h, _ in direct]), "direct_ms": mean([w for _, w in direct]),
            "replayed_host_ms": mean([h for h, _ in replayed]), "replayed_ms": mean([w for _, w in replayed])}


def stream_workload(args, shape, name, rates):
    """The Poisson streams and the burst of one shape."""
    import torch

    from pagedserve_amd.engine import ContinuousBatchScheduler
    from pagedserve_amd.sampling import SamplingParams

    short = "bf16" if args.dtype == "bfloat16" else "fp32"
    engine, sampler, config = _build(args.dtype, max_requests=64, max_step_tokens=PREFILL_TOKENS,
                                     layers=args.layers, shape=shape)
    requests = stream_requests(config, args.requests)
    # the kernels' code is loaded by a few requests that are not part of the measurement
    warm = ContinuousBatchScheduler(engine, sampler, max_batch_size=64, eos_token_id=None)
    for request in requests[:2]:
        warm.add_token_request(request.prompt_token_ids[:80], 4,
                               sampling=SamplingParams(max_new_tokens=4, ignore_eos=True))
    warm.run_until_complete()
    runs = {}
    for rate in rates:
        runs[f"poisson_{int(rate)}_per_s"] = stream_run(engine, sampler, config, requests, rate, "poisson", short)
    runs["burst"] = stream_run(engine, sampler, config, requests, None, "burst", short)
    # several prompts may share an iteration's 512 prompt tokens: the last portion of one
    # prompt runs beside the first of the next instead of alone
    runs["burst_prompts_share_an_iteration"] = stream_run(engine, sampler, config, requests, None, "burst",
                                                         short, prompts_per_iteration=8)
    mixed = mixed_step_times(engine, config)
    best = max(run["output_tok_s"] for key, run in runs.items() if "share" not in key)
    record = {
        "metric": f"output tok/s of streams of {args.requests} requests (GPT-2 {name} shape, prompts 32-896, "
                  "outputs 16-128, prompt portions of 512, up to 64 requests an iteration)",
        "value": best, "unit": "tokens/s", "higher_is_better": True, "dtype": short,
        "data": "synthetic (random weights, uniform-random prompt ids and lengths, seeded arrivals)",
        "requests": args.requests, "prompt_tokens": sum(len(r.prompt_token_ids) for r in requests),
        "output_tokens": sum(r.max_new_tokens for r in requests),
        "weights_resident_bytes": engine.weights_resident_bytes,
        "runs": runs, "mixed_step": mixed,
        "config": dict(_shape_keys(config, shape), model=f"gpt2-{name}-shape", strategy="sarathi",
                       prefill_chunk_size=512, max_batch_size=64, arrivals="poisson seed 1234 / burst"),
    }
    del engine, sampler, warm
    torch.cuda.empty_cache()
    return record


def xl_workload(args):
    """GPT-2 XL shape: 64 concurrent requests of 768 prompt + 256 output tokens, temperature
    0.8, seed 7."""
    import torch

    from pagedserve_amd.engine import ContinuousBatchScheduler
    from pagedserve_amd.sampling import SamplingParams

    # (prompts are prefilled 4,096 tokens a step: 184 k prompt tokens a second where steps of
    # 2,048 give 141 k: the products fill the chip with whole rounds of tiles)
    engine, sampler, config = _build(args.dtype, max_requests=64, max_step_tokens=2 * PREFILL_TOKENS,
                                     layers=args.layers, shape=XL)
    scheduler = ContinuousBatchScheduler(engine, sampler, max_batch_size=64, eos_token_id=None)
    generator = torch.Generator().manual_seed(0)
    prompt_len, output_len, batch = 768, 256, 64
    # (untimed: a few requests of the same shape, among them one whole prefill step, so that
    # every kernel that the measurement launches has been loaded once)
    for _ in range(7):
        scheduler.add_token_request(_random_prompt(generator, prompt_len, config.vocab_size), 4,
                                    sampling=SamplingParams(max_new_tokens=4, temperature=0.8, seed=7, ignore_eos=True))
    scheduler.run_until_complete()
    for _ in range(batch):
        scheduler.add_token_request(
            _random_prompt(generator, prompt_len, config.vocab_size), output_len,
            sampling=SamplingParams(max_new_tokens=output_len, temperature=0.8, seed=7, ignore_eos=True))
    torch.cuda.synchronize()
    started = time.perf_counter()
    while scheduler.waiting:
        scheduler.step()
    torch.cuda.synchronize()
    prefilled = time.perf_counter() - started
    steps = 0
    while scheduler.has_work():
        scheduler.step()
        steps += 1
    torch.cuda.synchronize()
    wall = time.perf_counter() - started
    engine.cache.check_invariants()
    decode_tokens = batch * (output_len - 1)
    short = "bf16" if args.dtype == "bfloat16" else "fp32"
    element = 2 if args.dtype == "bfloat16" else 4
    step_seconds = (wall - prefilled) / steps
    moved = decode_bytes(config, element, batch, prompt_len + output_len / 2.0)
    prefill_flops = step_flops(config, [prompt_len] * batch, batch)
    graphs = engine.graph_summary()
    record = {
        "metric": "decode tok/s of 64 requests x (768 prompt + 256 output), temperature 0.8 seed 7 (GPT-2 XL shape)",
        "value": round(decode_tokens / (wall - prefilled), 1), "unit": "tokens/s", "n_gpus": 1,
        "higher_is_better": True, "dtype": short,
        "data": "synthetic (random weights, uniform-random prompt ids)",
        "wall_s": round(wall, 3), "prefill_s": round(prefilled, 3),
        "prefill_tok_s": round(batch * prompt_len / prefilled, 1),
        "prefill_of_peak_flops": round(prefill_flops / prefilled / (PEAK_TFLOPS[short] * 1e12), 4),
        "decode_steps": steps, "ms_per_step": round(step_seconds * 1e3, 4),
        "roofline": {"bound": "hbm", "achieved": round(moved / step_seconds / 1e9, 1), "peak": HBM_GBPS,
                     "unit": "GB/s", "frac": round(moved / step_seconds / 1e9 / HBM_GBPS, 4)},
        "weights_resident_bytes": engine.weights_resident_bytes,
        "steps_run_ahead": scheduler.steps_run_ahead,
        "graphs": {"kept": graphs["captured_graphs"], "captures": graphs["captures"],
                   "evicted": graphs["evicted"], "capture_ms": round(graphs["capture_seconds"] * 1e3, 1)},
        "config": dict(_shape_keys(config, XL), model="gpt2-xl-shape", global_batch=batch,
                       prompt_len=prompt_len, output_len=output_len, temperature=0.8, seed=7,
                       max_step_tokens=engine.max_step_tokens),
    }
    del engine, sampler, scheduler
    torch.cuda.empty_cache()
    return record


def long_points(args, short, element):
    """The small layer sizes with 8,192 positions: decode over long contexts, a long prefill."""
    import torch

    engine, sampler, config = _build(args.dtype, max_requests=32, max_step_tokens=8192, layers=args.layers,
                                     shape=LONG)
    points = {}
    for batch, context in ((8, 4096), (8, 8192), (32, 4096), (32, 8192)):
        steps = 32
        seconds, mean_context = decode_run(engine, sampler, config, batch, context, steps, 8, seed=context + batch)
        points[f"decode_b{batch}_ctx{context}"] = {
            "value": round(batch * steps / seconds, 1), "ms_per_step": round(seconds / steps * 1e3, 4),
            "frac": _fraction(config, element, batch, mean_context, seconds / steps)}
    seconds = prefill_run(engine, config, reps=4, warmup=4, prompts=2, length=4096)
    flops = step_flops(config, [4096, 4096], 2)
    points["prefill_2x4096"] = {"value": round(8192 / seconds, 1), "tokens": 8192, "ms": round(seconds * 1e3, 4),
                                "frac": round(flops / seconds / (PEAK_TFLOPS[short] * 1e12), 4)}
    points["n_positions"] = config.n_positions
    del engine, sampler
    torch.cuda.empty_cache()
    return points


def fp32_points(args):
    """Decode at batch 8 and the prefill step in true 32-bit (no reduced-precision matrix mode)."""
    import torch

    engine, sampler, config = _build("float32", max_requests=8, max_step_tokens=PREFILL_TOKENS, layers=args.layers)
    steps = 32
    seconds, mean_context = decode_run(engine, sampler, config, 8, config.n_positions, steps, 8)
    points = {"decode_b8": {"value": round(8 * steps / seconds, 1), "ms_per_step": round(seconds / steps * 1e3, 4),
                            "frac": _fraction(config, 4, 8, mean_context, seconds / steps)}}
    seconds = prefill_run(engine, config, reps=3, warmup=3)
    flops = step_flops(config, [PREFILL_TOKENS // 2] * 2, 2)
    points["prefill"] = {"value": round(PREFILL_TOKENS / seconds, 1), "tokens": PREFILL_TOKENS,
                         "ms": round(seconds * 1e3, 4),
                         "frac": round(flops / seconds / (PEAK_TFLOPS["fp32"] * 1e12), 4)}
    del engine, sampler
    torch.cuda.empty_cache()
    return points


def kernel_tables(args):
    """``--kernels``: the per-kernel tables of ``pagedserve_amd.measure.kernel_table``."""
    from pagedserve_amd.measure import kernel_table as table

    only = [piece for piece in (args.only or "").split(",") if piece] or None
    peaks = table.measured_peaks()
    print(f"measured peaks: copy {peaks['copy_GBps']} GB/s (published HBM {HBM_GBPS:.0f}), 4096-cubed "
          f"bfloat16 product of the library {peaks['product_4096_TFLOPs']} TFLOP/s (published "
          f"{PEAK_TFLOPS['bf16']:.0f})", file=sys.stderr, flush=True)
    names = list(SHAPES) if args.shape == "all" else [args.shape]
    tables = {}
    for name in names:
        raw = SHAPES[name]
        for rows in [int(piece) for piece in args.rows.split(",")]:
            key = f"{name}_decode_b{rows}_ctx{raw['n_positions']}"
            tables[key] = table.decode_table(raw, rows, raw["n_positions"], peaks, PAGE_SIZE, only)
            print(table.format_table(key, tables[key]), file=sys.stderr, flush=True)
        if not args.no_prefill:
            key = f"{name}_prefill_2x{PREFILL_TOKENS // 2}"
            tables[key] = table.prefill_table(raw, 2, PREFILL_TOKENS // 2, peaks, PAGE_SIZE, only)
            print(table.format_table(key, tables[key]), file=sys.stderr, flush=True)
            if only is None:
                # a step of the streams: 32 decoded tokens over 500 keys beside a portion of 512
                key = f"{name}_mixed_32_decoded_ctx500_beside_512"
                tables[key] = table.mixed_table(raw, 32, 500, 512, peaks, PAGE_SIZE)
                print(table.format_table(key, tables[key]), file=sys.stderr, flush=True)
    return {"metric": "microseconds per kernel, weights from memory", "unit": "us", "dtype": "bf16",
            "published_peak": {"hbm_GBps": HBM_GBPS, "bf16_TFLOPs": PEAK_TFLOPS["bf16"]},
            "measured_peak": peaks, "tables": tables}


def main(argv=None):
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=128)
    parser.add_argument("--warmup", type=int, default=16)
    parser.add_argument("--batch", type=int, default=8)
    parser.add_argument("--dtype", default="bfloat16", choices=("bfloat16", "float32"))
    parser.add_argument("--layers", type=int, default=None, help="fewer layers than the configuration")
    parser.add_argument("--no-points", action="store_true",
                        help="only the decode step at --batch (no prefill, points or workloads)")
    parser.add_argument("--no-workloads", action="store_true",
                        help="skip the medium, small-stream and XL workloads and the 32-bit and long points")
    parser.add_argument("--prefill-only", action="store_true",
                        help="only the 2,048-token prefill step, --steps times (for profiles)")
    parser.add_argument("--prefill-length", type=int, default=PREFILL_TOKENS // 2,
                        help="--prefill-only: tokens of each of the two prompts (beyond the small shape's "
                             "positions the configuration of points_long is used)")
    parser.add_argument("--workload", choices=("small", "medium", "small_stream", "xl"), default="small",
                        help="small: the whole record (default); medium / small_stream: the streams at "
                             "GPT-2 medium / small shape alone; xl: 64 x (768 + 256) at GPT-2 XL shape alone")
    parser.add_argument("--requests", type=int, default=256, help="requests of the streams")
    parser.add_argument("--request-rates", default=None,
                        help="mean arrivals a second of the Poisson streams, comma-separated "
                             "(default: 100,200,400 at medium shape, 300,600,1200 at small shape)")
    parser.add_argument("--kernels", action="store_true",
                        help="time every kernel of the decode and prefill steps alone (see above)")
    parser.add_argument("--shape", choices=("small", "medium", "xl", "all"), default="small",
                        help="layer sizes of --kernels")
    parser.add_argument("--rows", default="1,8,64", help="decode batch sizes of --kernels")
    parser.add_argument("--only", help="--kernels: only kernels whose name holds one of these (comma-separated)")
    parser.add_argument("--no-prefill", action="store_true", help="--kernels: decode tables only")
    args = parser.parse_args(argv)
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported by this engine")
        return 2

    import torch

    torch.cuda.init()
    if args.kernels:
        print(json.dumps(kernel_tables(args)), flush=True)
        return 0

    def rates(default):
        return [float(piece) for piece in args.request_rates.split(",")] if args.request_rates else default

    if args.workload == "medium":
        print(json.dumps(stream_workload(args, MEDIUM, "medium", rates([100.0, 200.0, 400.0]))), flush=True)
        return 0
    if args.workload == "small_stream":
        print(json.dumps(stream_workload(args, SMALL, "small", rates([300.0, 600.0, 1200.0]))), flush=True)
        return 0
    if args.workload == "xl":
        print(json.dumps(xl_workload(args)), flush=True)
        return 0
    short = "bf16" if args.dtype == "bfloat16" else "fp32"
    element = 2 if args.dtype == "bfloat16" else 4
    if args.prefill_only:
        length = args.prefill_length
        long = 2 * length > PREFILL_TOKENS
        engine, sampler, config = _build(args.dtype, max_requests=64, max_step_tokens=max(PREFILL_TOKENS, 2 * length),
                                         layers=args.layers, shape=LONG if long else SMALL)
        seconds = prefill_run(engine, config, reps=args.steps, warmup=max(min(args.warmup, 8), 5),
                              prompts=2, length=length)
        flops = step_flops(config, [length] * 2, 2)
        print(json.dumps({"prefill": {
            "value": round(2 * length / seconds, 1), "tokens": 2 * length,
            "ms": round(seconds * 1e3, 4),
            "frac": round(flops / seconds / (PEAK_TFLOPS[short] * 1e12), 4)}}), flush=True)
        return 0
    engine, sampler, config = _build(args.dtype, max_requests=64, max_step_tokens=PREFILL_TOKENS,
                                     layers=args.layers)
    context = config.n_positions
    elapsed, mean_context = decode_run(engine, sampler, config, args.batch, context, args.steps,
                                       args.warmup)
    ms_per_step = elapsed / args.steps * 1e3
    value = args.batch * args.steps / elapsed
    moved = decode_bytes(config, element, args.batch, mean_context)
    achieved = moved / (elapsed / args.steps) / 1e9
    record = {
        "metric": "decode tok/s at batch 1/8/64; prefill tok/s at 2,048 tokens (GPT-2 small)",
        "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": short,
        "data": "synthetic (random weights, uniform-random prompt ids)",
        "config": {
            "model": "gpt2-small-shape", "n_layer": config.n_layer, "n_layer_of_config": SMALL["n_layer"],
            "n_embd": config.n_embd, "n_head": config.n_head, "head_dim": config.head_dim,
            "n_inner": config.n_inner, "vocab_size": config.vocab_size,
            "n_positions": config.n_positions, "global_batch": args.batch, "seq_len": context,
            "page_size": PAGE_SIZE, "activation": config.activation_function,
            "parallelism": "single-gpu", "hip_graphs": bool(engine.use_graphs),
            "weights_resident_bytes": engine.weights_resident_bytes,
        },
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_GBPS,
                     "unit": "GB/s", "frac": round(achieved / HBM_GBPS, 4)},
    }
    if not args.no_points:
        seconds = prefill_run(engine, config)
        flops = step_flops(config, [PREFILL_TOKENS // 2] * 2, 2)
        record["prefill"] = {
            "value": round(PREFILL_TOKENS / seconds, 1), "tokens": PREFILL_TOKENS,
            "ms": round(seconds * 1e3, 4),
            "frac": round(flops / seconds / (PEAK_TFLOPS[short] * 1e12), 4)}
        points = {}
        fractions = {}
        for batch in (1, 64):
            steps = min(args.steps, 64)
            t, mean_context = decode_run(engine, sampler, config, batch, context, steps, min(args.warmup, 8),
                                         seed=batch)
            points[f"decode_b{batch}"] = round(batch * steps / t, 1)
            fractions[f"decode_b{batch}"] = _fraction(config, element, batch, mean_context, t / steps)
        # the benchmark configuration's decode points: prompts of 128 and 512 tokens, 128
        # output tokens, at batch 1, 8 and 64
        for prompt_len in (128, 512):
            for batch in (1, 8, 64):
                t, mean_context = decode_point(engine, sampler, config, batch, prompt_len, 128,
                                               seed=prompt_len + batch)
                name = f"p{prompt_len}_b{batch}"
                points[name] = round(batch * 128 / t, 1)
                fractions[name] = _fraction(config, element, batch, mean_context, t / 128)
        record["points"] = points
        record["points_roofline"] = fractions
        if not args.no_workloads and args.dtype == "bfloat16":
            del engine, sampler
            torch.cuda.empty_cache()
            record["points_long"] = long_points(args, short, element)
            record["points_fp32"] = fp32_points(args)
            args.requests = min(args.requests, 256)
            record["workloads"] = {
                "medium": stream_workload(args, MEDIUM, "medium", rates([100.0, 200.0, 400.0])),
                "small_stream": stream_workload(args, SMALL, "small", rates([300.0, 600.0, 1200.0])),
                "xl": xl_workload(args),
            }
    print(json.dumps(record), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
