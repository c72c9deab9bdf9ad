"""Decode and prefill throughput of the engine on one MI355X, GPT-2 small shape, bfloat16.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one decode step of the scheduler loop that serving runs: the engine's step
function over a batch of single tokens, token selection on the GPU and the copy of the
chosen tokens to the host.  The default run decodes a batch of 8 requests whose contexts
end at the model's context length, with random weights and uniform-random prompt ids.
One JSON line is printed: decoded tokens a second (``value``), the 2,048-token prefill
step (``prefill``), the decode step against the HBM roofline (``roofline``) and decode at
batch 1 and 64 (``points``).
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
PAGE_SIZE = 16
PREFILL_TOKENS = 2048


def _random_prompt(generator, length, vocab):
    import torch

    return torch.randint(0, vocab, (length,), generator=generator).tolist()


def _build(dtype, max_requests, max_step_tokens, layers=None):
    from pagedserve_amd.engine import Engine
    from pagedserve_amd.model import random_model
    from pagedserve_amd.sampling.sampler import Sampler

    raw = dict(SMALL)
    if layers is not None:
        raw["n_layer"] = layers
    model, config = random_model(raw, seed=0, dtype=dtype, device="cuda")
    pages = max_requests * (config.n_positions // PAGE_SIZE) + 8
    engine = Engine(model, num_pages=pages, page_size=PAGE_SIZE, max_requests=max_requests,
                    max_step_tokens=max_step_tokens)
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


def prefill_run(engine, config, reps=8, warmup=5, seed=1):
    """Seconds per step of 2 x 1024 prompt tokens (logits at each prompt's last token), in the
    steady state: the warm-up covers the steps that allocate buffers and record the layout's
    graph."""
    import torch

    from pagedserve_amd.engine import StepEntry

    generator = torch.Generator().manual_seed(seed)
    length = PREFILL_TOKENS // 2
    times = []
    for rep in range(reps + warmup):
        entries = [StepEntry(f"p{rep}_{i}", _random_prompt(generator, length, config.vocab_size),
                             [length - 1]) for i in range(2)]
        torch.cuda.synchronize()
        started = time.perf_counter()
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


def main(argv=None):
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=128)
    parser.add_argument("--warmup", type=int, default=16)
    parser.add_argument("--batch", type=int, default=8)
    parser.add_argument("--dtype", default="bfloat16", choices=("bfloat16", "float32"))
    parser.add_argument("--layers", type=int, default=None, help="fewer layers than the configuration")
    parser.add_argument("--no-points", action="store_true", help="skip batch 1 / 64 and prefill")
    parser.add_argument("--prefill-only", action="store_true",
                        help="only the 2,048-token prefill step, --steps times (for profiles)")
    args = parser.parse_args(argv)
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported by this engine")
        return 2

    import torch

    torch.cuda.init()
    short = "bf16" if args.dtype == "bfloat16" else "fp32"
    element = 2 if args.dtype == "bfloat16" else 4
    engine, sampler, config = _build(args.dtype, max_requests=64, max_step_tokens=PREFILL_TOKENS,
                                     layers=args.layers)
    context = config.n_positions
    if args.prefill_only:
        seconds = prefill_run(engine, config, reps=args.steps, warmup=max(min(args.warmup, 8), 5))
        flops = step_flops(config, [PREFILL_TOKENS // 2] * 2, 2)
        print(json.dumps({"prefill": {
            "value": round(PREFILL_TOKENS / seconds, 1), "tokens": PREFILL_TOKENS,
            "ms": round(seconds * 1e3, 4),
            "frac": round(flops / seconds / (PEAK_TFLOPS[short] * 1e12), 4)}}), flush=True)
        return 0
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
        for batch in (1, 64):
            steps = min(args.steps, 64)
            t, _ = decode_run(engine, sampler, config, batch, context, steps, min(args.warmup, 8),
                              seed=batch)
            points[f"decode_b{batch}"] = round(batch * steps / t, 1)
        record["points"] = points
    print(json.dumps(record), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
