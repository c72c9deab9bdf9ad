"""Command line of the engine, in the manner of the reference's main.py:257-342.

Options keep the reference's names and meanings where it has them (``--strategy``,
``--prefill-chunk-size``, ``--max-batch-size``, ``--kv-cache-memory-mb``,
``--kv-cache-memory-utilization``, ``--kv-cache-safety-mb``, ``--dtype``); ``--model`` is a
model folder (or ``reference`` for a small random model) instead of a fixed list of names,
and ``--disable-hip-graphs`` takes the place of ``--disable-cuda-graphs`` (also accepted).
There is one attention implementation and no quantized cache: ``--decode-attention-backend``
takes ``hip`` only (the reference's ``torch`` and ``triton`` do not exist here and are refused
with a message that says so), and ``--kv-cache-dtype`` takes ``model`` only and refuses
``int8``.
"""

import argparse
import sys

from pagedserve_amd.engine.llm import (DEFAULT_KV_MEMORY_UTILIZATION, DEFAULT_KV_SAFETY_MB,
                                        REFERENCE_MODEL, build_scheduler)
from pagedserve_amd.engine.scheduler import ORCA_STRATEGY, SUPPORTED_SCHEDULING_STRATEGIES
from pagedserve_amd.sampling.params import SamplingParams

SUPPORTED_DTYPES = ("float32", "bfloat16")
SUPPORTED_DECODE_ATTENTION_BACKENDS = ("hip",)    # the reference's option (main.py:27) with the one value built here
SUPPORTED_KV_CACHE_DTYPES = ("model", "int8")                      # main.py:28


def parse_args(argv=None):
    parser = argparse.ArgumentParser(description="Run the pagedserve_amd inference engine")
    parser.add_argument("--model", default=REFERENCE_MODEL,
                        help="model folder (config.json + model.safetensors), or 'reference' "
                             "for a small random model")
    parser.add_argument("--strategy", choices=SUPPORTED_SCHEDULING_STRATEGIES, default=ORCA_STRATEGY,
                        help="request scheduling strategy")
    parser.add_argument("--prefill-chunk-size", type=int, default=16,
                        help="prompt tokens per Sarathi prefill chunk")
    parser.add_argument("--max-batch-size", type=int, help="maximum requests per iteration (default: 32)")
    parser.add_argument("--max-num-batched-tokens", type=int,
                        help="token budget of one iteration (default: 2048)")
    parser.add_argument("--kv-cache-memory-mb", type=int,
                        help="explicit KV-cache budget in MiB; default: sized from free device memory")
    parser.add_argument("--kv-cache-memory-utilization", type=float, default=DEFAULT_KV_MEMORY_UTILIZATION,
                        help="target total GPU memory utilization for automatic KV sizing")
    parser.add_argument("--kv-cache-safety-mb", type=int, default=DEFAULT_KV_SAFETY_MB,
                        help="device memory retained for activations and temporary buffers")
    parser.add_argument("--num-kv-pages", type=int, help="explicit number of KV pages")
    parser.add_argument("--block-size", type=int, default=16, help="tokens per KV page")
    parser.add_argument("--dtype", choices=SUPPORTED_DTYPES, default="float32", help="execution dtype")
    parser.add_argument("--decode-attention-backend", default="hip",
                        help="attention implementation: 'hip', the only one built")
    parser.add_argument("--kv-cache-dtype", choices=SUPPORTED_KV_CACHE_DTYPES, default="model",
                        help="KV storage dtype: the model's (quantized caches are not built)")
    parser.add_argument("--disable-hip-graphs", "--disable-cuda-graphs", dest="disable_hip_graphs",
                        action="store_true", help="disable HIP-graph replay of decode steps")
    parser.add_argument("--random-weights", action="store_true",
                        help="ignore the folder's tensors and draw random weights for its config.json")
    parser.add_argument("--seed", type=int, default=0, help="seed of --random-weights / 'reference'")
    parser.add_argument("--prompt", action="append", help="text prompt (may be repeated)")
    parser.add_argument("--prompt-ids", action="append",
                        help="prompt as comma- or space-separated token ids (may be repeated)")
    parser.add_argument("--max-new-tokens", type=int, default=8)
    parser.add_argument("--temperature", type=float, default=0.0, help="0 = greedy")
    parser.add_argument("--sample-seed", type=int, help="seed of temperature sampling")
    parser.add_argument("--ignore-eos", action="store_true")
    args = parser.parse_args(argv)
    if args.kv_cache_dtype != "model":
        parser.error("--kv-cache-dtype int8: quantized caches are not built; the cache has the model's dtype")
    if args.decode_attention_backend not in SUPPORTED_DECODE_ATTENTION_BACKENDS:
        parser.error(f"--decode-attention-backend {args.decode_attention_backend}: this engine has one "
                     "attention implementation, 'hip' (hand-written kernels); leave the option out")
    return args


def main(argv=None):
    args = parse_args(argv)
    scheduler = build_scheduler(
        args.model, scheduling_strategy=args.strategy, prefill_chunk_size=args.prefill_chunk_size,
        max_batch_size=args.max_batch_size, kv_cache_memory_mb=args.kv_cache_memory_mb,
        kv_cache_memory_utilization=args.kv_cache_memory_utilization,
        kv_cache_safety_mb=args.kv_cache_safety_mb, execution_dtype=args.dtype,
        enable_hip_graphs=not args.disable_hip_graphs, block_size=args.block_size,
        num_kv_pages=args.num_kv_pages, max_num_batched_tokens=args.max_num_batched_tokens,
        random_weights=args.random_weights, seed=args.seed)
    sampling = SamplingParams(temperature=args.temperature, seed=args.sample_seed,
                              max_new_tokens=args.max_new_tokens, ignore_eos=args.ignore_eos)
    request_ids = []
    for text in args.prompt_ids or []:
        ids = [int(piece) for piece in text.replace(",", " ").split()]
        request_ids.append(scheduler.add_token_request(ids, args.max_new_tokens, sampling=sampling))
    prompts = args.prompt
    if not prompts and not request_ids:
        prompts = ["Paged attention", "Orca"]      # the reference's two prompts, main.py:337-338
    for prompt in prompts or []:
        request_ids.append(scheduler.add_request(prompt, args.max_new_tokens, sampling=sampling))
    results = scheduler.run_until_complete()
    for request_id in request_ids:
        state = scheduler.finished[request_id]
        print(f"request {request_id}: {results[request_id]!r}  tokens={state.generated_token_ids}")
    return 0


if __name__ == "__main__":
    sys.exit(main())
