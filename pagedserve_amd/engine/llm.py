"""Python entry points: ``build_scheduler`` in the reference's manner and ``LLM.generate``.

``build_scheduler`` mirrors main.py:136-254 of the reference: it loads the model, sizes the
key/value cache (explicit MiB, or from the device's free memory with a utilization target
and a safety margin, main.py:48-73), and wires cache, engine, sampler and scheduler.  The
model is named by its folder (``config.json`` + ``model.safetensors``), not by a fixed list.
"""

from dataclasses import dataclass
from typing import List, Optional, Sequence, Union

import torch

from ..cache.manager import kv_cache_budget
from ..config.base import read_config_json
from ..config.registry import find_preset
from ..model.loading import load_model, random_model, resolve_dtype
from ..sampling.params import SamplingParams
from . import hostgc
from .engine import Engine
from .scheduler import ORCA_STRATEGY, ContinuousBatchScheduler
from .tokenizer import load_tokenizer

MIB = 1024 * 1024
DEFAULT_KV_MEMORY_UTILIZATION = 0.90   # main.py:30
DEFAULT_KV_SAFETY_MB = 3072            # main.py:31
REFERENCE_MODEL = "reference"   # a preset that the architecture's registry entry names


def _bytes_per_page(model, page_size, dtype):
    groups, _ = model.cache_requirements()
    element = torch.empty(0, dtype=dtype).element_size()
    return sum(len(g.entries) * g.kv_heads * page_size * (g.head_dim + g.value_head_dim) * element
               for g in groups)


def build_scheduler(model=REFERENCE_MODEL, scheduling_strategy=ORCA_STRATEGY, prefill_chunk_size=16,
                    max_batch_size=None, kv_cache_memory_mb=None,
                    kv_cache_memory_utilization=DEFAULT_KV_MEMORY_UTILIZATION,
                    kv_cache_safety_mb=DEFAULT_KV_SAFETY_MB, execution_dtype="float32",
                    enable_hip_graphs=True, block_size=16, num_kv_pages=None,
                    max_num_batched_tokens=None, max_prefill_requests=None, random_weights=False,
                    seed=0, eos_token_id="config", model_name=None, enable_cuda_graphs=None,
                    decode_attention_backend="hip", kv_cache_dtype="model"):
    """Load ``model`` (a folder, or a preset's name such as ``"reference"`` for a small random
    model) and return a ``ContinuousBatchScheduler`` ready for ``add_request`` /
    ``run_until_complete``.

    The reference's names for the same things are taken as well (main.py:136-150):
    ``model_name`` for ``model``, ``enable_cuda_graphs`` for ``enable_hip_graphs``.  Of its
    ``decode_attention_backend`` only ``"hip"`` exists here and of ``kv_cache_dtype`` only
    ``"model"`` (quantized caches are not built); other values are errors."""
    if model_name is not None:
        model = model_name
    if enable_cuda_graphs is not None:
        enable_hip_graphs = bool(enable_cuda_graphs)
    if decode_attention_backend != "hip":
        raise ValueError(f"Unknown decode attention backend '{decode_attention_backend}': "
                         "the one implementation here is 'hip'")
    if kv_cache_dtype != "model":
        raise ValueError(f"KV cache dtype '{kv_cache_dtype}': quantized caches are not built; "
                         "the cache has the model's dtype ('model')")
    if not torch.cuda.is_available():
        raise RuntimeError("pagedserve_amd needs a GPU (MI355X); there is no CPU path")
    dtype = resolve_dtype(execution_dtype)
    device = torch.device("cuda")
    preset = find_preset(model) if isinstance(model, str) else None
    if preset is not None:
        # random weights are drawn in memory: the tensors that writing a folder and loading it
        # would give, without the folder
        loaded, config = random_model(preset, seed=seed, dtype=dtype, device=device)
    elif random_weights:
        loaded, config = random_model(read_config_json(model), seed=seed, dtype=dtype, device=device)
    else:
        loaded, config = load_model(model, dtype=dtype, device=device)
    if max_batch_size is None:
        max_batch_size = 32          # main.py:180-181 (its GPU default)
    if max_batch_size <= 0:
        raise ValueError("max_batch_size must be positive")
    per_page = _bytes_per_page(loaded, block_size, dtype)
    source = "explicit"
    if num_kv_pages is not None:
        pages = int(num_kv_pages)
    elif kv_cache_memory_mb is not None:
        if kv_cache_memory_mb <= 0:
            raise ValueError("kv_cache_memory_mb must be positive")
        pages = kv_cache_memory_mb * MIB // per_page
    else:
        torch.cuda.synchronize(device)
        free_memory, total_memory = torch.cuda.mem_get_info(device)
        budget = kv_cache_budget(free_memory, total_memory, kv_cache_memory_utilization,
                                 kv_cache_safety_mb * MIB)
        # never more than every slot at full context needs
        useful = max_batch_size * (-(-loaded.spec.max_positions // block_size)) * per_page
        pages = min(budget, useful) // per_page
        source = "device_auto"
    if pages <= 0:
        raise ValueError(f"Memory budget is too small; one block requires {per_page} bytes")
    step_tokens = max_num_batched_tokens or max(2048, max_batch_size)
    engine = Engine(loaded, num_pages=pages, page_size=block_size, max_requests=max_batch_size,
                    max_step_tokens=step_tokens, use_graphs=enable_hip_graphs)
    engine.memory_budget_source = source
    from ..sampling.sampler import Sampler

    # "config": what config.json says (null there means that no token ends a request); an
    # explicit value, None included, overrides it.  The scheduler never asks the tokenizer.
    eos = config.eos_token_id if eos_token_id == "config" else eos_token_id
    tokenizer = load_tokenizer(None if preset is not None else model, config.vocab_size, eos)
    scheduler = ContinuousBatchScheduler(
        engine, Sampler(device, max_batch_size), tokenizer=tokenizer,
        max_batch_size=max_batch_size, eos_token_id=eos,
        scheduling_strategy=scheduling_strategy, prefill_chunk_size=prefill_chunk_size,
        max_num_batched_tokens=step_tokens, max_prefill_requests=max_prefill_requests)
    scheduler.model_config = config
    hostgc.settle()
    return scheduler


@dataclass
class GenerationOutput:
    request_id: int
    prompt_token_ids: List[int]
    token_ids: List[int]
    text: Optional[str]
    finish_reason: Optional[str]


class LLM:
    """``LLM(model=folder, dtype=...).generate(prompts, sampling_params)``."""

    def __init__(self, model, dtype="float32", **engine_args):
        self.scheduler = build_scheduler(model, execution_dtype=dtype, **engine_args)
        self.engine = self.scheduler.engine

    def generate(self, prompts: Sequence[Union[str, Sequence[int]]],
                 sampling_params: Union[SamplingParams, Sequence[SamplingParams], None] = None
                 ) -> List[GenerationOutput]:
        prompts = list(prompts)
        if sampling_params is None:
            sampling_params = SamplingParams()
        if isinstance(sampling_params, SamplingParams):
            sampling_params = [sampling_params] * len(prompts)
        if len(sampling_params) != len(prompts):
            raise ValueError("one SamplingParams per prompt (or one for all) is needed")
        ids = []
        for prompt, params in zip(prompts, sampling_params):
            if isinstance(prompt, str):
                ids.append(self.scheduler.add_request(prompt, params.max_new_tokens, params))
            else:
                ids.append(self.scheduler.add_token_request(list(prompt), params.max_new_tokens,
                                                            sampling=params))
        while any(rid not in self.scheduler.finished for rid in ids):
            self.scheduler.step()
        outputs = []
        for rid in ids:
            state = self.scheduler.finished.pop(rid)
            text = None
            if self.scheduler.tokenizer is not None:
                text = self.scheduler.tokenizer.decode(state.generated_token_ids)
            outputs.append(GenerationOutput(rid, state.prompt_token_ids,
                                            list(state.generated_token_ids), text,
                                            state.finish_reason))
        return outputs
