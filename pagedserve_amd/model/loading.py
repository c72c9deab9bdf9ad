"""From a model folder to a bound model, and the random-weights mode."""

import json
import os

import torch

from ..config.base import read_config_json
from ..config.registry import resolve_architecture
from ..weights.loader import load_parameters
from ..weights.safetensors_io import write_safetensors
from .decoder import DecoderModel

DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def resolve_dtype(dtype):
    if isinstance(dtype, torch.dtype):
        if dtype not in DTYPES.values():
            raise ValueError(f"dtype {dtype} is not supported; choose float32 or bfloat16")
        return dtype
    if dtype not in DTYPES:
        raise ValueError(f"Unknown dtype '{dtype}'. Choose one of: {', '.join(DTYPES)}")
    return DTYPES[dtype]


def load_model(folder, dtype="float32", device="cuda"):
    """(model, typed config) of the folder's ``config.json`` + ``model.safetensors``."""
    raw = read_config_json(folder)
    architecture = resolve_architecture(raw)
    config = architecture.config_class.from_dict(raw)
    spec = architecture.build_spec(config)
    engine_dtype = resolve_dtype(dtype)
    model = DecoderModel(spec, engine_dtype, device)
    tensors = load_parameters(
        folder, model.parameters(), architecture.weight_sources(config, spec), engine_dtype,
        device, strip_prefixes=architecture.strip_prefixes,
        ignorable=lambda name: architecture.ignorable(config, name))
    model.bind(tensors)
    return model, config


def random_model(config, seed=0, dtype="bfloat16", device="cuda", draw_on=None):
    """A bound model with random weights of ``config`` (typed, or a raw config.json dict),
    made in memory: the same draws, layouts and casts as writing a folder and loading it.
    ``draw_on``: a device on which the architecture's initialiser draws instead of the CPU, if
    it takes one (seconds instead of a minute for billions of weights; the numbers then differ
    from a written folder's, the distributions do not)."""
    import inspect

    from ..weights.loader import target_dtype

    if isinstance(config, dict):
        architecture = resolve_architecture(config)
        config = architecture.config_class.from_dict(config)
    else:
        architecture = resolve_architecture({"architectures": [config.architecture]})
    spec = architecture.build_spec(config)
    engine_dtype = resolve_dtype(dtype)
    model = DecoderModel(spec, engine_dtype, device)
    if draw_on is not None and "device" in inspect.signature(architecture.random_tensors).parameters:
        drawn = architecture.random_tensors(config, seed, device=draw_on)
    else:
        drawn = architecture.random_tensors(config, seed)
    sources = architecture.weight_sources(config, spec)
    tensors = {}
    for target, param in model.parameters().items():
        source = sources[target]
        tensor = source.assemble(drawn.__getitem__)
        if tuple(tensor.shape) != tuple(param.shape):
            raise ValueError(f"random tensor {source.label()} has shape {tuple(tensor.shape)}, "
                             f"parameter {target} needs {tuple(param.shape)}")
        tensors[target] = tensor.to(target_dtype(param.role, engine_dtype)).contiguous().to(device)
    model.bind(tensors)
    return model, config


def write_random_model(folder, config, seed=0, store_dtype=torch.float32, stored_name=None):
    """Write ``config.json`` and ``model.safetensors`` of a random model of ``config``.

    ``config`` is a typed configuration of a registered architecture or a raw dict with that
    architecture's config.json keys (``architectures`` or ``model_type`` among them).  Tensors
    are named as the architecture's checkpoints name them, or by ``stored_name(name)``."""
    if isinstance(config, dict):
        raw = dict(config)
        architecture = resolve_architecture(raw)
        raw.setdefault("architectures", [architecture.name])
        config = architecture.config_class.from_dict(raw)
    else:
        architecture = resolve_architecture({"architectures": [config.architecture]})
    if stored_name is None:
        stored_name = lambda name: architecture.stored_name(config, name)  # noqa: E731
    os.makedirs(folder, exist_ok=True)
    tensors = architecture.random_tensors(config, seed)
    stored = {stored_name(name): tensor.to(store_dtype).contiguous() for name, tensor in tensors.items()}
    write_safetensors(os.path.join(folder, "model.safetensors"), stored,
                      metadata={"format": "pt", "seed": seed})
    with open(os.path.join(folder, "config.json"), "w") as handle:
        json.dump(config.to_dict(), handle, indent=2)
    return config
