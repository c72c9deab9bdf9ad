"""The one registry from an architecture's name to what builds its model.

The reference picks a model by a fixed tuple of names and an if/elif chain
(main.py:22-25,104-130).  Here ``config.json``'s ``architectures[0]`` is the key.
An entry bundles the typed configuration class, the function that turns it into a
``ModelSpec`` (parts, run order), the map from checkpoint tensor names to the
parts' parameters, how the checkpoint's names are prefixed, and the random initialiser of
the random-weights mode.
"""

from dataclasses import dataclass
from typing import Any, Callable, Dict

from .base import ConfigError
from .spec import ModelSpec


@dataclass(frozen=True)
class Architecture:
    name: str
    config_class: Any
    # config -> ModelSpec
    build_spec: Callable[[Any], ModelSpec]
    # (config, spec) -> {parameter path: WeightSource}
    weight_sources: Callable[[Any, ModelSpec], Dict[str, Any]]
    # (config, seed) -> {checkpoint tensor name: float32 tensor}
    random_tensors: Callable[[Any, int], Dict[str, Any]]
    # names of checkpoint tensors that may be present and are not weights
    ignorable: Callable[[Any, str], bool] = lambda config, name: False
    model_type: str = ""
    # prefixes under which checkpoints of this architecture may store their tensors
    strip_prefixes: tuple = ()
    # (config, canonical tensor name) -> the name under which the random-weights mode stores it
    stored_name: Callable[[Any, str], str] = lambda config, name: name
    # named raw configurations of this architecture (config.json keys) that a model name may
    # stand for instead of a folder: small random models for trying the engine out
    presets: tuple = ()      # ((name, raw config dict), ...)


ARCHITECTURES: Dict[str, Architecture] = {}


def register_architecture(entry: Architecture) -> Architecture:
    if entry.name in ARCHITECTURES:
        raise ValueError(f"architecture {entry.name!r} is already registered")
    ARCHITECTURES[entry.name] = entry
    return entry


def _load_builtin():
    # Importing the module registers it.
    from ..model import gpt2  # noqa: F401


def find_preset(name: str):
    """The raw configuration that an architecture registered under ``name``, or None."""
    _load_builtin()
    for entry in ARCHITECTURES.values():
        for preset, raw in entry.presets:
            if preset == name:
                return dict(raw)
    return None


def preset_names():
    _load_builtin()
    return sorted(preset for entry in ARCHITECTURES.values() for preset, _ in entry.presets)


def resolve_architecture(raw_config: dict) -> Architecture:
    """The entry for a ``config.json`` dict, or one clear error listing what exists."""
    _load_builtin()
    names = raw_config.get("architectures")
    if isinstance(names, (list, tuple)) and names:
        name = names[0]
        if name in ARCHITECTURES:
            return ARCHITECTURES[name]
        raise ConfigError(
            f"architecture {name!r} is not registered; known: {', '.join(sorted(ARCHITECTURES))}")
    model_type = raw_config.get("model_type")
    for entry in ARCHITECTURES.values():
        if model_type and entry.model_type == model_type:
            return entry
    raise ConfigError(
        "config.json names no 'architectures' entry (and no known 'model_type'); "
        f"known architectures: {', '.join(sorted(ARCHITECTURES))}")
