"""Registries of part kinds.  A kind is a name in a ``PartSpec``; registering a class
under a new name is all it takes to make it available to every model."""

from typing import Callable, Dict

NORMS: Dict[str, Callable] = {}
MIXERS: Dict[str, Callable] = {}
FEED_FORWARDS: Dict[str, Callable] = {}
POSITIONS: Dict[str, Callable] = {}
ARRANGEMENTS: Dict[str, Callable] = {}
EMBEDDINGS: Dict[str, Callable] = {}
HEADS: Dict[str, Callable] = {}

# role of a block's named part -> the registry its kind is looked up in
ROLES = {"norm": NORMS, "mixer": MIXERS, "feed_forward": FEED_FORWARDS}


def _register(table, what):
    def decorator(name):
        def apply(cls):
            if name in table and table[name] is not cls:
                raise ValueError(f"{what} kind {name!r} is already registered")
            table[name] = cls
            return cls
        return apply
    return decorator


register_norm = _register(NORMS, "norm")
register_mixer = _register(MIXERS, "mixer")
register_feed_forward = _register(FEED_FORWARDS, "feed-forward")
register_position = _register(POSITIONS, "position encoding")
register_arrangement = _register(ARRANGEMENTS, "block arrangement")
register_embedding = _register(EMBEDDINGS, "embedding")
register_head = _register(HEADS, "output head")


def build_part(table, what, spec, **common):
    if spec.kind not in table:
        raise KeyError(f"unknown {what} kind {spec.kind!r}; known: {', '.join(sorted(table))}")
    return table[spec.kind](**common, **spec.as_dict())
