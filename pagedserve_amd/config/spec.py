"""Architecture-neutral description of a model as data.

A model is an embedding, a list of blocks, an order in which the blocks run, a final
norm and an output head, each of them a part chosen by kind.  Every block names its parts by *kind* with the sizes and
constants they need, so two layers of one model may use different mixers or
feed-forwards, and nothing in a part knows which model it belongs to.

The engine, the cache manager and the weight loader read only these records; an
architecture (for instance ``pagedserve_amd.model.gpt2``) produces them from its own
typed configuration.
"""

from dataclasses import dataclass, field
from typing import Any, Mapping, Optional, Tuple


def _freeze(params):
    return tuple(sorted(params.items()))


@dataclass(frozen=True)
class PartSpec:
    """One part chosen by ``kind`` from its registry, built with ``params``."""

    kind: str
    params: Tuple[Tuple[str, Any], ...] = ()

    @staticmethod
    def make(kind: str, **params) -> "PartSpec":
        return PartSpec(kind, _freeze(params))

    def as_dict(self) -> Mapping[str, Any]:
        return dict(self.params)


@dataclass(frozen=True)
class BlockSpec:
    """One layer: how its parts are arranged and which parts they are.

    ``arrangement`` names a block class; the class says which named parts it is made of and
    what role each plays (``"pre_norm"``: ``norm1``, ``mixer``, ``norm2``, ``feed_forward``,
    run as ``h += mixer(norm1(h))`` then ``h += feed_forward(norm2(h))``).  ``parts`` gives a
    ``PartSpec`` for each of those names, so an arrangement with another number of parts needs
    no other record.
    """

    arrangement: str
    parts: Tuple[Tuple[str, PartSpec], ...]

    @staticmethod
    def make(arrangement: str, **parts: PartSpec) -> "BlockSpec":
        return BlockSpec(arrangement, tuple(parts.items()))

    def with_part(self, name: str, spec: PartSpec) -> "BlockSpec":
        """This block with the part ``name`` replaced (or added)."""
        parts = dict(self.parts)
        parts[name] = spec
        return BlockSpec(self.arrangement, tuple(parts.items()))

    def part(self, name: str) -> PartSpec:
        for key, spec in self.parts:
            if key == name:
                return spec
        raise KeyError(f"block of arrangement {self.arrangement!r} has no part {name!r}; "
                       f"it has: {', '.join(key for key, _ in self.parts)}")

    def __getattr__(self, name):
        # block.mixer, block.norm1, ...: the named part
        if name.startswith("__") or name in ("arrangement", "parts"):
            raise AttributeError(name)
        try:
            return self.part(name)
        except KeyError as error:
            raise AttributeError(str(error)) from None


@dataclass(frozen=True)
class LayerCall:
    """One entry of the run order.

    ``block`` indexes ``ModelSpec.blocks`` (a block may be named twice: its weights
    are shared).  ``cache`` is the cache entry that the call's mixer uses; two calls
    that name the same entry share keys and values, and only calls with
    ``writes_cache`` store new ones (a layer that reads another layer's cache has
    ``writes_cache=False``).
    """

    block: int
    cache: int
    writes_cache: bool = True


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    vocab_size: int
    width: int
    max_positions: int
    position: PartSpec
    blocks: Tuple[BlockSpec, ...]
    schedule: Tuple[LayerCall, ...]
    final_norm: PartSpec
    tie_head: bool
    eos_token_id: Optional[int] = None
    extra: Tuple[Tuple[str, Any], ...] = field(default=())
    # how token ids become rows of the stream, and how the last rows become logits
    embedding: PartSpec = PartSpec("lookup")
    head: PartSpec = PartSpec("linear")

    def __post_init__(self):
        if not self.blocks:
            raise ValueError("a model needs at least one block")
        if not self.schedule:
            raise ValueError("a model needs a non-empty run order")
        writers = {}
        for call in self.schedule:
            if not 0 <= call.block < len(self.blocks):
                raise ValueError(f"run order names block {call.block}, model has {len(self.blocks)}")
            if call.cache < 0:
                raise ValueError("cache entries are numbered from 0")
            if call.writes_cache:
                if call.cache in writers:
                    raise ValueError(f"cache entry {call.cache} has two writers")
                writers[call.cache] = call
        seen = set()
        for call in self.schedule:
            if not call.writes_cache and call.cache not in seen:
                raise ValueError(
                    f"a call reads cache entry {call.cache} before any call has written it")
            if call.writes_cache:
                seen.add(call.cache)
        entries = sorted({call.cache for call in self.schedule})
        if entries != list(range(len(entries))):
            raise ValueError("cache entries must be numbered 0..n-1 without gaps")

    @property
    def num_cache_entries(self) -> int:
        return len({call.cache for call in self.schedule})
