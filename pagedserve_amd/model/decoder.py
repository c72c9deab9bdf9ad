"""A decoder-only language model assembled from a ``ModelSpec``.

Embedding (+ position table), the blocks in the order of the run list, final norm on
the rows whose logits are wanted, output head.  The class knows no architecture: the
kinds and sizes of all parts come from the spec, and the run list may name a block
twice or let a call read the cache entry that another call writes.
"""

from typing import Dict, List

import torch

from ..cache.manager import CacheGroupSpec, StateSpec
from ..config.spec import ModelSpec
from ..ops import kernels
from ..parts import (ARRANGEMENTS, EMBEDDINGS, HEADS, NORMS, POSITIONS, ROLES, CacheView,
                     PagedKVSpec, SlotStateSpec, build_part)
from ..weights.loader import ParamSpec


class DecoderModel:
    def __init__(self, spec: ModelSpec, dtype: torch.dtype, device):
        self.spec = spec
        self.dtype = dtype
        self.device = torch.device(device)
        common = dict(width=spec.width, dtype=dtype)
        self.position = build_part(POSITIONS, "position encoding", spec.position, **common)
        self.embedding = build_part(EMBEDDINGS, "embedding", spec.embedding,
                                    vocab_size=spec.vocab_size, **common)
        self.head = build_part(HEADS, "output head", spec.head, vocab_size=spec.vocab_size,
                               tied=spec.tie_head, **common)
        self.blocks = []
        for block_spec in spec.blocks:
            if block_spec.arrangement not in ARRANGEMENTS:
                raise KeyError(f"unknown block arrangement {block_spec.arrangement!r}; "
                               f"known: {', '.join(sorted(ARRANGEMENTS))}")
            arrangement = ARRANGEMENTS[block_spec.arrangement]
            parts = {}
            for name, role in arrangement.roles.items():
                if role not in ROLES:
                    raise KeyError(f"arrangement {block_spec.arrangement!r} gives part {name!r} the "
                                   f"unknown role {role!r}; known: {', '.join(sorted(ROLES))}")
                parts[name] = build_part(ROLES[role], f"{role} ({name})", block_spec.part(name), **common)
                if role == "mixer":
                    parts[name].set_position(self.position)
            unknown = [name for name, _ in block_spec.parts if name not in arrangement.roles]
            if unknown:
                raise KeyError(f"arrangement {block_spec.arrangement!r} has no part named "
                               f"{', '.join(unknown)}; it has: {', '.join(arrangement.roles)}")
            self.blocks.append(arrangement(width=spec.width, dtype=dtype, parts=parts))
        self.final_norm = build_part(NORMS, "norm", spec.final_norm, **common)
        # Queries of a prompt portion are handed to the mixers in tiles; each mixer says which
        # size (or sizes) its kernel takes, and the step lists the tiles once per size that is
        # asked for.
        sizes = set()
        for block in self.blocks:
            asked = getattr(block.mixer, "query_tile", None)
            if asked:
                sizes.update(int(size) for size in (asked if isinstance(asked, (tuple, list)) else (asked,)))
        self.query_tiles = tuple(sorted(sizes))
        # the mixer of the call that writes a cache entry decides what the entry holds
        self._entry_spec = {}
        for call in spec.schedule:
            if call.writes_cache:
                self._entry_spec[call.cache] = self.blocks[call.block].mixer.cache_spec()
        for call in spec.schedule:
            mine = self.blocks[call.block].mixer.cache_spec()
            if not call.writes_cache and mine != self._entry_spec[call.cache]:
                raise ValueError(
                    f"block {call.block} reads cache entry {call.cache}, whose writer keeps "
                    f"{self._entry_spec[call.cache]}, but needs {mine}")

    # ------------------------------------------------------------- parameters
    def _named_parts(self):
        """(prefix of the parameter paths, part) of every part that may own parameters."""
        yield "embedding.", self.embedding
        yield "position.", self.position
        for index, block in enumerate(self.blocks):
            for part_name, part in block.parts().items():
                yield f"blocks.{index}.{part_name}.", part
        yield "final_norm.", self.final_norm
        yield "head.", self.head

    def parameters(self) -> Dict[str, ParamSpec]:
        return {prefix + name: spec for prefix, part in self._named_parts()
                for name, spec in part.parameters().items()}

    def bind(self, tensors: Dict[str, torch.Tensor]):
        for prefix, part in self._named_parts():
            mine = {name: tensors[prefix + name] for name in part.parameters()}
            if part is self.head:
                # a tied head is the token table itself, not a copy
                # (src/model/paged_decoder.py:300-301)
                part.bind(mine, embedding_table=tensors["embedding.table"])
            else:
                part.bind(mine)
        self.tensors = dict(tensors)     # parameter path -> the tensor that was bound (no copies)
        self.parameter_bytes = sum(t.numel() * t.element_size() for t in tensors.values())
        self.parameter_count = sum(t.numel() for t in tensors.values())

    # ------------------------------------------------------------------ cache
    def cache_requirements(self):
        """Cache groups (entries of equal geometry share a pool) and state tensors."""
        by_geometry: Dict[tuple, List[int]] = {}
        states = []
        for entry in sorted(self._entry_spec):
            spec = self._entry_spec[entry]
            if isinstance(spec, PagedKVSpec):
                by_geometry.setdefault((spec.kv_heads, spec.head_dim, spec.window, spec.value_dim),
                                       []).append(entry)
            elif isinstance(spec, SlotStateSpec):
                states.append(StateSpec(entry, tuple(spec.shape), spec.dtype))
            elif spec is not None:
                raise TypeError(f"unknown cache spec {spec!r}")
        groups = [CacheGroupSpec(tuple(entries), kv_heads, head_dim, window, value_dim)
                  for (kv_heads, head_dim, window, value_dim), entries in by_geometry.items()]
        return groups, states

    def cache_views(self, cache) -> List[CacheView]:
        """One view per call of the run list, in order."""
        views = []
        for call in self.spec.schedule:
            spec = self._entry_spec[call.cache]
            view = CacheView(entry=call.cache, writes=call.writes_cache)
            if isinstance(spec, PagedKVSpec):
                view.group = cache.entry_group(call.cache)
                view.k_pool, view.v_pool = cache.entry_pools(call.cache)
            elif isinstance(spec, SlotStateSpec):
                view.state = cache.state(call.cache)
            views.append(view)
        return views

    # ---------------------------------------------------------------- forward
    @property
    def graph_safe(self) -> bool:
        """Whether a step of this model may be recorded and replayed as a graph: every part
        says so of itself."""
        parts = [self.embedding, self.position, self.final_norm, self.head] + list(self.blocks)
        return all(getattr(part, "graph_safe", False) for part in parts)

    def forward(self, ctx, views, logit_rows, logits_out, choose=None):
        """Run the step's tokens; write logits of ``logit_rows`` (int32 indices into the
        step's tokens) into the float tensor ``logits_out``.  ``choose = (kernels.TopChoice,
        tokens)``: a head that can also writes each row's most likely token into ``tokens``;
        ``self.tokens_chosen`` says whether it did."""
        self.tokens_chosen = False
        tokens = ctx.tokens
        h = ctx.workspace.first_rows("residual", self.spec.width, torch.float32, tokens)
        self.embedding.forward(ctx, self.position.embedding_table(), h)
        for call, view in zip(self.spec.schedule, views):
            self.blocks[call.block].forward(h, ctx, view)
        wanted = logit_rows.numel()
        if wanted == 0:
            return logits_out[:0]
        final = ctx.workspace.first_rows("final", self.spec.width, self.dtype, wanted)
        normed = None
        if getattr(self.head, "accepts_pending_norm", False):
            normed = self.final_norm.pending(h, final, rows=logit_rows)
        if normed is None:
            normed = self.final_norm.forward(h, final, rows=logit_rows)
        out = logits_out[:wanted]
        if choose is not None and getattr(self.head, "chooses_tokens", False):
            self.tokens_chosen = bool(self.head.forward(normed, out, choose=choose))
        else:
            self.head.forward(normed, out)
        return out
