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
from ..parts import (ARRANGEMENTS, FEED_FORWARDS, MIXERS, NORMS, POSITIONS, CacheView,
                     PagedKVSpec, SlotStateSpec, build_part)
from ..weights.loader import MATRIX, TABLE, ParamSpec


class DecoderModel:
    def __init__(self, spec: ModelSpec, dtype: torch.dtype, device):
        self.spec = spec
        self.dtype = dtype
        self.device = torch.device(device)
        common = dict(width=spec.width, dtype=dtype)
        self.position = build_part(POSITIONS, "position encoding", spec.position, **common)
        self.blocks = []
        for block_spec in spec.blocks:
            if block_spec.arrangement not in ARRANGEMENTS:
                raise KeyError(f"unknown block arrangement {block_spec.arrangement!r}; "
                               f"known: {', '.join(sorted(ARRANGEMENTS))}")
            mixer = build_part(MIXERS, "mixer", block_spec.mixer, **common)
            mixer.set_position(self.position)
            block = ARRANGEMENTS[block_spec.arrangement](
                width=spec.width, dtype=dtype,
                norm1=build_part(NORMS, "norm", block_spec.norm1, **common),
                mixer=mixer,
                norm2=build_part(NORMS, "norm", block_spec.norm2, **common),
                feed_forward=build_part(FEED_FORWARDS, "feed-forward", block_spec.feed_forward,
                                        **common))
            self.blocks.append(block)
        self.final_norm = build_part(NORMS, "norm", spec.final_norm, **common)
        self.embedding_table = None
        self.head_weight = None
        self.head_packed = None
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
    def parameters(self) -> Dict[str, ParamSpec]:
        params = {"embedding.table": ParamSpec((self.spec.vocab_size, self.spec.width), TABLE)}
        for name, spec in self.position.parameters().items():
            params[f"position.{name}"] = spec
        for index, block in enumerate(self.blocks):
            for part_name, part in block.parts().items():
                for name, spec in part.parameters().items():
                    params[f"blocks.{index}.{part_name}.{name}"] = spec
        for name, spec in self.final_norm.parameters().items():
            params[f"final_norm.{name}"] = spec
        if not self.spec.tie_head:
            params["head.weight"] = ParamSpec((self.spec.vocab_size, self.spec.width), MATRIX)
        return params

    def bind(self, tensors: Dict[str, torch.Tensor]):
        def take(prefix, part):
            part.bind({name: tensors[prefix + name] for name in part.parameters()})

        self.embedding_table = tensors["embedding.table"]
        take("position.", self.position)
        for index, block in enumerate(self.blocks):
            for part_name, part in block.parts().items():
                take(f"blocks.{index}.{part_name}.", part)
        take("final_norm.", self.final_norm)
        # the tied head is the embedding table itself, not a copy
        # (src/model/paged_decoder.py:300-301)
        self.head_weight = self.embedding_table if self.spec.tie_head else tensors["head.weight"]
        self.head_packed = kernels.pack_decode_weight(self.head_weight)
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
                by_geometry.setdefault((spec.kv_heads, spec.head_dim, spec.window), []).append(entry)
            elif isinstance(spec, SlotStateSpec):
                states.append(StateSpec(entry, tuple(spec.shape), spec.dtype))
            elif spec is not None:
                raise TypeError(f"unknown cache spec {spec!r}")
        groups = [CacheGroupSpec(tuple(entries), kv_heads, head_dim, window)
                  for (kv_heads, head_dim, window), entries in by_geometry.items()]
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
        parts = [self.position, self.final_norm] + list(self.blocks)
        return all(getattr(part, "graph_safe", False) for part in parts)

    def forward(self, ctx, views, logit_rows, logits_out):
        """Run the step's tokens; write logits of ``logit_rows`` (int32 indices into the
        step's tokens) into the float tensor ``logits_out``."""
        tokens = ctx.tokens
        h = ctx.workspace.rows("residual", self.spec.width, torch.float32)[:tokens]
        kernels.embed(self.embedding_table, self.position.embedding_table(), ctx.token_ids,
                      ctx.positions, h, token_src=ctx.token_src, carried=ctx.carried_tokens)
        for call, view in zip(self.spec.schedule, views):
            self.blocks[call.block].forward(h, ctx, view)
        wanted = logit_rows.numel()
        if wanted == 0:
            return logits_out[:0]
        final = ctx.workspace.rows("final", self.spec.width, self.dtype)[:wanted]
        pending = self.final_norm.pending(h, final, rows=logit_rows)
        if pending is None:
            pending = self.final_norm.forward(h, final, rows=logit_rows)
        # logits = f @ table^T without bias, always float
        # (src/model/paged_decoder.py:295-301,605)
        out = logits_out[:wanted]
        kernels.linear(pending, self.head_weight, None, out, packed=self.head_packed)
        return out
