"""The step function: one batch of (request, its next tokens) through the model.

The reference's ``forward_iteration`` (src/model/paged_decoder.py:509-619) takes a flat
token vector with per-request items, checks positions against the cache, runs the
layers once over all tokens and returns logits for the items that produce output.
This engine keeps that contract with two changes of design: pages are taken *before*
the layers run and the kernels store keys and values straight into them, so a prompt
portion, a whole prompt and a decoded token are the same case for attention (a query
at position p reads keys 0..p from the pages); and logits can be asked for at any of
the step's tokens, not only at the last one of an item.

All per-step indices travel to the GPU in one packed int32 copy whose layout depends
only on (tokens, items, wanted rows), so a captured HIP graph of a decode step stays
valid from step to step.
"""

from dataclasses import dataclass, field
from typing import Hashable, List, Optional, Sequence

import numpy as np
import torch

from ..cache.manager import CacheFull, CacheManager
from ..parts.base import StepContext, StepItem, Workspace


@dataclass
class StepEntry:
    """One request's next tokens and the places among them whose logits are wanted."""

    request_id: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = field(default_factory=list)


@dataclass
class StepOutput:
    logits: torch.Tensor            # float32 [wanted, vocab]; valid until the next step
    rows: List[tuple]               # (request_id, position) of each row


class StepError(ValueError):
    """A step that the engine refuses before anything ran."""


class Engine:
    def __init__(self, model, num_pages: int, page_size: int = 16, max_requests: int = 64,
                 max_step_tokens: int = 2048, use_graphs: bool = True):
        if not torch.cuda.is_available():
            raise RuntimeError("pagedserve_amd runs on a GPU only; no CPU path exists")
        self.model = model
        self.spec = model.spec
        self.device = model.device
        self.dtype = model.dtype
        self.page_size = page_size
        self.max_requests = max_requests
        self.max_step_tokens = max_step_tokens
        groups, states = model.cache_requirements()
        self.cache = CacheManager(groups, num_pages, page_size, max_requests, self.dtype,
                                  self.device, states, max_positions=self.spec.max_positions)
        self.views = model.cache_views(self.cache)
        self.workspace = Workspace(max_step_tokens, self.device)
        self.table_width = -(-self.spec.max_positions // page_size)
        capacity = (5 * max_step_tokens + 3 * max_requests + 1
                    + len(groups) * max_requests * self.table_width + 16)
        self._meta_device = torch.empty(capacity, dtype=torch.int32, device=self.device)
        self._meta_host = [torch.empty(capacity, dtype=torch.int32, pin_memory=True) for _ in range(2)]
        self._meta_events = [None, None]
        self._meta_turn = 0
        self._logits = None
        self.use_graphs = use_graphs
        self.steps = 0

    # ------------------------------------------------------------------ admin
    def is_live(self, request_id) -> bool:
        return request_id in self.cache.requests

    def length(self, request_id) -> int:
        return self.cache.length(request_id)

    def finish(self, request_id):
        """The request is over: its pages and its slot go back."""
        self.cache.release(request_id)

    def _logit_buffer(self, rows: int) -> torch.Tensor:
        if self._logits is None or self._logits.shape[0] < rows:
            capacity = max(rows, min(self.max_requests, 64))
            self._logits = torch.empty((capacity, self.spec.vocab_size), dtype=torch.float32,
                                       device=self.device)
        return self._logits

    # ------------------------------------------------------------------- step
    def _validate(self, entries):
        if not entries:
            raise StepError("a step needs at least one entry")
        seen = set()
        total = 0
        for entry in entries:
            if entry.request_id in seen:
                # src/model/iteration.py:61-63
                raise StepError(f"request {entry.request_id!r} appears twice in one step")
            seen.add(entry.request_id)
            count = len(entry.tokens)
            if count == 0:
                raise StepError(f"request {entry.request_id!r} brings no tokens")
            for token in entry.tokens:
                if not 0 <= int(token) < self.spec.vocab_size:
                    raise StepError(f"token {token} of request {entry.request_id!r} is outside "
                                    f"the vocabulary of {self.spec.vocab_size}")
            for index in entry.want:
                if not 0 <= int(index) < count:
                    raise StepError(f"request {entry.request_id!r} wants logits at place {index} "
                                    f"of {count} tokens")
            have = self.cache.length(entry.request_id) if self.is_live(entry.request_id) else 0
            if have + count > self.spec.max_positions:
                # src/model/paged_decoder.py:521-522
                raise StepError(f"request {entry.request_id!r} would reach position "
                                f"{have + count - 1}, the model has {self.spec.max_positions}")
            total += count
        if total > self.max_step_tokens:
            raise StepError(f"step of {total} tokens exceeds max_step_tokens={self.max_step_tokens}")
        new = sum(1 for entry in entries if not self.is_live(entry.request_id))
        if len(self.cache.requests) + new > self.max_requests:
            raise StepError(f"more than {self.max_requests} live requests")

    def step(self, entries: Sequence[StepEntry]) -> StepOutput:
        entries = list(entries)
        self._validate(entries)
        admitted = []
        try:
            for entry in entries:
                if not self.is_live(entry.request_id):
                    self.cache.admit(entry.request_id)
                    admitted.append(entry.request_id)
                self.cache.grow(entry.request_id,
                                self.cache.length(entry.request_id) + len(entry.tokens))
            output = self._run(entries)
        except Exception:
            # requests that this step admitted leave no trace
            # (src/scheduler/orca_scheduler.py:243-247)
            for request_id in admitted:
                self.cache.release(request_id)
            raise
        for entry in entries:
            self.cache.commit(entry.request_id,
                              self.cache.length(entry.request_id) + len(entry.tokens))
        self.steps += 1
        return output

    def _pack(self, entries):
        """Fill the packed index buffer on the host; returns views of the device copy."""
        tokens = sum(len(entry.tokens) for entry in entries)
        items = len(entries)
        wanted = sum(len(entry.want) for entry in entries)
        singles = sum(1 for entry in entries if len(entry.tokens) == 1)
        groups = len(self.cache.groups)
        width = self.table_width
        offsets = {}
        cursor = 0
        for name, size in (("token_ids", tokens), ("positions", tokens), ("tok_item", tokens),
                           ("cu_tokens", items + 1), ("kv_lens", items), ("slots", items),
                           ("rows", wanted), ("single_tokens", singles),
                           ("portion_tokens", tokens - singles)):
            offsets[name] = (cursor, size)
            cursor += size
        for group in range(groups):
            offsets[f"tables{group}"] = (cursor, items * width)
            cursor += items * width
        turn = self._meta_turn
        self._meta_turn ^= 1
        if self._meta_events[turn] is not None:
            self._meta_events[turn].synchronize()
        host = self._meta_host[turn].numpy()

        def section(name):
            begin, size = offsets[name]
            return host[begin:begin + size]

        token_ids, positions, tok_item = section("token_ids"), section("positions"), section("tok_item")
        cu, kv_lens, slots, rows = section("cu_tokens"), section("kv_lens"), section("slots"), section("rows")
        single_tokens, portion_tokens = section("single_tokens"), section("portion_tokens")
        tables = [section(f"tables{group}").reshape(items, width) for group in range(groups)]
        for table in tables:
            table.fill(-1)
        step_items = []
        row_keys = []
        flat = 0
        row_cursor = 0
        max_kv = 0
        single_cursor = 0
        portion_cursor = 0
        for index, entry in enumerate(entries):
            record = self.cache.requests[entry.request_id]
            count = len(entry.tokens)
            start = record.length
            token_ids[flat:flat + count] = np.asarray(entry.tokens, dtype=np.int32)
            positions[flat:flat + count] = np.arange(start, start + count, dtype=np.int32)
            tok_item[flat:flat + count] = index
            cu[index] = flat
            kv_lens[index] = start + count
            max_kv = max(max_kv, start + count)
            slots[index] = record.slot
            for group, table in enumerate(tables):
                pages = record.tables[group]
                table[index, :len(pages)] = pages
            for place in entry.want:
                rows[row_cursor] = flat + int(place)
                row_keys.append((entry.request_id, start + int(place)))
                row_cursor += 1
            if count == 1:
                single_tokens[single_cursor] = flat
                single_cursor += 1
            else:
                portion_tokens[portion_cursor:portion_cursor + count] = np.arange(
                    flat, flat + count, dtype=np.int32)
                portion_cursor += count
            step_items.append(StepItem(entry.request_id, record.slot, start, count, flat))
            flat += count
        cu[items] = flat
        device = self._meta_device
        device[:cursor].copy_(self._meta_host[turn][:cursor], non_blocking=True)
        event = torch.cuda.Event()
        event.record()
        self._meta_events[turn] = event

        def view(name):
            begin, size = offsets[name]
            return device[begin:begin + size]

        ctx = StepContext(
            tokens=tokens, dtype=self.dtype, device=self.device, items=step_items,
            token_ids=view("token_ids"), positions=view("positions"), tok_item=view("tok_item"),
            cu_tokens=view("cu_tokens"), kv_lens=view("kv_lens"), slots=view("slots"),
            tables=[view(f"tables{group}").view(items, width) for group in range(groups)],
            page_size=self.page_size, workspace=self.workspace,
            decode_only=singles == items, max_kv_len=max_kv,
            single_tokens=view("single_tokens"), portion_tokens=view("portion_tokens"),
            max_positions=self.spec.max_positions)
        return ctx, view("rows"), row_keys

    def _run(self, entries) -> StepOutput:
        ctx, rows, row_keys = self._pack(entries)
        logits = self._logit_buffer(len(row_keys))
        out = self.model.forward(ctx, self.views, rows, logits)
        return StepOutput(logits=out, rows=row_keys)
