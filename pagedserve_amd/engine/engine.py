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
from ..ops import kernels
from ..parts.base import StepContext, StepItem, Workspace


@dataclass
class StepEntry:
    """One request's next tokens and the places among them whose logits are wanted."""

    request_id: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = field(default_factory=list)
    # The one token of this entry is not known to the host yet: it is the token that the last
    # step chose on the device for its row ``carry``.  ``tokens`` then holds a placeholder.
    carry: Optional[int] = None


@dataclass
class StepOutput:
    logits: torch.Tensor            # float32 [wanted, vocab]; valid until the next step
    rows: List[tuple]               # (request_id, position) of each row
    tokens: Optional[torch.Tensor] = None   # int32 [wanted]: argmax of each row, if asked for
    # a copy of ``tokens`` in pinned host memory, complete once ``ready`` has happened; it is
    # overwritten by the second next step that chooses tokens
    host_tokens: Optional[torch.Tensor] = None
    ready: Optional[torch.cuda.Event] = None

    def token_list(self) -> List[int]:
        """The chosen tokens on the host (waits for this step only, not for later ones)."""
        if self.host_tokens is not None:
            self.ready.synchronize()
            return self.host_tokens.tolist()
        return self.tokens.tolist()


class _ReplayPlan:
    """What a captured decode step needs on later steps: where each index array lies in the
    packed buffer (numpy views for both staging buffers), the copy to the device, the graph
    and its outputs.  Replaying fills a few arrays, copies once and launches once."""

    def __init__(self, graph, used, sections, logits, tokens, items):
        self.graph = graph
        self.used = used
        self.sections = sections       # per staging buffer: dict name -> numpy view
        self.logits = logits
        self.tokens = tokens
        self.items = items


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
        # queries of an item with several tokens are listed in tiles, once for every tile size
        # that a mixer of the model asks for (none: no mixer wants tiles)
        self.query_tiles = tuple(getattr(model, "query_tiles", ()))
        capacity = ((7 + 2 * max(1, len(self.query_tiles))) * max_step_tokens + 5 * max_requests + 1
                    + len(groups) * max_requests * self.table_width + 16)
        self._meta_device = torch.empty(capacity, dtype=torch.int32, device=self.device)
        self._meta_host = [torch.empty(capacity, dtype=torch.int32, pin_memory=True) for _ in range(2)]
        self._meta_events = [torch.cuda.Event(), torch.cuda.Event()]
        self._meta_pending = [False, False]
        self._meta_owner = [None, None]   # replay plan whose constant arrays a buffer holds
        self._meta_turn = 0
        self._logits = None
        # chosen tokens: one per wanted row, and a step wants at most one row per token
        self._tokens = torch.zeros(max(max_requests, max_step_tokens), dtype=torch.int32,
                                   device=self.device)
        self._tokens_host = [torch.zeros(self._tokens.numel(), dtype=torch.int32, pin_memory=True)
                             for _ in range(2)]
        self._tokens_ready = [torch.cuda.Event(), torch.cuda.Event()]
        self._tokens_turn = 0
        from ..ops import kernels

        self._top_choice = kernels.TopChoice(min(self._tokens.numel(), 64), self.device)
        self.tokens_chosen_by_head = 0   # greedy steps (launched or recorded) without a sampling launch
        self._carried_rows = 0    # rows of the last step whose chosen tokens a step may carry on
        # The engine's work runs on a stream of its own (default priority): a capture cannot
        # record from the default stream.
        self.stream = torch.cuda.Stream(device=self.device)
        # a part that looks at host values of a step cannot be replayed
        self.use_graphs = use_graphs and getattr(model, "graph_safe", False)
        self.max_graphs = 48     # recorded layouts kept; the least recently replayed goes first
        # direct runs of a layout with a prompt portion before it is recorded (a decode layout
        # is recorded at its second step).  Recording costs as much as a step and a replay of
        # such a step saves the GPU 3 to 5 % of it (the host issues the step faster than the GPU
        # runs it either way), so only a layout that keeps coming back is worth it: in streams
        # of requests, recording at the third return instead cost 5 to 9 % of the throughput.
        self.record_after = 24
        self.max_layouts_remembered = 512
        self._graphs = {}        # key -> StepGraph
        self._graph_seen = {}     # layout -> steps that ran without a graph (buffers exist now)
        self._layouts = {}        # (tokens, items, wanted, singles, tiles) -> offsets, size, device views
        self._graph_failures = {}
        self._workspace_moved = 0
        self._graph_retired = []  # (event, graph): dropped, destroyed once the event has happened
        self.graphs_captured = 0
        self.graphs_evicted = 0
        self._replays_of_dropped = 0
        self.capture_seconds = 0.0
        self.steps = 0

    # ------------------------------------------------------------------ admin
    def is_live(self, request_id) -> bool:
        return request_id in self.cache.requests

    def length(self, request_id) -> int:
        return self.cache.length(request_id)

    def finish(self, request_id):
        """The request is over: its pages and its slot go back."""
        self.cache.release(request_id)

    def graph_summary(self) -> dict:
        """Counters in the manner of src/model/paged_decoder.py:498-507."""
        return {"enabled": self.use_graphs, "captured_graphs": len(self._graphs),
                "captures": self.graphs_captured, "evicted": self.graphs_evicted,
                "capture_seconds": round(self.capture_seconds, 4),
                "layouts_remembered": len(self._graph_seen),
                "graph_replays": self._replays_of_dropped
                + sum(plan.graph.replays for plan in self._graphs.values()),
                "graph_nodes": {str(key): plan.graph.nodes for key, plan in self._graphs.items()},
                "capture_failures": list(self._graph_failures.values())}

    def _logit_buffer(self, rows: int) -> torch.Tensor:
        if self._logits is None or self._logits.shape[0] < rows:
            capacity = max(rows, min(self.max_requests, 64))
            # rows start at multiples of 32 bytes, so that kernels store them in aligned pieces
            vocab = self.spec.vocab_size
            padded = -(-vocab // 8) * 8
            self._logits = torch.empty((capacity, padded), dtype=torch.float32,
                                       device=self.device)[:, :vocab]
        return self._logits

    def _context_class(self, longest: int) -> int:
        """Launch shapes inside a graph must not depend on a step's lengths, but a step whose
        longest context is 200 keys should not be cut into the ranges of one of 1,000: the
        longest cached length of a step falls into a class (128, 256, 512, 1,024, ... keys, the
        last one the model's positions), the class is part of a graph's key, and the parts see
        the class's bound as ``ctx.max_kv_len``.  (128 keys are what four waves take in one go:
        11 to 21 requests of 12 heads over up to 80 keys run 5 % faster as such blocks than as
        the blocks of 16 waves that 256 keys would ask for.  Steps of two, not four: up to
        twelve requests over 270 to 500 keys run 2 to 4 % faster with the ranges of 512 keys
        than with those of 1,024, half of which they leave empty; a layout is recorded once
        more on its way to long contexts.)"""
        bound = 128
        while bound < longest and bound < self.spec.max_positions:
            bound *= 2
        return min(bound, self.spec.max_positions)

    # ------------------------------------------------------------------- step
    def _validate(self, entries):
        if not entries:
            raise StepError("a step needs at least one entry")
        seen = set()
        total = 0
        new = 0
        vocab = self.spec.vocab_size
        requests = self.cache.requests
        max_positions = self.spec.max_positions
        for entry in entries:
            if entry.request_id in seen:
                # src/model/iteration.py:61-63
                raise StepError(f"request {entry.request_id!r} appears twice in one step")
            seen.add(entry.request_id)
            count = len(entry.tokens)
            if count == 1 and entry.want == [0]:
                # a decoded token with its logits wanted: the short way through the checks below
                record = requests.get(entry.request_id)
                carry = entry.carry
                if (record is not None and 0 <= entry.tokens[0] < vocab
                        and record.length < max_positions
                        and (carry is None or 0 <= carry < self._carried_rows)):
                    total += 1
                    continue
            if count == 0:
                raise StepError(f"request {entry.request_id!r} brings no tokens")
            if count > 16:
                # long portions are checked (and later packed) as arrays, converted once
                if not isinstance(entry.tokens, np.ndarray):
                    entry.tokens = np.asarray(entry.tokens, dtype=np.int64)
                low, high = int(entry.tokens.min()), int(entry.tokens.max())
            else:
                low, high = min(entry.tokens), max(entry.tokens)
            if low < 0 or high >= vocab:
                raise StepError(f"a token of request {entry.request_id!r} is outside "
                                f"the vocabulary of {vocab}")
            if entry.carry is not None and (count != 1 or not 0 <= entry.carry < self._carried_rows):
                raise StepError(f"request {entry.request_id!r} carries on row {entry.carry} of the "
                                f"last step, which chose {self._carried_rows} tokens")
            if entry.want and (min(entry.want) < 0 or max(entry.want) >= count):
                raise StepError(f"request {entry.request_id!r} wants logits at place "
                                f"{max(entry.want)} of {count} tokens")
            if len(set(entry.want)) != len(entry.want):
                # (the index buffers hold one wanted row per token at most)
                raise StepError(f"request {entry.request_id!r} wants logits at the same place twice")
            record = self.cache.requests.get(entry.request_id)
            have = record.length if record is not None else 0
            new += record is None
            if have + count > self.spec.max_positions:
                # src/model/paged_decoder.py:521-522
                raise StepError(f"request {entry.request_id!r} would reach position "
                                f"{have + count - 1}, the model has {self.spec.max_positions}")
            total += count
        if total > self.max_step_tokens:
            raise StepError(f"step of {total} tokens exceeds max_step_tokens={self.max_step_tokens}")
        if len(self.cache.requests) + new > self.max_requests:
            raise StepError(f"more than {self.max_requests} live requests")

    supports_draws = True

    def step(self, entries: Sequence[StepEntry], greedy: bool = False, draws=None) -> StepOutput:
        """Run one batch.  With ``greedy`` the argmax of every wanted row is computed on the
        GPU as part of the step (inside the graph of a replayed decode step) and returned as
        ``StepOutput.tokens``.  With ``draws``, one ``(1 / temperature, uniform number)`` per
        wanted row, each row's token is drawn there instead (argmax where the first is 0)."""
        entries = list(entries)
        self._validate(entries)
        if draws is not None:
            draws = [(float(a), float(b)) for a, b in draws]
            if len(draws) != sum(len(entry.want) for entry in entries):
                raise StepError(f"{len(draws)} draws for {sum(len(e.want) for e in entries)} wanted rows")
            greedy = draws
        admitted = []
        cache = self.cache
        try:
            for entry in entries:
                record = cache.requests.get(entry.request_id)
                if record is None:
                    cache.admit(entry.request_id)
                    admitted.append(entry.request_id)
                    record = cache.requests[entry.request_id]
                needed = record.length + len(entry.tokens)
                if needed > record.capacity:
                    cache.grow(entry.request_id, needed)
            caller = torch.cuda.current_stream(self.device)
            if caller.cuda_stream == self.stream.cuda_stream:
                with kernels.on_stream(self.stream):
                    output = self._run(entries, greedy)
            else:
                # the caller may still be reading the last step's logits
                self.stream.wait_stream(caller)
                with torch.cuda.stream(self.stream), kernels.on_stream(self.stream):
                    output = self._run(entries, greedy)
                caller.wait_stream(self.stream)
        except Exception:
            # requests that this step admitted leave no trace
            # (src/scheduler/orca_scheduler.py:243-247), and no later step may carry on rows
            # of a step before this one
            for request_id in admitted:
                cache.release(request_id)
            self._carried_rows = 0
            raise
        for entry in entries:
            cache.commit(entry.request_id, cache.requests[entry.request_id].length + len(entry.tokens))
        self.steps += 1
        return output

    def _pack(self, entries, select=None):
        """Fill the packed index buffer on the host, copy it, and return the step context.

        The layout depends only on (tokens, items, wanted rows, one-token items)."""
        cache = self.cache
        counts = [len(entry.tokens) for entry in entries]
        tokens = sum(counts)
        items = len(entries)
        wants = [len(entry.want) for entry in entries]
        wanted = sum(wants)
        singles = counts.count(1)
        # items with several tokens are cut into tiles of queries for the mixers' tiled kernels
        tile_sizes = self.query_tiles
        tiles = tuple(sum(-(-count // tile) for count in counts if count > 1) for tile in tile_sizes)
        groups = len(cache.groups)
        width = self.table_width
        # where each index array lies, and the device views of them, are the same for every
        # step of a layout: they are made once
        layout_key = (tokens, items, wanted, singles, tiles)
        layout = self._layouts.get(layout_key)
        if layout is None:
            offsets = {}
            cursor = 0
            for name, size in (("token_ids", tokens), ("token_src", tokens), ("positions", tokens),
                               ("tok_item", tokens),
                               ("cu_tokens", items + 1), ("kv_lens", items), ("slots", items),
                               ("rows", wanted), ("inv_temperature", wanted), ("uniform", wanted),
                               ("single_tokens", singles),
                               ("portion_tokens", tokens - singles)):
                offsets[name] = (cursor, size)
                cursor += size
            for tile, count in zip(tile_sizes, tiles):
                for name in (f"tile_item{tile}", f"tile_q0{tile}"):
                    offsets[name] = (cursor, count)
                    cursor += count
            for group in range(groups):
                offsets[f"tables{group}"] = (cursor, items * width)
                cursor += items * width
            views = {name: self._meta_device[begin:begin + size]
                     for name, (begin, size) in offsets.items()}
            for group in range(groups):
                views[f"tables{group}"] = views[f"tables{group}"].view(items, width)
            for name in ("inv_temperature", "uniform"):
                views[name] = views[name].view(torch.float32)
            if len(self._layouts) >= 512:
                self._layouts.clear()
            layout = self._layouts[layout_key] = (offsets, cursor, views)
        offsets, cursor, views = layout
        turn = self._meta_turn
        self._meta_turn ^= 1
        if self._meta_pending[turn]:
            self._meta_events[turn].synchronize()
        self._meta_owner[turn] = None
        host = self._meta_host[turn].numpy()

        def section(name):
            begin, size = offsets[name]
            return host[begin:begin + size]

        records = [cache.requests[entry.request_id] for entry in entries]
        starts = [record.length for record in records]
        slot_list = [record.slot for record in records]
        section("slots")[:] = slot_list
        token_src = section("token_src")
        token_src[:] = -1
        step_items = []
        row_keys = []
        if tokens == items:
            # every item brings one token: no per-item loops over numpy slices
            section("token_ids")[:] = [entry.tokens[0] for entry in entries]
            token_src[:] = [-1 if entry.carry is None else entry.carry for entry in entries]
            section("positions")[:] = starts
            index = np.arange(items + 1, dtype=np.int32)
            section("tok_item")[:] = index[:items]
            section("cu_tokens")[:] = index
            section("kv_lens")[:] = [start + 1 for start in starts]
            section("single_tokens")[:] = index[:items]
            rows = section("rows")
            row_cursor = 0
            for flat, (entry, record, start) in enumerate(zip(entries, records, starts)):
                if entry.want:
                    rows[row_cursor] = flat
                    row_keys.append((entry.request_id, start))
                    row_cursor += 1
                step_items.append(StepItem(entry.request_id, record.slot, start, 1, flat))
            max_kv = max(starts) + 1
        else:
            token_ids, positions = section("token_ids"), section("positions")
            tok_item, cu, kv_lens = section("tok_item"), section("cu_tokens"), section("kv_lens")
            rows = section("rows")
            single_tokens, portion_tokens = section("single_tokens"), section("portion_tokens")
            tile_lists = [(tile, section(f"tile_item{tile}"), section(f"tile_q0{tile}"))
                          for tile in tile_sizes]
            tile_cursors = [0] * len(tile_sizes)
            flat = row_cursor = single_cursor = portion_cursor = max_kv = 0
            for index, (entry, record, start, count) in enumerate(zip(entries, records, starts, counts)):
                token_ids[flat:flat + count] = entry.tokens
                if entry.carry is not None:
                    token_src[flat] = entry.carry
                positions[flat:flat + count] = np.arange(start, start + count, dtype=np.int32)
                tok_item[flat:flat + count] = index
                cu[index] = flat
                kv_lens[index] = start + count
                max_kv = max(max_kv, start + count)
                if count == 1:
                    single_tokens[single_cursor] = flat
                    single_cursor += 1
                else:
                    portion_tokens[portion_cursor:portion_cursor + count] = np.arange(
                        flat, flat + count, dtype=np.int32)
                    portion_cursor += count
                    for which, (tile, tile_item, tile_q0) in enumerate(tile_lists):
                        here = -(-count // tile)
                        at = tile_cursors[which]
                        tile_item[at:at + here] = index
                        tile_q0[at:at + here] = np.arange(0, count, tile, dtype=np.int32)
                        tile_cursors[which] = at + here
                for place in entry.want:
                    rows[row_cursor] = flat + int(place)
                    row_keys.append((entry.request_id, start + int(place)))
                    row_cursor += 1
                step_items.append(StepItem(entry.request_id, record.slot, start, count, flat))
                flat += count
            cu[items] = flat
            for (tile, tile_item, tile_q0), filled in zip(tile_lists, tile_cursors):
                if filled > 1:
                    # tiles that see the most keys first: the kernel's blocks start in this
                    # order, and the longest should not be the last to start
                    keys = np.asarray(starts, dtype=np.int64)[tile_item] + tile_q0
                    order = np.argsort(-keys, kind="stable")
                    tile_item[:] = tile_item[order]
                    tile_q0[:] = tile_q0[order]
        if isinstance(select, list):
            section("inv_temperature").view(np.float32)[:] = [a for a, _ in select]
            section("uniform").view(np.float32)[:] = [b for _, b in select]
        slot_index = np.asarray(slot_list, dtype=np.int64)
        for group in range(groups):
            section(f"tables{group}").reshape(items, width)[:] = cache.table_arrays[group][slot_index]
        device = self._meta_device
        device[:cursor].copy_(self._meta_host[turn][:cursor], non_blocking=True)
        self._meta_events[turn].record()
        self._meta_pending[turn] = True
        self._last_layout = (offsets, cursor)

        ctx = StepContext(
            tokens=tokens, dtype=self.dtype, device=self.device, items=step_items,
            token_ids=views["token_ids"], positions=views["positions"], tok_item=views["tok_item"],
            cu_tokens=views["cu_tokens"], kv_lens=views["kv_lens"], slots=views["slots"],
            tables=[views[f"tables{group}"] for group in range(groups)],
            page_size=self.page_size, workspace=self.workspace,
            decode_only=singles == items, max_kv_len=max_kv,
            single_tokens=views["single_tokens"], portion_tokens=views["portion_tokens"],
            max_positions=self.spec.max_positions,
            query_tiles={tile: (views[f"tile_item{tile}"], views[f"tile_q0{tile}"])
                         for tile in tile_sizes},
            token_src=views["token_src"], carried_tokens=self._tokens)
        self._draw_views = (views["inv_temperature"], views["uniform"])
        return ctx, views["rows"], row_keys

    def _forward(self, ctx, rows, logits, wanted, greedy):
        from ..ops import kernels

        if not (greedy and wanted):
            return self.model.forward(ctx, self.views, rows, logits), None
        tokens = self._tokens[:wanted]
        if isinstance(greedy, list):
            out = self.model.forward(ctx, self.views, rows, logits)
            inv_temperature, uniform = self._draw_views
            return out, kernels.sample(out, inv_temperature, uniform, tokens)
        # the most likely token: chosen by the head's own kernel where it can
        out = self.model.forward(ctx, self.views, rows, logits, choose=(self._top_choice, tokens))
        if self.model.tokens_chosen:
            self.tokens_chosen_by_head += 1
        else:
            kernels.sample(out, None, None, tokens)
        return out, tokens

    def _run(self, entries, greedy=False) -> StepOutput:
        output = self._run_step(entries, greedy)
        if output.tokens is not None:
            # the chosen tokens go to the host behind the step, without holding up the next one
            turn = self._tokens_turn
            self._tokens_turn ^= 1
            rows = output.tokens.numel()
            output.host_tokens = self._tokens_host[turn][:rows]
            output.host_tokens.copy_(output.tokens, non_blocking=True)
            output.ready = self._tokens_ready[turn]
            output.ready.record()
            self._carried_rows = rows
        else:
            self._carried_rows = 0
        return output

    def _run_step(self, entries, greedy=False) -> StepOutput:
        """Steps of one layout (numbers of tokens, items, wanted rows, one-token items and
        query tiles, and how tokens are chosen) issue the same launches with the same
        arguments: everything else lies in the packed index buffer.  The first step of a
        layout runs directly (buffers get allocated), the second is recorded as a HIP graph,
        later ones copy their indices and replay it."""
        items = len(entries)
        mode = 2 if isinstance(greedy, list) else int(bool(greedy))   # how tokens are chosen
        if self._graphs and self.workspace.moved != self._workspace_moved:
            # a scratch buffer was replaced by a larger one: recorded launches hold the old address
            for plan in self._graphs.values():
                self._retire_graph(plan)
            self._graphs.clear()
            self._graph_seen.clear()
        self._workspace_moved = self.workspace.moved
        if self.use_graphs and self._graphs:
            # every entry brings one token and wants its logits: the lean path
            requests = self.cache.requests
            longest = 1 + max(requests[entry.request_id].length for entry in entries)
            key = (items, items, items, items, 0, mode, self._context_class(longest))
            plan = self._graphs.get(key)
            if (plan is not None and plan.logits.data_ptr() == self._logit_buffer(items).data_ptr()
                    and all(len(e.tokens) == 1 and len(e.want) == 1 for e in entries)):
                self._used(key, plan)
                return self._replay(plan, entries, greedy)
        ctx, rows, row_keys = self._pack(entries, greedy)
        wanted = len(row_keys)
        logits = self._logit_buffer(wanted)
        singles = ctx.single_tokens.numel()
        kv_class = self._context_class(ctx.max_kv_len)
        tiles = sum(lists[0].numel() for lists in ctx.query_tiles.values())
        graph_key = (ctx.tokens, items, wanted, singles, tiles, mode, kv_class)
        if not self.use_graphs or graph_key in self._graph_failures:
            out, tokens = self._forward(ctx, rows, logits, wanted, greedy)
            return StepOutput(logits=out, rows=row_keys, tokens=tokens)
        # launch shapes inside a graph must not depend on this step's lengths
        exact_kv_len = ctx.max_kv_len
        ctx.max_kv_len = kv_class
        plan = self._graphs.get(graph_key)
        if plan is not None and plan.logits.data_ptr() == logits.data_ptr():
            # recorded: the indices are on their way already (``_pack`` copied them)
            self._used(graph_key, plan)
            plan.graph.launch()
            return StepOutput(logits=plan.logits[:wanted], rows=row_keys, tokens=plan.tokens)
        # The first step of a layout runs directly, so that every buffer exists before a
        # capture.  Recording costs about as much as a few steps: decode layouts come back
        # at once and are recorded at their second step, others when they keep coming back.
        seen_key = graph_key + (logits.data_ptr(),)
        seen = self._graph_seen.get(seen_key, 0)
        if seen < (1 if singles == ctx.tokens else self.record_after):
            # (re-inserted at the end: the layouts that have not come back for longest go first)
            self._graph_seen.pop(seen_key, None)
            self._graph_seen[seen_key] = seen + 1
            while len(self._graph_seen) > self.max_layouts_remembered:
                del self._graph_seen[next(iter(self._graph_seen))]
            out, tokens = self._forward(ctx, rows, logits, wanted, greedy)
            return StepOutput(logits=out, rows=row_keys, tokens=tokens)
        import time

        from ..ops.kernels import StepGraph

        capture_started = time.perf_counter()
        graph = StepGraph()
        StepGraph.begin()
        try:
            out, tokens = self._forward(ctx, rows, logits, wanted, greedy)
            graph.end()
        except Exception as error:       # the capture is abandoned, the step runs directly
            StepGraph.abort()
            self._graph_failures[graph_key] = f"{type(error).__name__}: {error}"
            ctx.max_kv_len = exact_kv_len
            out, tokens = self._forward(ctx, rows, logits, wanted, greedy)
            return StepOutput(logits=out, rows=row_keys, tokens=tokens)
        offsets, used = self._last_layout
        sections = []
        for host in self._meta_host:
            array = host.numpy()
            views = {name: array[begin:begin + size] for name, (begin, size) in offsets.items()}
            for group in range(len(self.cache.groups)):
                views[f"tables{group}"] = views[f"tables{group}"].reshape(items, self.table_width)
            sections.append(views)
        old = self._graphs.pop(graph_key, None)
        if old is not None:
            self._retire_graph(old)
        while len(self._graphs) >= self.max_graphs:
            oldest = next(iter(self._graphs))
            self._retire_graph(self._graphs.pop(oldest))
            self.graphs_evicted += 1
        self._graphs[graph_key] = _ReplayPlan(graph, used, sections, out, tokens, items)
        self.graphs_captured += 1
        self.capture_seconds += time.perf_counter() - capture_started
        graph.launch()
        return StepOutput(logits=out, rows=row_keys, tokens=tokens)

    def _used(self, key, plan):
        """A replayed layout moves to the end of the line: the one dropped when the ring is full
        is the one that has not been replayed for longest, not the one recorded first."""
        if len(self._graphs) > 1:
            del self._graphs[key]
            self._graphs[key] = plan

    def _retire_graph(self, plan):
        """A recorded layout is dropped.  Its last launch may still be running (the engine never
        waits for its stream), so the executable graph is destroyed only after an event
        recorded behind everything launched so far has happened."""
        event = torch.cuda.Event()
        event.record(self.stream)
        self._graph_retired.append((event, plan.graph))
        self._replays_of_dropped += plan.graph.replays
        still_busy = []
        for event, graph in self._graph_retired:
            if event.query():
                graph.destroy()
            else:
                still_busy.append((event, graph))
        self._graph_retired = still_busy

    def _replay(self, plan, entries, select=None) -> StepOutput:
        """A captured decode step: refresh the per-step indices, copy them, launch the graph."""
        cache = self.cache
        turn = self._meta_turn
        self._meta_turn ^= 1
        if self._meta_pending[turn]:
            self._meta_events[turn].synchronize()
        sections = plan.sections[turn]
        items = plan.items
        if self._meta_owner[turn] is not plan:
            # arrays that are the same on every step of this shape
            index = np.arange(items + 1, dtype=np.int32)
            sections["tok_item"][:] = index[:items]
            sections["cu_tokens"][:] = index
            sections["single_tokens"][:] = index[:items]
            sections["rows"][:] = index[:items]
            self._meta_owner[turn] = plan
        records = [cache.requests[entry.request_id] for entry in entries]
        starts = [record.length for record in records]
        slots = [record.slot for record in records]
        sections["token_ids"][:] = [entry.tokens[0] for entry in entries]
        sections["token_src"][:] = [-1 if entry.carry is None else entry.carry for entry in entries]
        sections["positions"][:] = starts
        sections["kv_lens"][:] = [start + 1 for start in starts]
        sections["slots"][:] = slots
        if isinstance(select, list):
            sections["inv_temperature"].view(np.float32)[:] = [a for a, _ in select]
            sections["uniform"].view(np.float32)[:] = [b for _, b in select]
        for group in range(len(cache.groups)):
            sections[f"tables{group}"][:] = cache.table_arrays[group][slots]
        self._meta_device[:plan.used].copy_(self._meta_host[turn][:plan.used], non_blocking=True)
        self._meta_events[turn].record()
        self._meta_pending[turn] = True
        plan.graph.launch()
        rows = [(entry.request_id, start) for entry, start in zip(entries, starts)]
        return StepOutput(logits=plan.logits, rows=rows, tokens=plan.tokens)
