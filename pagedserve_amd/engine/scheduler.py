"""Continuous batching above the step function.

Queues and life cycle follow the reference's ``ContinuousBatchScheduler``
(src/scheduler/orca_scheduler.py:32-303): requests wait until their whole prompt is
cached, then decode one token per iteration until ``max_new_tokens`` or the end token,
then give back what they hold.  Two selection strategies:

* ``orca``: requests in arrival order, decoding ones with their single token and
  waiting ones with their whole remaining prompt (``:128-146,187-188``);
* ``sarathi``: all decoding requests first, then prompt portions of at most
  ``prefill_chunk_size`` tokens (``:148-169,182-186``), one prefilling request per
  iteration as in the reference unless ``max_prefill_requests`` allows more.

Both run under a token budget per iteration (``max_num_batched_tokens``, at most what the
engine's buffers hold): a prompt that does not fit the budget is cut there and continues
in the next iteration.  The reference has no such budget; its iterations are bounded by
the number of requests only.

**When pages run out.**  A request is admitted only if the pages of its worst case
(``prompt + max_new_tokens`` tokens, in every cache group) fit beside what admitted
requests have reserved (``:119-122,138-142``); otherwise it and everything behind it wait
(first come, first served).  So a running request never fails for lack of pages, and
nothing is preempted.  A request whose worst case exceeds the whole pool is refused when
it is added.

**Running ahead.**  While every running request decodes and nobody waits, the
iteration after the current one is launched before the current one's tokens have reached
the host: its entries say "the token that the last step chose for row r" instead of a token
id, and the host's work for an iteration overlaps the GPU's work for the next.  A request
that ends by length is known beforehand and left out; one that ends at the end token has one
token too many computed, which is dropped.  The tokens that a request receives are the same
either way.
"""

from collections import deque
from dataclasses import dataclass, field
from typing import Dict, List, Optional

from ..sampling.params import SamplingParams, fresh_seed
from .engine import StepEntry

ORCA_STRATEGY = "orca"
SARATHI_STRATEGY = "sarathi"
SUPPORTED_SCHEDULING_STRATEGIES = (ORCA_STRATEGY, SARATHI_STRATEGY)


@dataclass
class RequestState:
    request_id: int
    prompt: str
    max_new_tokens: int
    prompt_token_ids: List[int]
    sampling: SamplingParams
    seed: int
    generated_token_ids: List[int] = field(default_factory=list)
    pending_token_id: Optional[int] = None
    reserved_blocks: List[int] = field(default_factory=list)   # per cache group; [] = not admitted
    prefill_cursor: int = 0
    finish_reason: Optional[str] = None

    @property
    def is_prefilling(self) -> bool:
        return self.pending_token_id is None


@dataclass
class _Pending:
    """An iteration that runs on the GPU and whose tokens the host has not read yet."""

    selected: list            # (request, number of tokens)
    entries: list
    producers: list           # requests that receive a token from it, in row order
    output: object
    can_carry: bool           # single-token rows chosen on the device: the next iteration may carry them on


class ContinuousBatchScheduler:
    def __init__(self, engine, sampler, tokenizer=None, max_batch_size: int = 32,
                 eos_token_id=None, scheduling_strategy: str = ORCA_STRATEGY,
                 prefill_chunk_size: int = 16, max_num_batched_tokens: Optional[int] = None,
                 max_prefill_requests: Optional[int] = None, run_ahead: bool = True):
        if max_batch_size <= 0:
            raise ValueError("max_batch_size must be positive")
        if scheduling_strategy not in SUPPORTED_SCHEDULING_STRATEGIES:
            choices = ", ".join(SUPPORTED_SCHEDULING_STRATEGIES)
            raise ValueError(f"Unknown scheduling strategy '{scheduling_strategy}'. "
                             f"Choose one of: {choices}")
        if prefill_chunk_size <= 0:
            raise ValueError("prefill_chunk_size must be positive")
        if max_batch_size > engine.max_requests:
            raise ValueError(f"max_batch_size {max_batch_size} exceeds the engine's "
                             f"{engine.max_requests} request slots")
        budget = engine.max_step_tokens if max_num_batched_tokens is None else max_num_batched_tokens
        if budget <= 0:
            raise ValueError("max_num_batched_tokens must be positive")
        if budget > engine.max_step_tokens:
            raise ValueError(f"max_num_batched_tokens {budget} exceeds the engine's "
                             f"max_step_tokens {engine.max_step_tokens}")
        self.engine = engine
        self.sampler = sampler
        self.tokenizer = tokenizer
        self.max_batch_size = max_batch_size
        self.eos_token_id = (eos_token_id if eos_token_id is not None
                             else getattr(tokenizer, "eos_token_id", None))
        self.scheduling_strategy = scheduling_strategy
        self.prefill_chunk_size = prefill_chunk_size
        self.max_num_batched_tokens = budget
        if max_prefill_requests is None:
            max_prefill_requests = 1 if scheduling_strategy == SARATHI_STRATEGY else max_batch_size
        self.max_prefill_requests = max_prefill_requests

        self.waiting = deque()                       # prompt tokens still to cache
        self.active: Dict[int, RequestState] = {}    # decoding
        self.finished: Dict[int, RequestState] = {}  # done, nothing held
        self.next_request_id = 0
        self.reserved_blocks = [0] * len(engine.cache.groups)
        self.iterations = 0
        self.run_ahead = run_ahead
        self.steps_run_ahead = 0
        self._inflight = None       # a launched iteration whose tokens the host has not read

    # ------------------------------------------------------------- admission
    def add_request(self, prompt, max_new_tokens=200, sampling: Optional[SamplingParams] = None):
        if not isinstance(prompt, str) or not prompt.strip():
            raise ValueError("prompt must be a non-empty string")
        if self.tokenizer is None:
            raise ValueError("this scheduler has no tokenizer; use add_token_request")
        return self.add_token_request(list(self.tokenizer.encode(prompt)),
                                      max_new_tokens=max_new_tokens, prompt=prompt,
                                      sampling=sampling)

    def add_token_request(self, prompt_token_ids, max_new_tokens=200,
                          prompt="<tokenized prompt>", sampling: Optional[SamplingParams] = None):
        """Add an already tokenized request (src/scheduler/orca_scheduler.py:85-116)."""
        if max_new_tokens <= 0:
            raise ValueError("max_new_tokens must be positive")
        if hasattr(prompt_token_ids, "tolist"):
            prompt_token_ids = prompt_token_ids.reshape(-1).tolist()
        prompt_token_ids = list(prompt_token_ids)
        if not prompt_token_ids:
            raise ValueError("The tokenizer produced an empty prompt")
        if any(isinstance(token, bool) or not isinstance(token, int) for token in prompt_token_ids):
            raise ValueError("The tokenizer must produce integer token IDs")
        if min(prompt_token_ids) < 0 or max(prompt_token_ids) >= self.engine.spec.vocab_size:
            raise ValueError("A prompt token is outside the model vocabulary")
        if len(prompt_token_ids) + max_new_tokens > self.engine.spec.max_positions:
            raise ValueError("Prompt plus requested generation exceeds the model context limit")
        sampling = sampling or SamplingParams(max_new_tokens=max_new_tokens)
        request = RequestState(
            request_id=self.next_request_id, prompt=prompt, max_new_tokens=max_new_tokens,
            prompt_token_ids=prompt_token_ids, sampling=sampling,
            seed=sampling.seed if sampling.seed is not None else fresh_seed())
        need = self._required_blocks(request)
        for group, (pages, pool) in enumerate(zip(need, self.engine.cache.pools)):
            if pages > pool.num_pages:
                raise ValueError(
                    f"the request needs {pages} pages of cache group {group}, the pool has "
                    f"{pool.num_pages}: it could never be scheduled")
        self.next_request_id += 1
        self.waiting.append(request)
        return request.request_id

    def _required_blocks(self, request) -> List[int]:
        """Worst-case pages per cache group (src/scheduler/orca_scheduler.py:119-122)."""
        total = len(request.prompt_token_ids) + request.max_new_tokens
        cache = self.engine.cache
        return [cache.pages_for_length(group, total, self.max_num_batched_tokens)
                for group in range(len(cache.groups))]

    def _fits(self, request, newly_reserved, newly_admitted=0) -> bool:
        """Worst-case pages fit beside all reservations, and a request slot is free."""
        admitted = sum(1 for r in self.waiting if r.reserved_blocks) + len(self.active)
        if admitted + newly_admitted >= self.engine.max_requests:
            return False
        need = self._required_blocks(request)
        return all(self.reserved_blocks[g] + newly_reserved[g] + need[g] <= pool.num_pages
                   for g, pool in enumerate(self.engine.cache.pools))

    # ------------------------------------------------------------- selection
    def select_requests(self):
        """[(request, tokens it brings)] for the next iteration."""
        if self.scheduling_strategy == SARATHI_STRATEGY:
            decoding = sorted(self.active.values(), key=lambda r: r.request_id)
            prefilling = list(self.waiting)
        else:
            pool = sorted(list(self.active.values()) + list(self.waiting),
                          key=lambda r: r.request_id)
            decoding, prefilling = None, None
        selected = []
        budget = self.max_num_batched_tokens
        newly = [0] * len(self.reserved_blocks)
        admitted_now = 0
        prefills = 0

        def take_prefill(request) -> bool:
            """False: this request and all behind it must wait (first come, first served)."""
            nonlocal budget, prefills, admitted_now
            if not request.reserved_blocks:
                if not self._fits(request, newly, admitted_now):
                    return False
                for g, pages in enumerate(self._required_blocks(request)):
                    newly[g] += pages
                admitted_now += 1
            remaining = len(request.prompt_token_ids) - request.prefill_cursor
            size = min(remaining, budget)
            if self.scheduling_strategy == SARATHI_STRATEGY:
                size = min(size, self.prefill_chunk_size)
            selected.append((request, size))
            budget -= size
            prefills += 1
            return True

        if self.scheduling_strategy == SARATHI_STRATEGY:
            # room is kept for one prompt portion when a prompt is waiting
            # (src/scheduler/orca_scheduler.py:165)
            head_fits = bool(prefilling) and (bool(prefilling[0].reserved_blocks)
                                              or self._fits(prefilling[0], newly))
            decode_capacity = self.max_batch_size - (1 if head_fits else 0)
            for request in decoding[:max(decode_capacity, 0)]:
                if budget == 0:
                    break
                selected.append((request, 1))
                budget -= 1
            for request in prefilling:
                if (len(selected) >= self.max_batch_size or budget == 0
                        or prefills >= self.max_prefill_requests):
                    break
                if not take_prefill(request):
                    break
        else:
            for request in pool:
                if len(selected) >= self.max_batch_size or budget == 0:
                    break
                if request.is_prefilling:
                    if prefills >= self.max_prefill_requests:
                        continue
                    if not take_prefill(request):
                        break
                else:
                    selected.append((request, 1))
                    budget -= 1
        return selected

    def build_step_entries(self, selected) -> List[StepEntry]:
        entries = []
        for request, size in selected:
            if request.is_prefilling:
                start = request.prefill_cursor
                tokens = request.prompt_token_ids[start:start + size]
                last = start + size == len(request.prompt_token_ids)
                # only the final portion of a prompt produces a token
                # (src/scheduler/orca_scheduler.py:191)
                entries.append(StepEntry(request.request_id, tokens, [size - 1] if last else []))
            else:
                entries.append(StepEntry(request.request_id, [request.pending_token_id], [0]))
        return entries

    # ------------------------------------------------------------------ step
    def step(self) -> Dict[int, int]:
        """One iteration.  With a real engine the whole iteration (step, token selection and
        the copy of the tokens) runs on the engine's own stream, which saves the hand-over
        between streams on every step."""
        stream = getattr(self.engine, "stream", None)
        if stream is None:
            return self._step()
        import torch

        previous = torch.cuda.current_stream(stream.device)
        torch.cuda.set_stream(stream)
        try:
            return self._step()
        finally:
            torch.cuda.set_stream(previous)

    def _step(self) -> Dict[int, int]:
        pending = self._inflight
        self._inflight = None
        if pending is None:
            pending = self._launch()
            if pending is None:
                return {}
        self._inflight = self._launch_ahead(pending)
        return self._resolve(pending)

    def _launch(self) -> Optional["_Pending"]:
        """Select, reserve, and start one iteration on the GPU."""
        selected = self.select_requests()
        if not selected:
            if self.waiting or self.active:
                raise RuntimeError("No request can be scheduled with the available KV memory")
            return None
        new_requests = [request for request, _ in selected if not request.reserved_blocks]
        for request in new_requests:
            request.reserved_blocks = self._required_blocks(request)
            for g, pages in enumerate(request.reserved_blocks):
                self.reserved_blocks[g] += pages
        entries = self.build_step_entries(selected)
        producers = [request for (request, size), entry in zip(selected, entries) if entry.want]
        # greedy rows are picked on the GPU inside the step (one launch less, and part of the
        # captured graph of a decode step)
        greedy = bool(producers) and all(r.sampling.temperature == 0 for r in producers)
        draws = None
        if producers and not greedy and getattr(self.engine, "supports_draws", False):
            draws = self._draws(producers, 0)
        try:
            if draws is not None:
                output = self.engine.step(entries, draws=draws)
            else:
                output = self.engine.step(entries, greedy=greedy)
        except Exception:
            for request in new_requests:
                for g, pages in enumerate(request.reserved_blocks):
                    self.reserved_blocks[g] -= pages
                request.reserved_blocks = []
            raise
        decode_only = all(not request.is_prefilling for request, _ in selected)
        return _Pending(selected, entries, producers, output,
                        (greedy or draws is not None) and decode_only)

    @staticmethod
    def _draws(producers, ahead):
        """(1 / temperature, uniform number) of the next token of each request; ``ahead`` = 1
        when the request's last token is still on its way to the host."""
        from ..sampling.params import uniform_for

        return [(0.0 if r.sampling.temperature == 0 else 1.0 / r.sampling.temperature,
                 uniform_for(r.seed, r.request_id, len(r.generated_token_ids) + ahead))
                for r in producers]

    def _launch_ahead(self, pending) -> Optional["_Pending"]:
        """Start the iteration after ``pending`` before ``pending``'s tokens are known, if
        it is certain which requests it holds: all of ``pending``'s that do not end by
        length, each carrying on the token that ``pending`` chooses for it."""
        if (not self.run_ahead or not pending.can_carry or self.waiting
                or getattr(pending.output, "host_tokens", None) is None
                or len(self.active) != len(pending.selected)):
            return None
        selected, entries = [], []
        for row, (request, _) in enumerate(pending.selected):
            if request.finish_reason is not None:
                continue      # ended at the end token while ``pending`` was already running
            if len(request.generated_token_ids) + 2 > request.max_new_tokens:
                continue      # ``pending`` brings its last token
            selected.append((request, 1))
            entries.append(StepEntry(request.request_id, [0], [0], carry=row))
        if not selected:
            return None
        producers = [request for request, _ in selected]
        try:
            if all(r.sampling.temperature == 0 for r in producers):
                output = self.engine.step(entries, greedy=True)
            else:
                output = self.engine.step(entries, draws=self._draws(producers, 1))
        except ValueError:
            return None       # the ordinary launch of the next iteration reports it
        self.steps_run_ahead += 1
        return _Pending(selected, entries, producers, output, True)

    def _resolve(self, pending) -> Dict[int, int]:
        """Read the tokens of a launched iteration and move its requests on."""
        selected, entries, producers, output = (pending.selected, pending.entries,
                                                pending.producers, pending.output)
        if output.logits.shape[0] != len(producers):
            raise RuntimeError("the engine returned a wrong number of logits rows")
        if getattr(output, "tokens", None) is not None:
            tokens = output.token_list() if hasattr(output, "token_list") else output.tokens.tolist()
        else:
            tokens = self.sampler.sample(
                output.logits, [r.sampling for r in producers], [r.request_id for r in producers],
                [len(r.generated_token_ids) for r in producers], [r.seed for r in producers])
        emitted = {}
        completed_prefill = set()
        next_token = iter(tokens)
        for (request, size), entry in zip(selected, entries):
            if request.finish_reason is not None:
                # ended at the end token after this iteration had been launched ahead: the
                # token computed for it here is dropped
                next(next_token)
                continue
            if request.is_prefilling:
                request.prefill_cursor += size
                if request.prefill_cursor < len(request.prompt_token_ids):
                    continue
                completed_prefill.add(request.request_id)
            token = int(next(next_token))
            request.generated_token_ids.append(token)
            request.pending_token_id = token
            emitted[request.request_id] = token
            reason = None
            if len(request.generated_token_ids) >= request.max_new_tokens:
                reason = "length"
            if (self.eos_token_id is not None and token == self.eos_token_id
                    and not request.sampling.ignore_eos):
                reason = "stop"
            if reason is not None:
                request.finish_reason = reason
                self.active.pop(request.request_id, None)
                self.engine.finish(request.request_id)
                for g, pages in enumerate(request.reserved_blocks):
                    self.reserved_blocks[g] -= pages
                request.reserved_blocks = []
                self.finished[request.request_id] = request
            else:
                self.active[request.request_id] = request
        if completed_prefill:
            self.waiting = deque(r for r in self.waiting if r.request_id not in completed_prefill)
        self.iterations += 1
        return emitted

    def has_work(self) -> bool:
        return bool(self.waiting or self.active or self._inflight is not None)

    def run_until_complete(self):
        while self.has_work():
            self.step()
        if self.tokenizer is None:
            return {rid: list(r.generated_token_ids) for rid, r in self.finished.items()}
        return {rid: self.tokenizer.decode(r.generated_token_ids) for rid, r in self.finished.items()}
