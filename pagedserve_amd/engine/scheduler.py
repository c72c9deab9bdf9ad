"""Continuous batching above the step function.

What a request goes through is what the reference's ``ContinuousBatchScheduler`` puts it
through (src/scheduler/orca_scheduler.py:32-303): it waits until its whole prompt is cached,
then decodes one token per iteration until ``max_new_tokens`` or the end token, then gives
back what it holds.  Two ways of choosing an iteration's work:

* ``orca``: requests in arrival order, decoding ones with their single token and waiting
  ones with their whole remaining prompt (``:128-146,187-188``);
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

**More decoding requests than an iteration holds.**  The engine may have more request slots
than ``max_batch_size``.  The decoding requests of an iteration are then those that were
served least recently, so that every one advances at the same rate; the reference always
takes the lowest ids (``:165-166``), and the others starve until those finish.

**Running ahead.**  Where the engine chooses the tokens on the device, the iteration after
the current one is chosen and launched before the current one's tokens have reached the
host: everything that decides its work is known without them (how far every prompt has come,
who decodes, who ends by length and gives its pages back, whose turn it is), and a decoding
request's entry says "the token that the last step chose for row r" instead of a token id.
So the host's work for an iteration (choosing, packing, launching) overlaps the GPU's work for
the one before, prompt portions included.  One that ends at the end token has one token too
many computed, which is dropped, and its pages come back an iteration later.  The tokens that
a request receives are the same either way, and without end tokens so is every iteration's
work.
"""

from dataclasses import dataclass, field
from typing import Dict, List, Optional

import numpy as np

from ..sampling.params import SamplingParams, fresh_seed, uniform_for
from .engine import StepEntry

ORCA_STRATEGY = "orca"
SARATHI_STRATEGY = "sarathi"
SUPPORTED_SCHEDULING_STRATEGIES = (ORCA_STRATEGY, SARATHI_STRATEGY)

# ``eos_token_id`` of the constructor when the caller leaves the choice to the tokenizer; ``None``
# means that no token ends a request.
FROM_TOKENIZER = "tokenizer"


@dataclass
class RequestState:
    request_id: int
    prompt: str
    max_new_tokens: int
    prompt_token_ids: List[int]
    sampling: SamplingParams
    seed: int
    generated_token_ids: List[int] = field(default_factory=list)
    pending_token_id: Optional[int] = None      # the token that the next decode step brings
    reserved_blocks: List[int] = field(default_factory=list)   # per cache group; [] = not admitted
    prefill_cursor: int = 0                     # prompt tokens that are cached
    finish_reason: Optional[str] = None
    last_served: int = -1                       # ticket of its last turn; tickets grow with time
    # row of the running iteration's chosen tokens that holds the token the next decode step
    # brings, while that token has not reached the host
    carry_row: Optional[int] = None
    ending: Optional[str] = None                # "length": the token on its way is the last one
    released: bool = False                      # pages, slot and promise have gone back
    prompt_array: Optional[object] = field(default=None, repr=False)   # the prompt as an int64 array

    @property
    def is_prefilling(self) -> bool:
        return self.pending_token_id is None and self.carry_row is None

    @property
    def prompt_left(self) -> int:
        return len(self.prompt_token_ids) - self.prefill_cursor


class _PageLedger:
    """Pages promised to admitted requests, per cache group.  A promise covers the request's
    worst case, so the sum never exceeds a pool and a running request never lacks a page."""

    def __init__(self, cache, longest_step):
        self.cache = cache
        self.longest_step = longest_step
        self.promised = [0] * len(cache.groups)

    def worst_case(self, request) -> List[int]:
        """Most pages per group that the request ever holds
        (src/scheduler/orca_scheduler.py:119-122)."""
        total = len(request.prompt_token_ids) + request.max_new_tokens
        return [self.cache.pages_for_length(group, total, self.longest_step)
                for group in range(len(self.cache.groups))]

    def ever_fits(self, request) -> Optional[str]:
        """None, or why no pool could ever hold the request."""
        for group, (pages, pool) in enumerate(zip(self.worst_case(request), self.cache.pools)):
            if pages > pool.num_pages:
                return (f"the request needs {pages} pages of cache group {group}, the pool has "
                        f"{pool.num_pages}: it could never be scheduled")
        return None

    def has_room(self, request, beside) -> bool:
        """Whether the request's worst case fits beside all promises and ``beside`` (pages that
        the iteration being planned is about to promise)."""
        return all(promised + extra + need <= pool.num_pages
                   for promised, extra, need, pool in zip(self.promised, beside,
                                                          self.worst_case(request), self.cache.pools))

    def promise(self, request):
        request.reserved_blocks = self.worst_case(request)
        for group, pages in enumerate(request.reserved_blocks):
            self.promised[group] += pages

    def withdraw(self, request):
        for group, pages in enumerate(request.reserved_blocks):
            self.promised[group] -= pages
        request.reserved_blocks = []


class _Plan:
    """The work of one iteration while it is being chosen: (request, tokens) pairs under the
    limits on requests, tokens and prompts, and the pages that newcomers among them need."""

    def __init__(self, scheduler):
        self.scheduler = scheduler
        self.chosen = []                          # (request, tokens it brings)
        self.tokens_left = scheduler.max_num_batched_tokens
        self.prompts = 0
        self.newcomers = 0
        self.newcomer_pages = [0] * len(scheduler.ledger.promised)

    @property
    def full(self) -> bool:
        return len(self.chosen) >= self.scheduler.max_batch_size or self.tokens_left == 0

    def add_decode(self, request):
        self.chosen.append((request, 1))
        self.tokens_left -= 1

    def admits(self, request) -> bool:
        """Whether a request that holds no promise yet could get one in this iteration."""
        scheduler = self.scheduler
        if scheduler.admitted_requests() + self.newcomers >= scheduler.engine.max_requests:
            return False
        return scheduler.ledger.has_room(request, self.newcomer_pages)

    def add_prompt(self, request, longest) -> bool:
        """A portion of the request's prompt; False when the request has to wait for pages
        or a slot (and with it everything behind it: first come, first served)."""
        if not request.reserved_blocks:
            if not self.admits(request):
                return False
            for group, pages in enumerate(self.scheduler.ledger.worst_case(request)):
                self.newcomer_pages[group] += pages
            self.newcomers += 1
        size = min(request.prompt_left, self.tokens_left, longest)
        self.chosen.append((request, size))
        self.tokens_left -= size
        self.prompts += 1
        return True


@dataclass
class _Flight:
    """An iteration that runs on the GPU and whose tokens the host has not read yet."""

    chosen: list              # (request, number of tokens)
    receivers: list           # requests that get a token from it, in the order of the logits rows
    output: object
    can_carry: bool           # its tokens are chosen on the device (or it chooses none)
    advanced: bool = False    # its requests have been moved on (all but the tokens' values)
    deliveries: list = field(default_factory=list)   # (request, row of its token)


class ContinuousBatchScheduler:
    def __init__(self, engine, sampler, tokenizer=None, max_batch_size: int = 32,
                 eos_token_id=FROM_TOKENIZER, scheduling_strategy: str = ORCA_STRATEGY,
                 prefill_chunk_size: int = 16, max_num_batched_tokens: Optional[int] = None,
                 max_prefill_requests: Optional[int] = None, run_ahead: bool = True):
        if scheduling_strategy not in SUPPORTED_SCHEDULING_STRATEGIES:
            raise ValueError(f"Unknown scheduling strategy '{scheduling_strategy}'. Choose one of: "
                             + ", ".join(SUPPORTED_SCHEDULING_STRATEGIES))
        for name, value in (("max_batch_size", max_batch_size), ("prefill_chunk_size", prefill_chunk_size)):
            if value <= 0:
                raise ValueError(f"{name} must be positive")
        if max_batch_size > engine.max_requests:
            raise ValueError(f"max_batch_size {max_batch_size} exceeds the engine's "
                             f"{engine.max_requests} request slots")
        budget = engine.max_step_tokens if max_num_batched_tokens is None else max_num_batched_tokens
        if not 0 < budget <= engine.max_step_tokens:
            raise ValueError(f"max_num_batched_tokens must lie in 1..{engine.max_step_tokens} "
                             f"(the engine's max_step_tokens), got {budget}")
        self.engine = engine
        self.sampler = sampler
        self.tokenizer = tokenizer
        self.max_batch_size = max_batch_size
        # "tokenizer": the tokenizer's end token, if it has one; None: nothing ends a request
        if eos_token_id == FROM_TOKENIZER:
            eos_token_id = getattr(tokenizer, "eos_token_id", None)
        self.eos_token_id = eos_token_id
        self.scheduling_strategy = scheduling_strategy
        self.prefill_chunk_size = prefill_chunk_size
        self.max_num_batched_tokens = budget
        if max_prefill_requests is None:
            max_prefill_requests = 1 if scheduling_strategy == SARATHI_STRATEGY else max_batch_size
        self.max_prefill_requests = max_prefill_requests
        self.run_ahead = run_ahead

        # Every request that is not finished, in arrival order (ids grow with arrival).
        self._live: Dict[int, RequestState] = {}
        self.finished: Dict[int, RequestState] = {}
        self.ledger = _PageLedger(engine.cache, budget)
        self.next_request_id = 0
        self.iterations = 0
        self._tickets = 0
        self.steps_run_ahead = 0
        self._inflight: Optional[_Flight] = None
        self._failed_ahead: Optional[Exception] = None   # raised by the next call of step()

    # ----------------------------------------------------------------- views
    @property
    def waiting(self) -> List[RequestState]:
        """Requests whose prompt is not wholly cached yet, in arrival order."""
        return [request for request in self._live.values() if request.is_prefilling]

    @property
    def active(self) -> Dict[int, RequestState]:
        """Decoding requests by id."""
        return {rid: request for rid, request in self._live.items() if not request.is_prefilling}

    @property
    def reserved_blocks(self) -> List[int]:
        return list(self.ledger.promised)

    def admitted_requests(self) -> int:
        return sum(1 for request in self._live.values() if request.reserved_blocks)

    def _required_blocks(self, request) -> List[int]:
        return self.ledger.worst_case(request)

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
        """Queue an already tokenized request; the checks of
        src/scheduler/orca_scheduler.py:85-116, and one more: a request that no pool could
        ever hold is refused here instead of waiting for ever."""
        if hasattr(prompt_token_ids, "tolist"):
            prompt_token_ids = prompt_token_ids.reshape(-1).tolist()
        tokens = list(prompt_token_ids)
        spec = self.engine.spec
        problem = None
        if max_new_tokens <= 0:
            problem = "max_new_tokens must be positive"
        elif not tokens:
            problem = "The tokenizer produced an empty prompt"
        elif not all(type(token) is int for token in tokens):
            problem = "The tokenizer must produce integer token IDs"
        elif not all(0 <= token < spec.vocab_size for token in tokens):
            problem = "A prompt token is outside the model vocabulary"
        elif len(tokens) + max_new_tokens > spec.max_positions:
            problem = "Prompt plus requested generation exceeds the model context limit"
        if problem:
            raise ValueError(problem)
        if sampling is None:
            sampling = SamplingParams(max_new_tokens=max_new_tokens)
        request = RequestState(
            request_id=self.next_request_id, prompt=prompt, max_new_tokens=max_new_tokens,
            prompt_token_ids=tokens, sampling=sampling,
            seed=fresh_seed() if sampling.seed is None else sampling.seed)
        problem = self.ledger.ever_fits(request)
        if problem:
            raise ValueError(problem)
        self.next_request_id += 1
        self._live[request.request_id] = request
        return request.request_id

    # ------------------------------------------------------------- selection
    def _decoding_in_turn(self, room: int) -> List[RequestState]:
        """At most ``room`` decoding requests, in arrival order.  When there are more, those
        that were served least recently are taken, so that all of them advance."""
        decoding = [request for request in self._live.values() if not request.is_prefilling]
        if len(decoding) > room:
            decoding.sort(key=lambda request: (request.last_served, request.request_id))
            decoding = sorted(decoding[:max(room, 0)], key=lambda request: request.request_id)
        return decoding

    def select_requests(self):
        """[(request, tokens it brings)] for the next iteration."""
        plan = _Plan(self)
        if self.scheduling_strategy == SARATHI_STRATEGY:
            prompts = self.waiting
            # room is kept for one prompt portion when a prompt can run
            # (src/scheduler/orca_scheduler.py:165)
            head_can_run = bool(prompts) and (bool(prompts[0].reserved_blocks) or plan.admits(prompts[0]))
            for request in self._decoding_in_turn(self.max_batch_size - int(head_can_run)):
                if plan.full:
                    break
                plan.add_decode(request)
            for request in prompts:
                if plan.full or plan.prompts >= self.max_prefill_requests:
                    break
                if not plan.add_prompt(request, self.prefill_chunk_size):
                    break
        else:
            in_turn = {request.request_id for request in self._decoding_in_turn(self.max_batch_size)}
            for request in self._live.values():
                if plan.full:
                    break
                if not request.is_prefilling:
                    if request.request_id in in_turn:
                        plan.add_decode(request)
                elif plan.prompts < self.max_prefill_requests:
                    if not plan.add_prompt(request, self.max_num_batched_tokens):
                        break
        return plan.chosen

    def build_step_entries(self, selected) -> List[StepEntry]:
        entries = []
        for request, size in selected:
            if request.is_prefilling:
                start = request.prefill_cursor
                # only the portion that ends the prompt produces a token
                # (src/scheduler/orca_scheduler.py:191)
                want = [size - 1] if size == request.prompt_left else []
                if size > 16:
                    # long portions travel as slices of one array, made once: the step function
                    # checks and packs arrays without a loop over their tokens
                    if request.prompt_array is None:
                        request.prompt_array = np.asarray(request.prompt_token_ids, dtype=np.int64)
                    tokens = request.prompt_array[start:start + size]
                else:
                    tokens = request.prompt_token_ids[start:start + size]
                entries.append(StepEntry(request.request_id, tokens, want))
            elif request.carry_row is not None:
                # the token is still on the device: row ``carry_row`` of the last step's choices
                entries.append(StepEntry(request.request_id, [0], [0], carry=request.carry_row))
            else:
                entries.append(StepEntry(request.request_id, [request.pending_token_id], [0]))
        return entries

    # ------------------------------------------------------------------ step
    def step(self) -> Dict[int, int]:
        """One iteration: {request id: the token it received}.  With a real engine the whole
        iteration (step, token selection and the copy of the tokens) runs on the engine's own
        stream, which saves the hand-over between streams on every step."""
        stream = getattr(self.engine, "stream", None)
        if stream is None:
            return self._iterate()
        import torch

        previous = torch.cuda.current_stream(stream.device)
        torch.cuda.set_stream(stream)
        try:
            return self._iterate()
        finally:
            torch.cuda.set_stream(previous)

    def _iterate(self) -> Dict[int, int]:
        if self._failed_ahead is not None:
            error, self._failed_ahead = self._failed_ahead, None
            raise error
        flight, self._inflight = self._inflight, None
        if flight is None:
            flight = self._take_off()
            if flight is None:
                return {}
        try:
            self._inflight = self._take_off_ahead(flight)
        except Exception as error:
            # The step ahead failed in a way that the ordinary start would not report.  The
            # iteration that is already running is not lost with it: it lands now and its
            # tokens go to the caller; the error is raised by the next call, before anything
            # else is started.
            self._inflight = None
            self._failed_ahead = error
        return self._land(flight)

    def _choose_on_device(self, receivers):
        """How the engine should pick the tokens of ``receivers``: keyword arguments of
        ``engine.step``.  Greedy rows are picked inside the step (one launch less, and part of
        a decode step's graph); with temperatures each row gets ``(1 / temperature, uniform
        number)``, if the engine draws; else the logits go to the sampler."""
        if not receivers:
            return {}
        if all(request.sampling.temperature == 0 for request in receivers):
            return {"greedy": True}
        if not getattr(self.engine, "supports_draws", False):
            return {}
        # a request whose last token is still on its way to the host draws its next but one
        return {"draws": [(0.0 if r.sampling.temperature == 0 else 1.0 / r.sampling.temperature,
                           uniform_for(r.seed, r.request_id,
                                       len(r.generated_token_ids) + (r.carry_row is not None)))
                          for r in receivers]}

    def _take_off(self, ahead: bool = False) -> Optional[_Flight]:
        """Choose an iteration's work, promise pages to its newcomers, start it on the GPU.
        ``ahead``: the iteration before it still runs, and nothing to choose is no error."""
        chosen = self.select_requests()
        if not chosen:
            if self._live and not ahead:
                raise RuntimeError("No request can be scheduled with the available KV memory")
            return None
        newcomers = [request for request, _ in chosen if not request.reserved_blocks]
        for request in newcomers:
            self.ledger.promise(request)
        entries = self.build_step_entries(chosen)
        receivers = [request for (request, _), entry in zip(chosen, entries) if entry.want]
        how = self._choose_on_device(receivers)
        try:
            output = self.engine.step(entries, **how)
        except Exception:
            # nothing ran: the newcomers' promises are withdrawn
            # (src/scheduler/orca_scheduler.py:243-247)
            for request in newcomers:
                self.ledger.withdraw(request)
            raise
        if receivers:
            on_device = bool(how) and getattr(output, "host_tokens", None) is not None
        else:
            # no token to wait for; only an engine that chooses tokens lets the next iteration
            # carry them on
            on_device = bool(getattr(self.engine, "supports_draws", False))
        return _Flight(chosen, receivers, output, on_device)

    def _take_off_ahead(self, flight) -> Optional[_Flight]:
        """Start the iteration after ``flight`` before ``flight``'s tokens are known: its
        requests are moved on first (all but the tokens' values), then the next iteration is
        chosen as ever; a request whose token is on its way carries it on from the device."""
        if not self.run_ahead or not flight.can_carry:
            return None
        self._advance(flight)
        try:
            ahead = self._take_off(ahead=True)
        except ValueError:
            return None         # the ordinary start of the next iteration reports it
        if ahead is not None:
            self.steps_run_ahead += 1
        return ahead

    def _advance(self, flight):
        """What a started iteration changes whatever tokens it chooses: prompts have come
        further, the receivers have a token on its way (``flight.deliveries``), those for whom
        it is the last by length give back what they hold, and everybody has had a turn."""
        flight.advanced = True
        rows = {id(request): row for row, request in enumerate(flight.receivers)}
        served = []
        for request, size in flight.chosen:
            if request.finish_reason is not None:
                continue        # ended at the end token after this iteration had been started ahead
            served.append(request)
            if request.is_prefilling:
                request.prefill_cursor += size
                if request.prompt_left:
                    continue
            row = rows[id(request)]
            request.carry_row = row
            flight.deliveries.append((request, row))
            if len(request.generated_token_ids) + 1 >= request.max_new_tokens:
                request.ending = "length"
                self._release(request)
        # those that had waited longest for this turn are also first in line for the next one
        for request in sorted(served, key=lambda request: (request.last_served, request.request_id)):
            request.last_served = self._tickets
            self._tickets += 1

    def _tokens_of(self, flight) -> List[int]:
        output = flight.output
        if output.logits.shape[0] != len(flight.receivers):
            raise RuntimeError("the engine returned a wrong number of logits rows")
        if not flight.receivers:
            return []
        if getattr(output, "tokens", None) is None:
            receivers = flight.receivers
            return self.sampler.sample(
                output.logits, [r.sampling for r in receivers], [r.request_id for r in receivers],
                [len(r.generated_token_ids) for r in receivers], [r.seed for r in receivers])
        return output.token_list() if hasattr(output, "token_list") else output.tokens.tolist()

    def _land(self, flight) -> Dict[int, int]:
        """Read the tokens of a started iteration and hand them to its requests."""
        if not flight.advanced:
            self._advance(flight)
        tokens = self._tokens_of(flight)
        emitted = {}
        for request, row in flight.deliveries:
            if request.finish_reason is not None:
                continue        # (cannot happen: a delivery is made once, and before any later one)
            token = int(tokens[row])
            request.generated_token_ids.append(token)
            request.pending_token_id = token
            request.carry_row = None
            emitted[request.request_id] = token
            if (token == self.eos_token_id and self.eos_token_id is not None
                    and not request.sampling.ignore_eos):
                self._retire(request, "stop")
            elif request.ending is not None:
                self._retire(request, request.ending)
        self.iterations += 1
        return emitted

    def _release(self, request):
        """Pages, slot and promise go back; the request takes part in nothing from here on."""
        if request.released:
            return
        request.released = True
        del self._live[request.request_id]
        self.engine.finish(request.request_id)
        self.ledger.withdraw(request)

    def _retire(self, request, reason):
        """The request is over and its last token is with it."""
        request.finish_reason = reason
        self._release(request)
        self.finished[request.request_id] = request

    def has_work(self) -> bool:
        return bool(self._live) or self._inflight is not None or self._failed_ahead is not None

    def run_until_complete(self):
        while self.has_work():
            self.step()
        if self.tokenizer is None:
            return {rid: list(r.generated_token_ids) for rid, r in self.finished.items()}
        return {rid: self.tokenizer.decode(r.generated_token_ids) for rid, r in self.finished.items()}
