"""Requests that arrive over time, run through the scheduler, with the times that serving is
judged by.

The reference's benchmark lets requests arrive at a fixed pace or as a Poisson process
(comparison_benchmark.py:356-387), submits each request when its time has come, and records
when every token of a request appeared; from those times it derives time to first token, time
per output token and end-to-end time with their mean, median, 95th and 99th percentile
(comparison_benchmark.py:444-472).  This module does the same above
``ContinuousBatchScheduler``: one loop that adds what has arrived and runs an iteration.
The clock is a parameter, so the loop can be tested on the CPU with a clock of its own.
"""

import itertools
import math
import random
import time
from dataclasses import dataclass, field
from typing import Callable, List, Optional, Sequence

from ..sampling.params import SamplingParams


ARRIVAL_PROCESSES = ("poisson", "even", "burst")


def arrival_times(count: int, rate: Optional[float] = None, process: str = "poisson", seed: int = 0):
    """When each of ``count`` requests arrives, in seconds after the start, ascending, the
    first at 0.  ``burst``: all at once (``rate`` is not looked at; an infinite rate means the
    same under every process); ``even``: one every ``1 / rate`` seconds; ``poisson``: the gaps
    are independent draws from the exponential distribution of mean ``1 / rate``, taken from a
    generator of its own that ``seed`` fixes (the arrival model of comparison_benchmark.py:356-387)."""
    if process not in ARRIVAL_PROCESSES:
        raise ValueError(f"unknown arrival process {process!r}; known: {', '.join(ARRIVAL_PROCESSES)}")
    if count <= 0:
        return []
    if process == "burst" or (rate is not None and math.isinf(rate)):
        return [0.0] * count
    if rate is None or not rate > 0:
        raise ValueError("the arrival rate (requests a second) must be positive")
    if process == "even":
        gaps = itertools.repeat(1.0 / rate, count - 1)
    else:
        draw = random.Random(seed).expovariate
        gaps = (draw(rate) for _ in range(count - 1))
    return list(itertools.accumulate(gaps, initial=0.0))


@dataclass
class TraceRequest:
    prompt_token_ids: Sequence[int]
    max_new_tokens: int
    sampling: Optional[SamplingParams] = None


@dataclass
class RequestTimes:
    """What happened to one request, in seconds since the start of the run."""

    scheduled_arrival: float
    submitted_at: Optional[float] = None
    token_times: List[float] = field(default_factory=list)
    request_id: Optional[int] = None

    def metrics(self):
        """Time to first token (from the scheduled arrival), time per output token after the
        first, end-to-end time, and the delay between arrival and submission."""
        if not self.token_times:
            return None
        first, last = self.token_times[0], self.token_times[-1]
        intervals = len(self.token_times) - 1
        return {"ttft": first - self.scheduled_arrival,
                "queue_delay": max(0.0, self.submitted_at - self.scheduled_arrival),
                "tpot": (last - first) / intervals if intervals else 0.0,
                "e2e": last - self.scheduled_arrival}


def percentile(values: Sequence[float], q: float) -> float:
    """Linear interpolation between the order statistics (q in 0..100)."""
    ordered = sorted(values)
    if not ordered:
        return float("nan")
    place = (len(ordered) - 1) * q / 100.0
    low = int(math.floor(place))
    high = min(low + 1, len(ordered) - 1)
    return ordered[low] + (ordered[high] - ordered[low]) * (place - low)


def summarize(values: Sequence[float]) -> dict:
    values = list(values)
    if not values:
        return {"mean": None, "p50": None, "p95": None, "p99": None, "max": None}
    return {"mean": sum(values) / len(values), "p50": percentile(values, 50),
            "p95": percentile(values, 95), "p99": percentile(values, 99), "max": max(values)}


def run_arrival_trace(scheduler, requests: Sequence[TraceRequest], offsets: Sequence[float],
                      clock: Callable[[], float] = time.perf_counter,
                      idle: Callable[[float], None] = time.sleep, synchronize=None) -> dict:
    """Submit ``requests[i]`` once ``offsets[i]`` seconds have passed, run iterations while there
    is work, and return the summary: tokens a second and the spread of the per-request times.
    ``synchronize`` (if given) is called before the clock is read at the start and at the end."""
    if len(requests) != len(offsets):
        raise ValueError("one arrival offset per request is needed")
    order = sorted(range(len(requests)), key=lambda index: offsets[index])
    records = [RequestTimes(scheduled_arrival=offsets[index]) for index in range(len(requests))]
    by_id = {}
    if synchronize:
        synchronize()
    started = clock()
    cursor = 0
    iterations_before = scheduler.iterations
    while cursor < len(order) or scheduler.has_work():
        now = clock() - started
        while cursor < len(order) and offsets[order[cursor]] <= now:
            index = order[cursor]
            request = requests[index]
            sampling = request.sampling or SamplingParams(max_new_tokens=request.max_new_tokens)
            rid = scheduler.add_token_request(request.prompt_token_ids, request.max_new_tokens,
                                              sampling=sampling)
            records[index].submitted_at = now
            records[index].request_id = rid
            by_id[rid] = records[index]
            cursor += 1
        if scheduler.has_work():
            emitted = scheduler.step()
            now = clock() - started
            for rid in emitted:
                by_id[rid].token_times.append(now)
        else:
            # nothing to run before the next arrival
            idle(min(max(offsets[order[cursor]] - now, 0.0), 0.001))
    if synchronize:
        synchronize()
    wall = clock() - started
    measured = [record.metrics() for record in records]
    measured = [item for item in measured if item is not None]
    output_tokens = sum(len(record.token_times) for record in records)
    prompt_tokens = sum(len(request.prompt_token_ids) for request in requests)
    return {
        "requests": len(requests), "completed": len(measured), "wall_seconds": wall,
        "prompt_tokens": prompt_tokens, "output_tokens": output_tokens,
        "output_tokens_per_second": output_tokens / wall if wall > 0 else float("nan"),
        "total_tokens_per_second": (prompt_tokens + output_tokens) / wall if wall > 0 else float("nan"),
        "iterations": scheduler.iterations - iterations_before,
        "ttft_seconds": summarize([item["ttft"] for item in measured]),
        "tpot_seconds": summarize([item["tpot"] for item in measured if item["tpot"] > 0]),
        "e2e_seconds": summarize([item["e2e"] for item in measured]),
        "queue_delay_seconds": summarize([item["queue_delay"] for item in measured]),
        "records": records,
    }
