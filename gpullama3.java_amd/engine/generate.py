"""The generation loop above the step function.

The reference's loop serves one sequence: it feeds the prompt one token per
forward pass, then samples, reports and checks stop tokens until the position
bound (J/inference/InferenceEngine.java:83-131, GPU twin :278-366). Here requests
are served in batches that start together: the prompts of a batch go through one
step, then every live sequence gets one token per step; a sequence that ends
leaves the batch and gives its slot back at once; when a batch has ended the next
requests form the next one. Once a batch has started no request joins it.

The loop only decides; the model is behind ``backend``:
``take_slot()``, ``give_back_slot(slot)``, ``step(entries) -> logits handle`` (last
row of each entry), ``sample(logits, temperatures, top_ps, uniforms) -> ids``,
``max_context``, ``page_size``, ``tokens_capacity()``, ``slots_free()``; optionally
``decode_run_length`` and ``decode_run(entries, n, temperatures, top_ps, uniforms[n]) ->
ids[n]``: n steps in a row, each feeding back what it sampled.
"""
from __future__ import annotations

import time
from dataclasses import dataclass, field
from typing import Callable, Optional, Sequence

from ..cache.pages import CacheFull
from ..sampling import SamplingParams, uniform


@dataclass
class Request:
    prompt: Sequence[int]
    max_new_tokens: int
    sampling: SamplingParams = SamplingParams()
    stop_ids: frozenset = frozenset()
    # a sequence that goes on: the slot that holds its earlier tokens (kept when the request ends)
    # and how many they are; ``prompt`` then holds the tokens that follow them
    slot: Optional[int] = None
    cached: int = 0


@dataclass
class Generated:
    tokens: list = field(default_factory=list)      # generated ids only, a stop token included
    finish_reason: Optional[str] = None             # "stop" | "length"


@dataclass
class RunMetrics:
    """Prompt and generated tokens with their times, kept apart; the reference reports
    one figure over both (J/auxiliary/LastRunMetrics.java:27-31)."""
    prompt_tokens: int = 0
    generated_tokens: int = 0
    prefill_seconds: float = 0.0
    decode_seconds: float = 0.0
    decode_steps: int = 0

    @property
    def total_tokens_per_second(self):
        t = self.prefill_seconds + self.decode_seconds
        return (self.prompt_tokens + self.generated_tokens) / t if t > 0 else 0.0


def _rounded(n, page):
    return -(-n // page) * page


def plan_batch(requests, first, max_batch, capacity, page_size, max_context):
    """How many requests from ``first`` on form the next batch: as many as there are
    slots, and as their longest possible lengths fit into the cache together."""
    held, n = 0, 0
    for r in requests[first:first + max_batch]:
        longest = min(len(r.prompt) + max(r.max_new_tokens - 1, 0), max_context)
        need = _rounded(max(longest, 1), page_size)
        if held + need > capacity:
            break
        held += need
        n += 1
    if n == 0:
        r = requests[first]
        raise ValueError(f"request {first} may hold {len(r.prompt)} + {r.max_new_tokens} tokens; "
                         f"the cache holds {capacity}")
    return n


def generate(backend, requests, on_token: Optional[Callable[[int, int], None]] = None, max_batch=None,
             metrics: Optional[RunMetrics] = None):
    """Serve ``requests`` and return a ``Generated`` per request, in request order."""
    for i, r in enumerate(requests):
        if len(r.prompt) == 0:
            raise ValueError(f"request {i} has an empty prompt")
        if r.cached + len(r.prompt) > backend.max_context:
            raise ValueError(f"request {i}: a prompt of {r.cached + len(r.prompt)} tokens exceeds the context of "
                             f"{backend.max_context}")
        if r.slot is None and r.cached:
            raise ValueError(f"request {i} names earlier tokens but no slot that holds them")
    results = [Generated() for _ in requests]
    metrics = metrics if metrics is not None else RunMetrics()
    if any(r.slot is not None for r in requests):
        # sequences that go on hold their slots already: they form one batch as they are
        if len({r.slot for r in requests}) != len(requests) or any(r.slot is None for r in requests):
            raise ValueError("sequences that go on must each name a slot of their own, and all of a call must go on")
        _run_batch(backend, requests, results, range(len(requests)), on_token, metrics)
        return results
    first = 0
    while first < len(requests):
        slots = backend.slots_free()
        if slots < 1:
            raise CacheFull("no slot is free for the next batch")
        n = plan_batch(requests, first, min(max_batch or slots, slots), backend.tokens_capacity(),
                       backend.page_size, backend.max_context)
        _run_batch(backend, requests, results, range(first, first + n), on_token, metrics)
        first += n
    return results


def _run_batch(backend, requests, results, ids, on_token, metrics):
    live = []                     # (request index, slot), in request order
    try:
        for i in ids:
            if requests[i].max_new_tokens <= 0:
                results[i].finish_reason = "length"
                continue
            live.append((i, requests[i].slot if requests[i].slot is not None else backend.take_slot()))
        if not live:
            return
        held = {i: requests[i].cached + len(requests[i].prompt) for i, _ in live}

        def leave(i, slot):
            if requests[i].slot is None:         # a slot that the caller holds stays the caller's
                backend.give_back_slot(slot)

        def take(i, slot, tok):
            """Record a sampled token; true if the sequence goes on."""
            r, out = requests[i], results[i]
            out.tokens.append(int(tok))
            metrics.generated_tokens += 1
            if on_token is not None:
                on_token(i, int(tok))
            if int(tok) in r.stop_ids:
                out.finish_reason = "stop"       # the stop token is part of the result
            elif len(out.tokens) >= r.max_new_tokens or held[i] >= backend.max_context:
                out.finish_reason = "length"     # no room to feed this token back
            return out.finish_reason is None

        def params(rows, k=0):
            # the draw for the token at a position depends on (seed, request, that position): a sequence
            # that goes on over several calls in a slot it keeps never meets the same number twice, as
            # the reference's one generator runs on across the turns of a dialogue
            # (J/inference/sampler/Sampler.java:63)
            return ([requests[i].sampling.temperature for i in rows], [requests[i].sampling.top_p for i in rows],
                    [uniform(requests[i].sampling.seed, i,
                             requests[i].cached + len(requests[i].prompt) + len(results[i].tokens) + k) for i in rows])

        # the prompts of the batch in one step, and each sequence's first token
        t0 = time.perf_counter()
        logits = backend.step([(slot, list(requests[i].prompt)) for i, slot in live])
        first = backend.sample(logits, *params([i for i, _ in live]))
        metrics.prefill_seconds += time.perf_counter() - t0
        metrics.prompt_tokens += sum(len(requests[i].prompt) for i, _ in live)
        nxt = []
        for (i, slot), tok in zip(live, first):
            if take(i, slot, tok):
                nxt.append((i, slot))
            else:
                leave(i, slot)
        live = nxt

        # then one token per live sequence and step. A backend may run several steps before it
        # reports (it feeds each sampled token back itself): then a sequence that ends inside
        # such a run leaves the batch at the run's end, and what it sampled after its end is
        # dropped. No run is longer than the shortest remaining budget of its sequences.
        most = max(1, int(getattr(backend, "decode_run_length", 1)))
        if any(requests[i].slot is not None for i, _ in live):
            most = 1     # a slot that is kept must hold the sequence's own tokens only, none sampled after its end
        while live:
            rows = [i for i, _ in live]
            n = min([most] + [min(requests[i].max_new_tokens - len(results[i].tokens),
                                  backend.max_context - held[i]) for i in rows])
            t0 = time.perf_counter()
            if n <= 1 or not hasattr(backend, "decode_run"):
                n = 1
                logits = backend.step([(slot, [results[i].tokens[-1]]) for i, slot in live])
                sampled = [backend.sample(logits, *params(rows))]
            else:
                temps, tops, _ = params(rows)
                us = [params(rows, k)[2] for k in range(n)]
                sampled = backend.decode_run([(slot, results[i].tokens[-1]) for i, slot in live], n, temps, tops, us)
            metrics.decode_seconds += time.perf_counter() - t0
            metrics.decode_steps += n
            going = {i: True for i in rows}
            for k in range(n):
                for (i, slot), tok in zip(live, sampled[k]):
                    held[i] += 1                      # step k fed this sequence's previous token
                    if going[i]:
                        going[i] = take(i, slot, tok)
            nxt = []
            for i, slot in live:
                if going[i]:
                    nxt.append((i, slot))
                else:
                    leave(i, slot)
            live = nxt
    except BaseException:
        for i, slot in live:
            try:
                leave(i, slot)
            except Exception:
                pass
        raise
