"""Continuous batching above the step function.

The class answers to the reference's names (`ContinuousBatchingEngine` with `add_request`,
`step() -> list[TokenEvent]`, `run_until_complete`, `abort`, `reset`, `snapshot`,
`validate_request`, `has_unfinished`: src/llmserve/scheduler/engine.py:83-178), so a caller of
the reference finds what it knows.  What happens inside a step is this engine's own:

  one `step()` = one call of the step function, carrying everything that is scheduled:
    a. requests whose cancellation was asked for leave;
    b. the pool must hold the tokens every live request already has (`prompt + generated`);
       while it does not, the request admitted last gives its pages back and returns to the
       head of the queue, to be computed again from its first token (the reference's rule
       for a pool that runs dry: src/llmserve/scheduler/engine.py:255-274);
    c. every request that is decoding brings its one token;
    d. every request whose prompt is not yet in the cache brings its next portion, cut to what
       is left of the step's token budget (and to `max_prefill_chunk`);
    e. queued requests are admitted in arrival order, never one past another, while there is a
       slot, budget and room: the pages of the whole `prompt + generated` are set aside at
       admission and one more page per live request stays free
       (src/llmserve/scheduler/engine.py:212-234), so an admitted prompt can always be
       finished and only decoding can run short of pages.
  A request samples when its portion reaches the end of `prompt + generated`.  (The reference
  runs a whole-prompt forward and a decode forward per iteration; portions under a token budget
  in one mixed batch replace both here.)

Reading the sampled ids late.  A sampler that offers `sample_async` leaves its ids on the
device; they are fetched when the next `step()` begins.  If that next step merely continues
the last one (the same requests, all decoding, nobody queued or cancelled or at its last
token, pages at hand) and the runner can take its tokens from the device, it is launched
first and the ids of the step before are fetched while it runs: the GPU never waits for the
host.  A request that turns out to have produced its end-of-sequence token then already has a
row in the launched step; that row's result is thrown away.  Events and `token_times` thus
trail the GPU by one step; the tokens themselves are the same.
"""

from __future__ import annotations

import threading
from collections import deque
from dataclasses import dataclass
from time import perf_counter

from ..sampling.params import SamplingParams
from ..sampling.sampler import request_seed
from .request import EngineStats, Request, Status, TokenEvent
from .runner import StepEntry


def _add(total: dict[int, int], pages: dict[int, int]) -> None:
    """total += pages, group by group."""
    for gid, n in pages.items():
        total[gid] = total.get(gid, 0) + n


def _fits(need: dict[int, int], free: dict[int, int], spare: int = 0) -> bool:
    """Whether every group has `need` pages free and `spare` more (a group that is not named needs none)."""
    return all(free[gid] - n >= spare for gid, n in need.items())


@dataclass
class _Share:
    """One request's part of a planned step."""

    request: Request
    count: int  # tokens it feeds
    samples: bool  # whether the last of them ends `prompt + generated`


class ContinuousBatchingEngine:
    def __init__(self, runner, sampler, *, max_num_seqs: int = 8, max_num_batched_tokens: int = 2048,
                 max_prefill_chunk: int | None = None, seed: int = 0):
        self.runner = runner
        self.sampler = sampler
        self.manager = runner.manager
        if max_num_seqs > self.manager.max_seqs:
            raise ValueError(f"max_num_seqs={max_num_seqs} exceeds the cache manager's {self.manager.max_seqs} slots")
        if max_num_batched_tokens < max_num_seqs:
            raise ValueError("max_num_batched_tokens must be at least max_num_seqs (one token per decoding request)")
        self.max_num_seqs = max_num_seqs
        self.max_num_batched_tokens = max_num_batched_tokens
        self.max_prefill_chunk = max_prefill_chunk
        # the most tokens of one request in a step: what a windowed cache group holds beside its window
        self._portion = min(max_num_batched_tokens, max_prefill_chunk or max_num_batched_tokens)
        self.seed = seed
        self.waiting: deque[Request] = deque()  # arrival order; a preempted request re-enters at the left
        self.running: list[Request] = []  # admission order, oldest first
        self.finished: dict[int, Request] = {}
        self.stats = EngineStats()
        self._ids_issued = 0
        self._cancel: set[int] = set()
        self._cancel_lock = threading.Lock()
        # (requests in row order, ids still on the device) of a launched step that has not been fetched
        self._in_flight: tuple[list[Request], object] | None = None
        self._reads_late = hasattr(sampler, "sample_async")
        # a runner whose logits may live in a replayed graph's memory lends them: they are sampled at once
        self._step_options = {"borrow": True} if getattr(runner, "lends_logits", False) else {}

    # ================================================================== intake
    def validate_request(self, prompt_len: int, max_new_tokens: int) -> None:
        """Refuse, with `ValueError`, a request that could never be served: an empty prompt, nothing
        to generate, more positions than the model has, more pages than the pool has (the four checks
        of src/llmserve/scheduler/engine.py:111-125)."""
        positions = prompt_len + max_new_tokens
        # what the request holds at most, group by group, against each group's whole pool (a model that keeps
        # only fixed-size state has no pages to run out of)
        need, pools = self.manager.pages_for(positions, self._portion), self.manager.capacity()
        short = [(gid, n) for gid, n in need.items() if n > pools[gid]]
        problems = (
            (prompt_len < 1, "an empty prompt cannot be continued: give at least one token"),
            (max_new_tokens < 1, f"max_new_tokens is {max_new_tokens}; nothing would be generated"),
            (positions > self.runner.max_model_len,
             f"{prompt_len} prompt tokens and {max_new_tokens} new ones need {positions} positions; "
             f"the model stops at {self.runner.max_model_len}"),
            (bool(short), f"{positions} tokens fill {short[0][1] if short else 0} cache pages "
                          f"and the whole pool is {pools[short[0][0]] if short else 0}"),
        )
        for failed, message in problems:
            if failed:
                raise ValueError(message)

    def add_request(self, prompt_ids: list[int], params: SamplingParams, *, req_id: int | None = None,
                    arrival_time: float | None = None) -> int:
        """Queue a request; returns its id (the caller's, or the next unused number)."""
        self.validate_request(len(prompt_ids), params.max_new_tokens)
        vocab = self.runner.vocab_size
        strangers = [t for t in prompt_ids if not 0 <= t < vocab]
        if strangers:
            raise ValueError(f"token ids {strangers[:5]} of the prompt are not in the vocabulary of {vocab} entries")
        rid = self._ids_issued if req_id is None else req_id
        if any(r.req_id == rid for r in self.waiting) or any(r.req_id == rid for r in self.running):
            raise ValueError(f"request id {rid} is already queued or running")
        self._ids_issued = max(self._ids_issued, rid + 1)
        when = perf_counter() if arrival_time is None else arrival_time
        self.waiting.append(Request(req_id=rid, prompt_ids=list(prompt_ids), params=params, arrival_time=when,
                                    seed=request_seed(params, self.seed, rid)))
        return rid

    def abort(self, req_id: int) -> None:
        """Ask for a request to be dropped; it leaves when the next step begins.  May be called from
        another thread."""
        with self._cancel_lock:
            self._cancel.add(req_id)

    def reset(self) -> None:
        """Forget everything in flight: queued requests vanish, live ones give back what they hold,
        a launched step's ids are never fetched."""
        self._in_flight = None
        while self.running:
            self.manager.free_sequence(self.running.pop().req_id)
        self.waiting.clear()
        with self._cancel_lock:
            self._cancel.clear()  # (a stale cancellation must not hit a later request that reuses the id)

    # ================================================================== observation
    def has_unfinished(self) -> bool:
        return len(self.waiting) + len(self.running) > 0

    def snapshot(self) -> dict:
        """Counters for a dashboard (the keys of src/llmserve/scheduler/engine.py:164-173, and this
        engine's own beside them)."""
        m, s = self.manager, self.stats
        report = dict(running=len(self.running), waiting=len(self.waiting), free_blocks=m.num_free_blocks,
                      total_blocks=m.num_blocks, kv_utilization=round(m.utilization(), 4),
                      internal_fragmentation=round(m.internal_fragmentation(), 4))
        for name in ("preemptions", "tokens_generated", "steps", "prefill_tokens", "decode_tokens"):
            report[name] = getattr(s, name)
        return report

    def run_until_complete(self) -> dict[int, Request]:
        while self.has_unfinished():
            self.step()
        return self.finished

    # ================================================================== one step
    def step(self) -> list[TokenEvent]:
        events: list[TokenEvent] = []
        self.stats.steps += 1
        if self._in_flight is not None:
            if self._is_plain_continuation():
                self._launch_continuation(events)
                return events
            self._fetch_in_flight(events)
        self._drop_cancelled(events)
        evicted = self._evict_until_known_tokens_fit()
        shares = self._plan(admit=not evicted)
        if shares:
            self._launch(shares, events)
        return events

    def _launch(self, shares: list[_Share], events: list[TokenEvent]) -> None:
        entries = []
        for s in shares:
            r = s.request
            entries.append(StepEntry(r.req_id, r.tokens(r.num_computed_tokens, s.count),
                                     [s.count - 1] if s.samples else []))
        logits = self.runner.step(entries, **self._step_options)  # (sampled from before the next step)
        drawing = [s.request for s in shares if s.samples]
        draws = [(r.params, r.seed, len(r.generated)) for r in drawing]
        for s in shares:
            r = s.request
            decoding = s.count == 1 and r.generated and r.num_computed_tokens > 0
            if decoding:
                self.stats.decode_tokens += 1
            else:
                self.stats.prefill_tokens += s.count
            r.num_computed_tokens += s.count
        if self._reads_late:
            self._in_flight = (drawing, self.sampler.sample_async(logits, draws))
        else:
            self._take_tokens(drawing, self.sampler.sample(logits, draws), events)

    # ------------------------------------------------------------------ ids fetched a step late
    def _fetch_in_flight(self, events: list[TokenEvent]) -> None:
        requests, ids = self._in_flight
        self._in_flight = None
        self._take_tokens(requests, ids.result(), events)

    def _is_plain_continuation(self) -> bool:
        """Whether the coming step is exactly the launched one's requests again, each with the one
        token that still sits on the device, and the runner can read it there."""
        requests, _ = self._in_flight
        if not getattr(self.runner, "takes_device_tokens", False):
            return False
        if self.waiting or self._cancel or not requests or len(requests) != len(self.running):
            return False
        pages: dict[int, int] = {}
        for launched, live in zip(requests, self.running):
            if launched is not live or live.status is not Status.RUNNING:
                return False  # another set of requests, or one has stopped meanwhile
            if live.num_computed_tokens != live.num_tokens:
                return False  # its known tokens are not all in the cache: it is not decoding
            if len(live.generated) + 2 > live.params.max_new_tokens:
                return False  # the token on the device is its last: no step follows it
            _add(pages, self.manager.pages_owed(live.req_id, 1, self._portion))
        return _fits(pages, self.manager.free_pages())

    def _launch_continuation(self, events: list[TokenEvent]) -> None:
        requests, ids = self._in_flight
        placeholder = [StepEntry(r.req_id, [0], [0]) for r in requests]  # the values come from `ids.device`
        logits = self.runner.step(placeholder, device_tokens=ids.device, **self._step_options)
        after = self.sampler.sample_async(logits, [(r.params, r.seed, len(r.generated) + 1) for r in requests])
        for r in requests:
            r.num_computed_tokens += 1
        self.stats.decode_tokens += len(requests)
        self._fetch_in_flight(events)  # the step before this one; who stopped there is skipped from now on
        self._in_flight = (requests, after)

    # ------------------------------------------------------------------ leaving
    def _retire(self, request: Request, reason: str, token: int | None, events: list[TokenEvent]) -> None:
        """Record a request's end (its pages are already back)."""
        request.status, request.finish_reason, request.finish_time = Status.FINISHED, reason, perf_counter()
        self.finished[request.req_id] = request
        events.append(TokenEvent(request.req_id, token, True, reason))

    def _drop_cancelled(self, events: list[TokenEvent]) -> None:
        with self._cancel_lock:
            asked, self._cancel = sorted(self._cancel), set()
        if not asked:
            return
        queued = {r.req_id: r for r in self.waiting}
        live = {r.req_id: r for r in self.running}
        for rid in asked:
            if rid in queued:
                self.waiting.remove(queued[rid])
                self._retire(queued[rid], "abort", None, events)
            elif rid in live:
                self.running.remove(live[rid])
                self.manager.free_sequence(rid)
                self._retire(live[rid], "abort", None, events)
            # anything else has ended by itself, or never existed

    def _take_tokens(self, requests: list[Request], tokens: list[int], events: list[TokenEvent]) -> None:
        """Append each sampled id to its request and let those go that are done."""
        stamp = perf_counter()
        for request, token in zip(requests, tokens):
            if request.status is not Status.RUNNING:
                continue  # stopped one step earlier; this row was computed in vain
            request.generated.append(token)
            request.token_times.append(stamp)
            self.stats.tokens_generated += 1
            p = request.params
            if p.eos_token_id is not None and token == p.eos_token_id:
                reason = "stop"
            elif len(request.generated) >= p.max_new_tokens:
                reason = "length"
            else:
                events.append(TokenEvent(request.req_id, token, False))
                continue
            self.running.remove(request)
            self.manager.free_sequence(request.req_id)
            self._retire(request, reason, token, events)

    # ------------------------------------------------------------------ pages
    def _pages_owed(self, request: Request) -> dict[int, int]:
        """Pages the request has yet to take for tokens it already has, per cache group."""
        missing = request.num_tokens - self.manager.lengths[request.req_id]
        return self.manager.pages_owed(request.req_id, missing, self._portion)

    def _all_owed(self) -> dict[int, int]:
        owed: dict[int, int] = {}
        for r in self.running:
            _add(owed, self._pages_owed(r))
        return owed

    def _evict_until_known_tokens_fit(self) -> bool:
        """Send the most recent admissions back to the queue until what remains can store its known
        tokens; the oldest request is never sent back.  True if anyone was."""
        evicted = False
        while len(self.running) > 1:
            if _fits(self._all_owed(), self.manager.free_pages()):
                break
            victim = self.running.pop()
            self.manager.free_sequence(victim.req_id)
            victim.status = Status.WAITING
            victim.num_computed_tokens = 0  # everything it has, generated tokens too, is computed again
            victim.num_preemptions += 1
            self.stats.preemptions += 1
            self.waiting.appendleft(victim)
            evicted = True
        return evicted

    # ------------------------------------------------------------------ planning
    def _cut(self, outstanding: int, budget: int) -> int:
        size = min(outstanding, budget)
        if outstanding > 1 and self.max_prefill_chunk is not None:
            size = min(size, self.max_prefill_chunk)
        return size

    def _plan(self, admit: bool) -> list[_Share]:
        budget = self.max_num_batched_tokens
        shares: list[_Share] = []

        def give(request: Request, outstanding: int) -> None:
            nonlocal budget
            size = self._cut(outstanding, budget)
            shares.append(_Share(request, size, size == outstanding))
            budget -= size

        backlog = {id(r): r.num_tokens - r.num_computed_tokens for r in self.running}
        # decoding requests first (one token each), then prompts that are under way
        for r in sorted(self.running, key=lambda r: backlog[id(r)] > 1):  # (stable: admission order within each)
            if budget <= 0:
                break
            give(r, backlog[id(r)])
        if not admit:
            return shares
        set_aside = self._all_owed()
        while self.waiting and budget > 0 and len(self.running) < self.max_num_seqs:
            candidate = self.waiting[0]
            pages = self.manager.pages_for(candidate.num_tokens, self._portion)  # (what the cache manager says it costs)
            wanted = dict(set_aside)
            _add(wanted, pages)
            spare = len(self.running)  # one page per request already live stays free, in every group
            if not _fits(wanted, self.manager.free_pages(), spare) or self.manager.num_free_slots < 1:
                break  # the head of the queue does not fit, and nobody overtakes it
            self.waiting.popleft()
            self.manager.add_sequence(candidate.req_id)
            candidate.status, candidate.num_computed_tokens = Status.RUNNING, 0
            self.running.append(candidate)
            set_aside = wanted
            give(candidate, candidate.num_tokens)
        return shares
