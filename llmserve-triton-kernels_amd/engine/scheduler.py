"""Continuous batching above the step function.

Public face as the reference's `ContinuousBatchingEngine`
(src/llmserve/scheduler/engine.py:83-194): `add_request`, `step() -> list[TokenEvent]`,
`run_until_complete`, `abort`, `reset`, `snapshot`, `validate_request`, `has_unfinished`.

One `step()` is one call of the step function with everything that is scheduled:
  1. aborts asked for since the last step;
  2. pages: every running request must be able to store the tokens it already has
     (`prompt + generated`); while the free pages do not cover that, the most recently
     admitted request is preempted: its pages are freed and it goes to the front of the
     queue, to be recomputed later (src/llmserve/scheduler/engine.py:255-274);
  3. one token for every request that is decoding;
  4. the next portion of every request whose prompt is not yet in the cache, cut to the
     step's token budget (and to `max_prefill_chunk`);
  5. new requests, first come first served and never out of order, while there are slots,
     budget and pages: the whole of `prompt + generated` is reserved at admission and one
     spare page is kept per live request (src/llmserve/scheduler/engine.py:212-234), so a
     prompt that was admitted can always finish and only decoding can run out of pages.
A request samples when its portion reaches the end of `prompt + generated`.  The reference
prefills a prompt whole and runs two forwards per iteration; portions under a token budget
and the single mixed batch are this engine's own.

Reading tokens back one step late.  With a sampler that can leave its ids on the device
(`sample_async`) a step does not wait for them: they are read at the start of the next `step()`.
And when that next step is a plain continuation (the same requests, all decoding, nothing
waiting, aborted or about to reach its length, pages at hand) it is started first, on the ids
still on the device, and the ids of the step before are read while it runs, so the GPU never
waits for the host's bookkeeping.  A request that turns out to have stopped (its end-of-sequence
token) has then one more row in the step already started; that row's token is dropped.  Events
and `token_times` therefore lag a step behind the GPU; which tokens are produced does not change.
"""

from __future__ import annotations

import threading
from collections import deque
from time import perf_counter

from ..sampling.params import SamplingParams
from ..sampling.sampler import request_seed
from .request import EngineStats, Request, Status, TokenEvent
from .runner import StepEntry


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
        self.seed = seed
        self.waiting: deque[Request] = deque()
        self.running: list[Request] = []  # in order of admission
        self.finished: dict[int, Request] = {}
        self.stats = EngineStats()
        self._next_id = 0
        self._aborts: set[int] = set()
        self._lock = threading.Lock()
        # the requests (in row order) and the token ids of a step that has been started but not read yet
        self._pending: tuple[list[Request], object] | None = None
        self._lagged = hasattr(sampler, "sample_async")

    # ------------------------------------------------------------------ public
    def validate_request(self, prompt_len: int, max_new_tokens: int) -> None:
        """The reference's four checks (src/llmserve/scheduler/engine.py:111-125)."""
        if prompt_len < 1:
            raise ValueError("prompt must contain at least one token")
        if max_new_tokens < 1:
            raise ValueError("max_new_tokens must be >= 1")
        total = prompt_len + max_new_tokens
        limit = self.runner.max_model_len
        if total > limit:
            raise ValueError(f"prompt + max_new_tokens = {total} exceeds model limit {limit}")
        if self.manager.blocks_for(total) > self.manager.num_blocks:
            raise ValueError(f"request needs {self.manager.blocks_for(total)} KV blocks but the pool has "
                             f"only {self.manager.num_blocks}")

    def add_request(self, prompt_ids: list[int], params: SamplingParams, *, req_id: int | None = None,
                    arrival_time: float | None = None) -> int:
        self.validate_request(len(prompt_ids), params.max_new_tokens)
        vocab = self.runner.vocab_size
        bad = [t for t in prompt_ids if not 0 <= t < vocab]
        if bad:
            raise ValueError(f"prompt holds token ids outside the vocabulary [0, {vocab}): {bad[:5]}")
        if req_id is None:
            req_id = self._next_id
        self._next_id = max(self._next_id, req_id + 1)
        self.waiting.append(Request(
            req_id=req_id, prompt_ids=list(prompt_ids), params=params,
            arrival_time=perf_counter() if arrival_time is None else arrival_time,
            seed=request_seed(params, self.seed, req_id)))
        return req_id

    def abort(self, req_id: int) -> None:
        """Takes effect at the start of the next step.  Thread-safe."""
        with self._lock:
            self._aborts.add(req_id)

    def reset(self) -> None:
        """Drop every request in flight and give back what they hold."""
        self._pending = None
        for r in self.running:
            self.manager.free_sequence(r.req_id)
        self.running.clear()
        self.waiting.clear()

    def has_unfinished(self) -> bool:
        return bool(self.waiting or self.running)

    def snapshot(self) -> dict:
        return {
            "running": len(self.running), "waiting": len(self.waiting),
            "free_blocks": self.manager.num_free_blocks, "total_blocks": self.manager.num_blocks,
            "kv_utilization": round(self.manager.utilization(), 4),
            "internal_fragmentation": round(self.manager.internal_fragmentation(), 4),
            "preemptions": self.stats.preemptions, "tokens_generated": self.stats.tokens_generated,
            "steps": self.stats.steps, "prefill_tokens": self.stats.prefill_tokens,
            "decode_tokens": self.stats.decode_tokens,
        }

    def run_until_complete(self) -> dict[int, Request]:
        while self.has_unfinished():
            self.step()
        return self.finished

    # -------------------------------------------------------------------- step
    def step(self) -> list[TokenEvent]:
        events: list[TokenEvent] = []
        self.stats.steps += 1
        if self._pending is not None:
            if self._can_continue():
                self._continue(events)
                return events
            self._read_pending(events)
        self._process_aborts(events)
        preempted = self._make_room()
        plan = self._plan(admit=not preempted)
        if not plan:
            return events
        entries = [StepEntry(r.req_id, r.tokens(r.num_computed_tokens, n),
                             [n - 1] if samples else []) for r, n, samples in plan]
        logits = self.runner.step(entries)
        sampling = [r for r, _, samples in plan if samples]
        items = [(r.params, r.seed, len(r.generated)) for r in sampling]
        for r, n, _ in plan:
            if n == 1 and r.num_computed_tokens > 0 and r.generated:
                self.stats.decode_tokens += 1
            else:
                self.stats.prefill_tokens += n
            r.num_computed_tokens += n
        if self._lagged:
            self._pending = (sampling, self.sampler.sample_async(logits, items))  # read at the next step
        else:
            self._append_tokens(sampling, self.sampler.sample(logits, items), events)
        return events

    # ------------------------------------------------- a step whose tokens are read later
    def _read_pending(self, events: list[TokenEvent]) -> None:
        reqs, pending = self._pending
        self._pending = None
        self._append_tokens(reqs, pending.result(), events)

    def _can_continue(self) -> bool:
        """Whether the next step is the pending one's requests again, each with the one token
        that is still on the device."""
        reqs, pending = self._pending
        if (self.waiting or self._aborts or not reqs or len(reqs) != len(self.running)
                or not getattr(self.runner, "takes_device_tokens", False)):
            return False
        need = 0
        for r, q in zip(reqs, self.running):
            # the same requests in the same order, none stopped meanwhile, none at its last token
            if r is not q or r.status is not Status.RUNNING or len(r.generated) + 2 > r.params.max_new_tokens:
                return False
            if r.num_computed_tokens != r.num_tokens:  # (every token it has is in the cache: it is decoding)
                return False
            need += self.manager.extra_blocks_needed(r.req_id, 1)
        return need <= self.manager.num_free_blocks

    def _continue(self, events: list[TokenEvent]) -> None:
        reqs, pending = self._pending
        logits = self.runner.step([StepEntry(r.req_id, [0], [0]) for r in reqs], device_tokens=pending.device)
        following = self.sampler.sample_async(logits, [(r.params, r.seed, len(r.generated) + 1) for r in reqs])
        for r in reqs:
            r.num_computed_tokens += 1
        self.stats.decode_tokens += len(reqs)
        self._read_pending(events)  # the step before; a request that stopped there is skipped from now on
        self._pending = (reqs, following)

    # --------------------------------------------------------------- internals
    def _process_aborts(self, events: list[TokenEvent]) -> None:
        with self._lock:
            aborts, self._aborts = self._aborts, set()
        for rid in sorted(aborts):
            req = next((r for r in self.waiting if r.req_id == rid), None)
            if req is not None:
                self.waiting.remove(req)
            else:
                req = next((r for r in self.running if r.req_id == rid), None)
                if req is None:
                    continue  # already finished
                self.running.remove(req)
                self.manager.free_sequence(rid)
            self._finish(req, "abort", events, emit_token=None)

    def _known_need(self, r: Request) -> int:
        """Pages `r` still has to take for the tokens it already has."""
        return self.manager.extra_blocks_needed(r.req_id, r.num_tokens - self.manager.lengths[r.req_id])

    def _make_room(self) -> bool:
        """Preempt, newest admission first, until the running requests' known tokens fit."""
        preempted = False
        while len(self.running) > 1 and sum(self._known_need(r) for r in self.running) > self.manager.num_free_blocks:
            self._preempt(self.running[-1])
            preempted = True
        return preempted

    def _preempt(self, req: Request) -> None:
        self.running.remove(req)
        self.manager.free_sequence(req.req_id)
        req.status = Status.WAITING
        req.num_computed_tokens = 0
        req.num_preemptions += 1
        self.stats.preemptions += 1
        self.waiting.appendleft(req)  # prompt + generated are recomputed when it is admitted again

    def _portion(self, remaining: int, budget: int) -> int:
        n = min(remaining, budget)
        if self.max_prefill_chunk is not None and remaining > 1:
            n = min(n, self.max_prefill_chunk)
        return n

    def _plan(self, admit: bool) -> list[tuple[Request, int, bool]]:
        """(request, tokens it feeds, whether it samples) for this step."""
        budget = self.max_num_batched_tokens
        plan: list[tuple[Request, int, bool]] = []
        decoding = [r for r in self.running if r.num_tokens - r.num_computed_tokens == 1]
        prefilling = [r for r in self.running if r.num_tokens - r.num_computed_tokens > 1]
        for r in decoding + prefilling:
            if budget <= 0:
                break
            remaining = r.num_tokens - r.num_computed_tokens
            n = self._portion(remaining, budget)
            plan.append((r, n, n == remaining))
            budget -= n
        if not admit:
            return plan
        reserved = sum(self._known_need(r) for r in self.running)
        while self.waiting and len(self.running) < self.max_num_seqs and budget > 0:
            req = self.waiting[0]
            total = req.num_tokens
            need = self.manager.blocks_for(total)
            headroom = len(self.running)  # one spare page per request already live
            if self.manager.num_free_blocks - reserved - need < headroom:
                break
            if self.manager.num_free_slots < 1:
                break
            self.waiting.popleft()
            self.manager.add_sequence(req.req_id)
            req.status = Status.RUNNING
            req.num_computed_tokens = 0
            self.running.append(req)
            reserved += need
            n = self._portion(total, budget)
            plan.append((req, n, n == total))
            budget -= n
        return plan

    def _append_tokens(self, reqs: list[Request], tokens: list[int], events: list[TokenEvent]) -> None:
        now = perf_counter()
        for r, tok in zip(reqs, tokens):
            if r.status is not Status.RUNNING:
                continue  # it stopped a step earlier; this row was computed for nothing
            r.generated.append(tok)
            r.token_times.append(now)
            self.stats.tokens_generated += 1
            reason = None
            if r.params.eos_token_id is not None and tok == r.params.eos_token_id:
                reason = "stop"
            elif len(r.generated) >= r.params.max_new_tokens:
                reason = "length"
            if reason:
                self.running.remove(r)
                self.manager.free_sequence(r.req_id)
                self._finish(r, reason, events, emit_token=tok)
            else:
                events.append(TokenEvent(r.req_id, tok, False))

    def _finish(self, req: Request, reason: str, events: list[TokenEvent], emit_token: int | None) -> None:
        req.status = Status.FINISHED
        req.finish_reason = reason
        req.finish_time = perf_counter()
        self.finished[req.req_id] = req
        events.append(TokenEvent(req.req_id, emit_token, True, reason))
