"""Chooses the next token of every request of a step on the device and reads back only
the ids.

Greedy is argmax with the lowest index winning ties; otherwise temperature, top-k and
top-p as the reference filters them (src/llmserve/sampling/sampler.py:16-39), and the token
is the inverse CDF, in vocabulary order, at a uniform number.  The reference draws from a
per-request `torch.Generator` (src/llmserve/sampling/sampler.py:8-13); here the uniform
number is a pure function of (seed, index of the token being generated), so neither
batching nor preemption can change what a seeded request produces.
"""

from __future__ import annotations

import torch

from ..ops import library as ops
from .params import SamplingParams

_MASK64 = (1 << 64) - 1


def _splitmix64(x: int) -> int:
    x = (x + 0x9E3779B97F4A7C15) & _MASK64
    x = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & _MASK64
    x = ((x ^ (x >> 27)) * 0x94D049BB133111EB) & _MASK64
    return x ^ (x >> 31)


def uniform(seed: int, index: int) -> float:
    """A number in [0, 1) with 24 random bits, fixed by (seed, index)."""
    h = _splitmix64(_splitmix64(seed & _MASK64) ^ ((index * 0xD1342543DE82EF95) & _MASK64))
    return (h >> 40) / float(1 << 24)


def request_seed(params: SamplingParams, engine_seed: int, request_id: int) -> int:
    """The request's own seed, or one derived from the engine's seed and the request id."""
    if params.seed is not None:
        return params.seed
    return _splitmix64((engine_seed << 32) ^ (request_id & 0xFFFFFFFF))


class PendingTokens:
    """Token ids that were chosen on the device and are on their way to the host: `device` is the
    int32 tensor the sampling kernel wrote (the next step can read it there), `result()` waits for
    the copy and returns the ids."""

    def __init__(self, device: torch.Tensor | None):
        self.device = device
        self._host = None
        self._event = None
        if device is not None:
            self._host = torch.empty(device.shape, dtype=torch.int32, pin_memory=True)
            self._host.copy_(device, non_blocking=True)
            self._event = torch.cuda.Event()
            self._event.record(torch.cuda.current_stream(device.device))

    def result(self) -> list[int]:
        if self._host is None:
            return []
        self._event.synchronize()
        return self._host.tolist()  # the step's one read-back


class _Staging:
    """A small ring of pinned host buffers for a step's sampling options, each guarded by an event: the options go
    to the device with one copy that the host does not wait for (a copy from pageable memory would make it wait)."""

    def __init__(self, ring: int = 4):
        self._buffers: list[torch.Tensor | None] = [None] * ring
        self._events: list[torch.cuda.Event | None] = [None] * ring
        self._next = 0

    def send(self, values: torch.Tensor, device: torch.device) -> torch.Tensor:
        """values: int32 [n] on the host (pageable).  Returns the same numbers on the device."""
        i = self._next
        self._next = (i + 1) % len(self._buffers)
        n = values.numel()
        if self._events[i] is not None:
            self._events[i].synchronize()  # the copy that last used this buffer is done
        if self._buffers[i] is None or self._buffers[i].numel() < n:
            self._buffers[i] = torch.empty(max(256, 2 * n), dtype=torch.int32, pin_memory=True)
        host = self._buffers[i][:n]
        host.copy_(values)
        out = torch.empty(n, dtype=torch.int32, device=device)
        out.copy_(host, non_blocking=True)
        if self._events[i] is None:
            self._events[i] = torch.cuda.Event()
        self._events[i].record(torch.cuda.current_stream(device))
        return out


class Sampler:
    def __init__(self, device: torch.device):
        self.device = device
        self._staging = _Staging()

    def sample(self, logits: torch.Tensor, items: list[tuple[SamplingParams, int, int]]) -> list[int]:
        """logits float32 [R, V]; items[r] = (params, seed, index of the token being generated)."""
        return self.sample_async(logits, items).result()

    def sample_async(self, logits: torch.Tensor, items: list[tuple[SamplingParams, int, int]]) -> PendingTokens:
        """As `sample`, but returns at once: the ids stay on the device for the next step and come
        to the host when `result()` is asked."""
        r = logits.shape[0]
        if r != len(items):
            raise ValueError(f"{r} rows of logits for {len(items)} requests")
        if r == 0:
            return PendingTokens(None)
        out = torch.empty(r, dtype=torch.int32, device=logits.device)
        if all(p.temperature <= 0 for p, _, _ in items):
            ops.sample_rows(out, logits)
        else:
            # temperature, top-p and the uniform numbers as 32-bit floats, top-k as integers: one buffer, one copy
            floats = torch.tensor([[max(p.temperature, 0.0) for p, _, _ in items], [float(p.top_p) for p, _, _ in items],
                                   [uniform(seed, index) for _, seed, index in items]], dtype=torch.float32)
            top_k = torch.tensor([p.top_k for p, _, _ in items], dtype=torch.int32)
            sent = self._staging.send(torch.cat([floats.view(torch.int32).reshape(-1), top_k]), logits.device)
            options = sent[: 3 * r].view(torch.float32)
            ops.sample_rows(out, logits, temperature=options[:r], top_k=sent[3 * r:], top_p=options[r: 2 * r],
                            uniform=options[2 * r:])
        return PendingTokens(out)
