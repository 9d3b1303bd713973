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


class Sampler:
    def __init__(self, device: torch.device):
        self.device = device

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
            host = torch.tensor(
                [[max(p.temperature, 0.0), float(p.top_p), uniform(seed, index)] for p, seed, index in items],
                dtype=torch.float32).t().contiguous().to(logits.device)
            top_k = torch.tensor([p.top_k for p, _, _ in items], dtype=torch.int32).to(logits.device)
            ops.sample_rows(out, logits, temperature=host[0], top_k=top_k, top_p=host[1], uniform=host[2])
        return PendingTokens(out)
