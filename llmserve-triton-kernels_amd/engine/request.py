"""Records of a request's life, with the reference's names: `Request`, `Status`,
`TokenEvent`, `EngineStats` (src/llmserve/scheduler/engine.py:36-80) and `GenerationResult`
(src/llmserve/datatypes.py:16-27)."""

from __future__ import annotations

from dataclasses import dataclass, field
from enum import Enum

from ..sampling.params import SamplingParams


class Status(Enum):
    WAITING = "waiting"
    RUNNING = "running"
    FINISHED = "finished"


@dataclass
class Request:
    req_id: int
    prompt_ids: list[int]
    params: SamplingParams
    arrival_time: float
    seed: int = 0
    generated: list[int] = field(default_factory=list)
    status: Status = Status.WAITING
    num_computed_tokens: int = 0  # how much of prompt + generated the cache holds
    token_times: list[float] = field(default_factory=list)  # host clock at which each generated token was read
    finish_time: float | None = None
    finish_reason: str | None = None  # one of "stop" (end-of-sequence id), "length", "abort"
    num_preemptions: int = 0  # times its pages were taken away and it started over

    @property
    def num_tokens(self) -> int:
        return len(self.prompt_ids) + len(self.generated)

    def tokens(self, start: int, count: int) -> list[int]:
        """`count` tokens of prompt + generated from position `start`, without building the whole list."""
        n = len(self.prompt_ids)
        if start >= n:
            return self.generated[start - n: start - n + count]
        if start + count <= n:
            return self.prompt_ids[start: start + count]
        return self.prompt_ids[start:] + self.generated[: start + count - n]


@dataclass
class TokenEvent:
    req_id: int
    token: int | None
    finished: bool
    finish_reason: str | None = None
    error: str | None = None


@dataclass
class EngineStats:
    steps: int = 0
    prefill_tokens: int = 0
    decode_tokens: int = 0
    tokens_generated: int = 0
    preemptions: int = 0


@dataclass
class GenerationResult:
    tokens: list[int]
    ttft_s: float  # from the call to the first generated token
    step_latencies_s: list[float] = field(default_factory=list)  # from each token to the next
    total_s: float = 0.0
    peak_memory_bytes: int = 0
    finish_reason: str | None = None

    @property
    def decode_tokens_per_s(self) -> float:
        """Tokens after the first, per second of the time between them (0 when there were none)."""
        gaps = self.step_latencies_s
        spent = sum(gaps)
        if not gaps or spent <= 0:
            return 0.0
        return len(gaps) / spent
