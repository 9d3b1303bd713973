"""Request options, with the reference's names and defaults (src/llmserve/datatypes.py:6-13)."""

from __future__ import annotations

from dataclasses import dataclass


@dataclass
class SamplingParams:
    temperature: float = 0.0  # <= 0 means greedy
    top_k: int = 0  # 0 disables
    top_p: float = 1.0  # 1.0 disables
    max_new_tokens: int = 128
    eos_token_id: int | None = None
    seed: int | None = None
