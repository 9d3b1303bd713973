"""Options of the engine, as opposed to the model.

The reference scatters them over constructor arguments: ``num_blocks`` and ``block_size``
(src/llmserve/kvcache/paged.py:114-121), ``max_batch_size`` and ``max_prefill_tokens``
(src/llmserve/scheduler/engine.py:84-92) and the server's ``--kv-mem-mib``
(src/llmserve/server/__main__.py:28,52-55).  Here they are one dataclass.
"""

from __future__ import annotations

from dataclasses import dataclass

DTYPE_NAMES = ("bfloat16", "float32")


@dataclass
class EngineConfig:
    dtype: str = "bfloat16"
    block_size: int = 16  # tokens in a page of the key/value cache
    num_blocks: int | None = None  # pages per cache group; or give a byte budget instead
    kv_bytes: int | None = None
    gpu_memory_fraction: float = 0.85  # of free memory, when neither of the two is given
    max_num_seqs: int = 64  # live requests (state slots)
    max_num_batched_tokens: int = 2048  # token budget of one step
    max_prefill_chunk: int | None = None  # longest portion of one prompt in one step
    max_model_len: int | None = None  # defaults to the model's max_position_embeddings
    seed: int = 0
    # replay steps from captured HIP graphs: decode-only steps, and steps with portions of prompts that are small
    # enough for the host's launches to be their limit (a rule by sizes; a bucket of sizes is captured at its second use)
    use_graphs: bool = True

    def validate(self) -> None:
        if self.dtype not in DTYPE_NAMES:
            raise ValueError(f"dtype={self.dtype!r}; choose from {DTYPE_NAMES}")
        if self.block_size < 1:
            raise ValueError("block_size must be >= 1")
        if self.num_blocks is not None and self.num_blocks < 1:
            raise ValueError("num_blocks must be >= 1")
        if self.max_num_seqs < 1 or self.max_num_batched_tokens < 1:
            raise ValueError("max_num_seqs and max_num_batched_tokens must be >= 1")
        if self.max_prefill_chunk is not None and self.max_prefill_chunk < 1:
            raise ValueError("max_prefill_chunk must be >= 1")
