"""Run-time settings of the engine (not of the model).

Names follow the reference where it has them: ``max_seqs``, ``num_blocks``, ``block_size``,
``max_len`` (src/miniserve/paged_engine.py:24-36, src/miniserve/server.py:435-448).  The token
budget and the portion limit are this engine's own: the reference prefills whole prompts one at
a time (src/miniserve/engine.py:13-14).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional


@dataclass
class EngineConfig:
    dtype: str = "bfloat16"            # "bfloat16" | "float32"
    block_size: int = 16               # tokens per page
    num_blocks: Optional[int] = None   # pages per cache group (the null page not counted); None: from max_seqs * max_len
    max_seqs: int = 32                 # requests that may run at once
    max_len: int = 1024                # prompt + generated tokens of one request
    max_num_batched_tokens: int = 2048  # token budget of one step
    max_prefill_chunk: Optional[int] = None  # largest portion of one prompt in one step (None: the budget)
    hip_graphs: bool = False           # replay decode-only steps from captured graphs
    device: str = "cuda:0"

    def __post_init__(self):
        if self.dtype not in ("bfloat16", "float32"):
            raise ValueError(f"dtype must be 'bfloat16' or 'float32', got {self.dtype!r}")
        if self.block_size <= 0 or self.max_seqs <= 0 or self.max_len <= 0 or self.max_num_batched_tokens <= 0:
            raise ValueError("block_size, max_seqs, max_len and max_num_batched_tokens must be positive")
        if self.max_prefill_chunk is not None and self.max_prefill_chunk <= 0:
            raise ValueError("max_prefill_chunk must be positive")

    @property
    def pages_per_request(self) -> int:
        return -(-self.max_len // self.block_size)

    def resolved_num_blocks(self) -> int:
        if self.num_blocks is not None:
            return self.num_blocks
        return self.max_seqs * self.pages_per_request
