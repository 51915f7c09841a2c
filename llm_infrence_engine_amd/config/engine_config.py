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
    num_blocks: Optional[int] = None   # pages per cache group (the null page not counted); None: from the memory
                                       # budget if one is given, else max_seqs * pages of max_len
    gpu_memory_fraction: Optional[float] = None  # share of the device's memory the process may hold, weights included
    max_seqs: int = 32                 # requests that may run at once
    max_len: int = 1024                # prompt + generated tokens of one request
    max_num_batched_tokens: int = 2048  # token budget of one step
    max_prefill_chunk: Optional[int] = None  # largest portion of one prompt in one step (None: the budget)
    hip_graphs: Optional[bool] = None  # replay decode-only steps from captured graphs; None: when serving in bfloat16
    decode_steps_per_launch: int = 1   # decode steps queued in one graph launch while everybody decodes greedily
    graph_portion_tokens: Optional[int] = None  # with hip_graphs: steps with prompt portions of up to this many tokens
                                       # are replayed from graphs too (None: as far as the host would be what the
                                       # step waits for; 0: decode steps only)
    device: str = "cuda:0"

    def __post_init__(self):
        if self.dtype not in ("bfloat16", "float32"):
            raise ValueError(f"dtype must be 'bfloat16' or 'float32', got {self.dtype!r}")
        if self.block_size <= 0 or self.max_seqs <= 0 or self.max_len <= 0 or self.max_num_batched_tokens <= 0:
            raise ValueError("block_size, max_seqs, max_len and max_num_batched_tokens must be positive")
        if self.max_prefill_chunk is not None and self.max_prefill_chunk <= 0:
            raise ValueError("max_prefill_chunk must be positive")
        if self.gpu_memory_fraction is not None and not 0.0 < self.gpu_memory_fraction <= 1.0:
            raise ValueError("gpu_memory_fraction must be in (0, 1]")
        if self.decode_steps_per_launch < 1:
            raise ValueError("decode_steps_per_launch must be at least 1")
        if self.hip_graphs is None:
            self.hip_graphs = self.dtype == "bfloat16"

    @property
    def pages_per_request(self) -> int:
        return -(-self.max_len // self.block_size)

    def resolved_num_blocks(self, bytes_per_token: Optional[int] = None, device_total_bytes: Optional[int] = None,
                            device_used_bytes: int = 0, other_bytes: int = 0) -> int:
        """Pages of every group's pool.  Given by hand, or what ``max_seqs`` requests of ``max_len`` tokens can
        fill (the reference's default is the same product, src/miniserve/server.py:145); with
        ``gpu_memory_fraction`` no more than fits into that share of the device's memory beside what is held
        already (``device_used_bytes``: the weights, and whatever the allocator keeps cached) and what the engine
        will take beside the pages (``other_bytes``: per-request state, the static logits and activations of the
        captured graphs), counted in bytes as the reference counts its pool (src/miniserve/paged.py:162-168)."""
        if self.num_blocks is not None:
            return self.num_blocks
        most = self.max_seqs * self.pages_per_request
        if self.gpu_memory_fraction is None or not bytes_per_token or not device_total_bytes:
            return most
        budget = int(self.gpu_memory_fraction * device_total_bytes) - device_used_bytes - other_bytes
        pages = budget // (bytes_per_token * self.block_size) - 1          # one of them is the null page
        if pages < self.pages_per_request:
            raise ValueError(f"{self.gpu_memory_fraction:.2f} of the device's memory leaves {max(budget, 0)} bytes for the "
                             f"cache, less than one request of max_len {self.max_len} needs "
                             f"({self.pages_per_request * bytes_per_token * self.block_size} bytes)")
        return min(most, pages)
