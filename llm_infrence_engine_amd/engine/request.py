"""A request and what is recorded about it, with the reference's names
(``Request`` and ``StepRecord``, src/miniserve/engine.py:32-91)."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional, Tuple


@dataclass
class Request:
    prompt_ids: List[int]
    max_new_tokens: int = 64
    eos_ids: Tuple[int, ...] = ()
    temperature: float = 0.0   # <= 0: greedy
    top_k: int = 0             # 0: off
    top_p: float = 1.0         # 1: off
    seed: Optional[int] = None  # None: a fresh seed per request

    # --- filled in by the engine ---
    id: int = -1
    state: str = "waiting"     # waiting -> running -> finished
    output_ids: List[int] = field(default_factory=list)
    finish_reason: Optional[str] = None   # "stop" | "length" | "abort"
    cancelled: bool = False
    num_computed: int = 0      # tokens of prompt + output whose keys and values are in the cache
    admit_seq: int = 0         # admission order; the youngest running request is preempted first
    preemptions: int = 0
    arrival_time: float = 0.0
    admitted_time: Optional[float] = None
    first_token_time: Optional[float] = None
    finish_time: Optional[float] = None
    token_times: List[float] = field(default_factory=list)
    sample_seed: int = 0       # the seed the draws actually use

    def __post_init__(self):
        self.prompt_ids = [int(t) for t in self.prompt_ids]
        self.eos_ids = tuple(int(t) for t in self.eos_ids)
        if self.max_new_tokens < 1:
            raise ValueError("max_new_tokens must be at least 1")
        if self.top_k < 0:
            raise ValueError("top_k must be >= 0")
        if not 0.0 < self.top_p <= 1.0:
            raise ValueError("top_p must be in (0, 1]")

    @property
    def tokens(self) -> List[int]:
        """Everything the model has to have seen before the next token: prompt and output so far."""
        return self.prompt_ids + self.output_ids

    @property
    def num_tokens(self) -> int:
        return len(self.prompt_ids) + len(self.output_ids)

    # timing, as in the reference (engine.py:63-82)
    @property
    def ttft(self) -> Optional[float]:
        return None if self.first_token_time is None else self.first_token_time - self.arrival_time

    @property
    def queue_wait(self) -> Optional[float]:
        return None if self.admitted_time is None else self.admitted_time - self.arrival_time

    @property
    def e2e(self) -> Optional[float]:
        return None if self.finish_time is None else self.finish_time - self.arrival_time

    @property
    def tpot(self) -> Optional[float]:
        n = len(self.token_times)
        return None if n < 2 else (self.token_times[-1] - self.token_times[0]) / (n - 1)


@dataclass
class StepRecord:
    n_prefill_tokens: int   # tokens of prompt portions (and of recomputation after a preemption)
    decode_batch: int       # requests that ran a single decoded token
    useful_rows: int        # requests that got a token this step
    duration: float
    n_preempted: int = 0
    n_admitted: int = 0
    decode_steps: int = 0   # decode steps this record covers (several when one launch ran several steps)


@dataclass
class Scheduled:
    """One request's share of a step: tokens[start : start + count]; ``sample`` if they reach its end."""

    request: Request
    start: int
    count: int
    sample: bool
