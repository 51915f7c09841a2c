"""Token choice for a step's rows: greedy, temperature, top-k, top-p, repeatable from a seed.

Options and their order follow the reference (src/miniserve/sampler.py:12-55): temperature <= 0 is the
argmax; otherwise logits / temperature, keep the top_k largest (ties kept), keep the smallest set whose
mass reaches top_p (the most likely token always stays), softmax, draw.  The whole batch is decided by one
kernel launch and one copy back (the reference does one argmax for all greedy rows, engine.py:260-277).
The draw uses a counter-based generator keyed by (seed, index of the token in the output), so a preempted
and recomputed request draws the same tokens again; the stream is not that of torch.multinomial.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional, Sequence, Tuple

import torch

from ..kernels import ops


@dataclass
class SamplingParams:
    max_new_tokens: int = 64
    temperature: float = 0.0
    top_k: int = 0
    top_p: float = 1.0
    seed: Optional[int] = None
    eos_ids: Tuple[int, ...] = ()


class Sampler:
    def __init__(self, device):
        self.device = device

    def sample(self, logits: torch.Tensor, requests: Sequence) -> List[int]:
        """One token per row of float logits [M, V]; ``requests[i]`` gives row i its temperature, top_k,
        top_p, sample_seed and the index of the token to draw (its output length)."""
        M = logits.shape[0]
        if M == 0:
            return []
        out = torch.empty(M, dtype=torch.int32, device=logits.device)
        if all(r.temperature <= 0.0 for r in requests):
            ops.sample(logits, out)
        else:
            dev = logits.device
            f = torch.tensor([[r.temperature, r.top_p] for r in requests], dtype=torch.float32).to(dev)
            i = torch.tensor([[r.top_k, len(r.output_ids)] for r in requests], dtype=torch.int32).to(dev)
            seeds = torch.tensor([r.sample_seed & 0x7FFFFFFFFFFFFFFF for r in requests], dtype=torch.int64).to(dev)
            V = logits.shape[1]
            ops.sample(logits, out, f[:, 0].contiguous(), i[:, 0].contiguous(), f[:, 1].contiguous(), seeds,
                       i[:, 1].contiguous(), use_top_k=any(0 < r.top_k < V for r in requests),
                       use_top_p=any(r.top_p < 1.0 for r in requests))
        return out.tolist()
