"""``LLM(model_dir).generate(prompts, params)``: load once, generate for many prompts through the
continuous-batching engine.  The reference has no such class (its package root is empty); the options are
those of its ``Request`` (src/miniserve/engine.py:32-38) and its engine's constructor
(src/miniserve/paged_engine.py:24-36)."""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional, Sequence, Union

from ..loading import load_model
from ..parts.model import Model
from ..sampling import SamplingParams
from .engine import Engine
from .request import Request


@dataclass
class Output:
    token_ids: List[int]
    finish_reason: str
    prompt_len: int
    ttft: Optional[float]
    e2e: Optional[float]
    preemptions: int


class LLM:
    def __init__(self, model: Union[str, Model], dtype: str = "bfloat16", device: str = "cuda:0", **engine_options):
        """``model``: a folder with config.json and safetensors, or a loaded model.  ``engine_options`` go to
        ``Engine`` (num_blocks, block_size, max_seqs, max_len, max_num_batched_tokens, max_prefill_chunk, hip_graphs)."""
        self.model = model if isinstance(model, Model) else load_model(model, dtype, device)
        self.engine = Engine(self.model, **engine_options)

    def generate(self, prompts: Sequence[Sequence[int]],
                 params: Union[SamplingParams, Sequence[SamplingParams], None] = None) -> List[Output]:
        """Token ids in, token ids out; one ``Output`` per prompt, in order."""
        if params is None:
            params = SamplingParams()
        plist = [params] * len(prompts) if isinstance(params, SamplingParams) else list(params)
        if len(plist) != len(prompts):
            raise ValueError("one SamplingParams per prompt, or one for all")
        reqs = [self.engine.add_request(Request(list(p), sp.max_new_tokens, tuple(sp.eos_ids), sp.temperature,
                                                sp.top_k, sp.top_p, sp.seed)) for p, sp in zip(prompts, plist)]
        self.engine.run_until_idle()
        return [Output(list(r.output_ids), r.finish_reason, len(r.prompt_ids), r.ttft, r.e2e, r.preemptions)
                for r in reqs]
