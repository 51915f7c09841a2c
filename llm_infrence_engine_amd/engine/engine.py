"""The serving loop: scheduler above, step function below, sampler beside.

Public face after the reference's ``Engine`` / ``PagedEngine`` (src/miniserve/engine.py:94-205,
src/miniserve/paged_engine.py:24-80): ``add_request``, ``has_work``, ``cancel``, ``step``,
``run_until_idle``, ``finished``, ``steps``, ``stats``; and ``generate`` after
src/miniserve/generate.py:85-135.
"""
from __future__ import annotations

import time
from dataclasses import dataclass, field
from typing import Callable, List, Optional, Sequence

import torch

from ..cache import CacheLayout
from ..cache.allocator import OutOfPages
from ..config.engine_config import EngineConfig
from ..parts.model import Model
from ..sampling import Sampler
from .batch import Sampling, StepEntry
from .request import Request, StepRecord
from .runner import ModelRunner
from .scheduler import Scheduler


def memory_beside_the_pages(config: EngineConfig, model: Model, layout: CacheLayout) -> int:
    """An estimate, in bytes, of what an engine holds on the device beside its weights and cache pages: the
    per-request state of the runs that keep one (one slot more than requests), the block tables, and with graphs
    the float logits that every batch-size bucket keeps and the activations of the largest captured step (all
    graphs share one pool): some ten rows of the widest activation per token."""
    itemsize = model.rt.dtype.itemsize
    total = 0
    for need in layout.state_needs.values():
        for n in (need if isinstance(need, tuple) else (need,)):
            size = 1
            for s in n.shape:
                size *= s
            total += (config.max_seqs + 1) * size * torch.empty(0, dtype=n.dtype).element_size()
    total += len(layout.group_keys) * (config.max_seqs + 1) * config.pages_per_request * 4
    widest = max([model.spec.hidden_size * 4] + [s.shape[0] * itemsize for s in model.tensor_specs()
                                                  if s.role == "matrix" and len(s.shape) == 2
                                                  and s.shape[0] != model.spec.vocab_size])
    tokens = config.max_num_batched_tokens
    if config.hip_graphs:
        from .graph import default_batch_sizes

        total += sum(default_batch_sizes(config.max_seqs)) * model.spec.vocab_size * 4
        tokens += config.max_seqs
    return total + 10 * tokens * widest


class Engine:
    def __init__(self, model: Model, num_blocks: Optional[int] = None, block_size: int = 16, max_seqs: int = 32,
                 max_len: int = 1024, max_num_batched_tokens: int = 2048, max_prefill_chunk: Optional[int] = None,
                 on_token: Optional[Callable[[Request, int], None]] = None,
                 on_finish: Optional[Callable[[Request], None]] = None,
                 clock: Callable[[], float] = time.perf_counter, hip_graphs: Optional[bool] = None,
                 decode_steps_per_launch: int = 1, capture_at_start: bool = True,
                 gpu_memory_fraction: Optional[float] = None, graph_portion_tokens: Optional[int] = None):
        """``hip_graphs`` None: on when the model serves in bfloat16 (float32 is the checking path and launches
        every kernel itself).  ``num_blocks`` None: as many pages as ``max_seqs`` requests of ``max_len`` tokens can
        fill, or with ``gpu_memory_fraction`` as many of them as that share of the device's memory has room for
        beside the weights.
        With ``hip_graphs`` every graph that serving can reach is captured here, before the first request
        (as the reference's constructor does, src/miniserve/graph_decode.py:46-47), unless ``capture_at_start``
        is False: then a graph is captured when a step first needs it.
        ``decode_steps_per_launch`` > 1 (with ``hip_graphs``): while every running request is decoding and
        nobody waits, up to that many decode steps run in one graph launch, each fed the token the one before
        chose on the device (the argmax, or the request's own draw); a stop id is then noticed up to that many
        steps late (the surplus tokens are dropped), so outputs do not change.
        ``graph_portion_tokens`` (with ``hip_graphs``): steps with prompt portions of up to that many tokens are
        replayed from graphs too (None: as far as the host would otherwise be what such a step waits for)."""
        dtype = {torch.float32: "float32", torch.bfloat16: "bfloat16"}[model.rt.dtype]
        self.config = EngineConfig(dtype=dtype, block_size=block_size, num_blocks=num_blocks, max_seqs=max_seqs,
                                   max_len=max_len, max_num_batched_tokens=max_num_batched_tokens,
                                   max_prefill_chunk=max_prefill_chunk, hip_graphs=hip_graphs,
                                   decode_steps_per_launch=decode_steps_per_launch,
                                   gpu_memory_fraction=gpu_memory_fraction, graph_portion_tokens=graph_portion_tokens,
                                   device=str(model.rt.device))
        self.model = model
        pages = self.config.resolved_num_blocks()
        if num_blocks is None and gpu_memory_fraction is not None:
            free, total = torch.cuda.mem_get_info(model.rt.device)
            layout = CacheLayout(model.run_needs())
            per_token = layout.bytes_per_token(model.rt.dtype.itemsize)
            pages = self.config.resolved_num_blocks(per_token, total, total - free,
                                                    memory_beside_the_pages(self.config, model, layout))
        self.runner = ModelRunner(model, block_size, pages, max_seqs, max_len, hip_graphs=self.config.hip_graphs,
                                  graph_portion_tokens=self.config.graph_portion_tokens)
        self.scheduler = Scheduler(self.runner.manager, self.config, clock, on_token, on_finish)
        self.sampler = Sampler(model.rt.device)
        self.clock = clock
        self.decode_steps_per_launch = max(1, decode_steps_per_launch) if self.runner.graphs is not None else 1
        if capture_at_start:
            self.warm_up()
        self.steps: List[StepRecord] = []
        self.peak_running = 0
        self.peak_pages_in_use = 0
        self.prefill_tokens_computed = 0

    def launch_sizes(self) -> List[int]:
        """The numbers of decode steps one graph launch may hold: powers of two up to ``decode_steps_per_launch``."""
        sizes, k = [], 1
        while k <= self.decode_steps_per_launch:
            sizes.append(k)
            k *= 2
        return sizes

    def warm_up(self) -> int:
        """Capture every decode graph this engine can need (all batch-size buckets, context classes and
        launch sizes), so that no step of serving holds a capture.  Returns the number of graphs held."""
        if self.runner.graphs is None:
            return 0
        return self.runner.graphs.warm_up(self.launch_sizes())

    # ------------------------------------------------------------------ the reference's public face
    def add_request(self, req: Request) -> Request:
        vocab = self.model.spec.vocab_size
        for t in req.prompt_ids:
            if not 0 <= t < vocab:
                raise ValueError(f"token id {t} is outside the vocabulary of {vocab}")
        return self.scheduler.add_request(req)

    def has_work(self) -> bool:
        return self.scheduler.has_work()

    def cancel(self, req: Request) -> None:
        self.scheduler.cancel(req)

    @property
    def finished(self) -> List[Request]:
        return self.scheduler.finished

    @property
    def running(self) -> List[Request]:
        return self.scheduler.running

    @property
    def waiting(self):
        return self.scheduler.waiting

    @property
    def preemptions(self) -> int:
        return self.scheduler.preemptions

    def _steps_ahead(self, sched, limit: int) -> int:
        """How many decode steps the next launch may hold: a power of two within the configured limit and
        within what every request still has to generate, if all of them decode and nobody waits; 0 if the step
        is not one of single decoded tokens that a graph launch can take."""
        if self.runner.graphs is None or len(sched) > self.runner.graphs.max_batch:
            return 0
        for s in sched:
            if s.count != 1 or s.start == 0 or not s.sample:
                return 0
        limit = min(limit, self.decode_steps_per_launch)
        if limit < 2 or self.scheduler.waiting:
            return 1
        for s in sched:
            r = s.request
            limit = min(limit, r.max_new_tokens - len(r.output_ids), self.config.max_len - r.num_computed)
        k = 1
        while k * 2 <= limit:
            k *= 2
        if k > 1:
            m = self.runner.manager
            try:
                for s in sched:
                    m.grow(s.request.id, s.start + k)
            except OutOfPages:
                return 1           # what was grown stays with its request: it will need it soon anyway
        return k

    def step(self, max_decode_steps: int = 1 << 30) -> StepRecord:
        t0 = self.clock()
        sched = self.scheduler.schedule()
        useful = 0
        if not sched and self.scheduler.has_work():
            raise RuntimeError("the scheduler could place no request although work is waiting")
        ahead = self._steps_ahead(sched, max_decode_steps) if sched else 0
        sampled = any(s.request.temperature > 0.0 for s in sched)
        if ahead > 1 or (ahead == 1 and sampled):
            # a request's newest token: its last output, or its prompt's last token when a portion left only that
            entries = [StepEntry(s.request.id, [(s.request.output_ids or s.request.prompt_ids)[-1]]) for s in sched]
            how = None
            if sampled:       # the draws happen on the device too, by each request's own rule, seed and count
                how = [Sampling(r.temperature, r.top_k, r.top_p, r.sample_seed, len(r.output_ids))
                       for r in (s.request for s in sched)]
            tokens = self.runner.decode_steps(entries, ahead, how)
            for k in range(ahead):      # as the single steps would have: a finished request drops its later tokens
                for i, s in enumerate(sched):
                    if s.request.state == "running":
                        s.request.num_computed += 1
                        self.scheduler._emit(s.request, tokens[k][i])
                        useful += 1
        elif sched:
            entries, rows = [], []
            for s in sched:
                toks = s.request.tokens[s.start:s.start + s.count]
                entries.append(StepEntry(s.request.id, toks, [s.count - 1] if s.sample else []))
                if s.sample:
                    rows.append(s.request)
            logits = self.runner.step(entries)
            greedy = self.runner.greedy_tokens
            if greedy is not None and len(rows) == len(entries) and all(r.temperature <= 0.0 for r in rows):
                chosen = greedy.tolist()       # the captured graph has already taken the argmax
            else:
                chosen = self.sampler.sample(logits, rows)
            useful = self.scheduler.commit(sched, chosen)
        n_decode = sum(1 for s in sched if s.count == 1 and s.start > 0)
        n_prefill = sum(s.count for s in sched) - n_decode
        decode_steps = max(ahead, 1) if n_decode else 0
        self.prefill_tokens_computed += n_prefill
        self.peak_running = max(self.peak_running, len(self.scheduler.running))
        in_use = max((g.allocator.num_in_use() for g in self.runner.manager.groups), default=0)
        self.peak_pages_in_use = max(self.peak_pages_in_use, in_use)
        rec = StepRecord(n_prefill, n_decode, useful, self.clock() - t0, self.scheduler.last_preempted,
                         self.scheduler.last_admitted, decode_steps)
        self.steps.append(rec)
        return rec

    def run_until_idle(self) -> None:
        while self.has_work():
            self.step()

    def stats(self) -> dict:
        m = self.runner.manager
        return {
            "prefill_tokens_computed": self.prefill_tokens_computed,
            "preemptions": self.scheduler.preemptions,
            "peak_running": self.peak_running,
            "peak_blocks_in_use": self.peak_pages_in_use,
            "pool_blocks": m.num_pages,
            "pool_mib": self.runner.pools.total_bytes() / 2 ** 20,
        }


# ---------------------------------------------------------------------------------------------- one sequence
@dataclass
class GenerationResult:
    """As the reference's (src/miniserve/generate.py:19-37)."""

    token_ids: List[int]
    prompt_len: int
    ttft: float
    total_time: float
    step_times: List[float] = field(default_factory=list)
    finish_reason: str = "length"
    cache_bytes: int = 0

    @property
    def decode_tps(self) -> float:
        t = sum(self.step_times)
        return len(self.step_times) / t if t > 0 else 0.0

    @property
    def ms_per_token(self) -> float:
        return 1000 * sum(self.step_times) / len(self.step_times) if self.step_times else 0.0


def generate(model: Model, prompt_ids: Sequence[int], max_new_tokens: int = 64, eos_ids: Sequence[int] = (),
             temperature: float = 0.0, top_k: int = 0, top_p: float = 1.0, seed: Optional[int] = None,
             block_size: int = 16) -> GenerationResult:
    """Generate from one prompt and measure, with the reference's option names
    (src/miniserve/generate.py:85-135).  The stop id is not part of the output."""
    need = len(prompt_ids) + max_new_tokens
    eng = Engine(model, num_blocks=-(-need // block_size), block_size=block_size, max_seqs=1, max_len=need,
                 max_num_batched_tokens=max(need, 1))
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    req = eng.add_request(Request(list(prompt_ids), max_new_tokens, tuple(eos_ids), temperature, top_k, top_p, seed))
    marks = []
    while eng.has_work():
        n = len(req.output_ids)
        eng.step()
        if len(req.output_ids) > n:
            marks.append(time.perf_counter())
    total = time.perf_counter() - t0
    per_token = eng.runner.layout.bytes_per_token(model.rt.dtype.itemsize)    # whatever the model's runs keep per token
    return GenerationResult(
        token_ids=list(req.output_ids), prompt_len=len(prompt_ids), ttft=(marks[0] - t0) if marks else total,
        total_time=total, step_times=[b - a for a, b in zip(marks, marks[1:])],
        finish_reason=req.finish_reason or "length", cache_bytes=per_token * (len(prompt_ids) + len(req.output_ids)))
