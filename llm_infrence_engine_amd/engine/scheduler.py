"""Continuous batching with chunked prefill over the paged cache: who runs in the next step.

Every step is one mixed batch under a token budget.  In order:

1. running requests that need a single token (decoding) get it first; if such a request needs a new page
   and none is free, the *youngest* running request is preempted, possibly the request itself
   (src/miniserve/paged_engine.py:152-161): its pages are given back, it returns to the front of the
   queue and is later recomputed from prompt + output so far, so its output does not change
   (paged_engine.py:179-187, 100);
2. running requests still inside their prompt get the next portion, as large as the budget, the portion
   limit and the free pages allow (a portion never preempts anyone);
3. waiting requests are admitted first come first served, without skipping (paged_engine.py:89-91), while a
   row, budget and pages for the first portion plus one spare page per running request are there
   (paged_engine.py:114-119);
4. if nothing could be scheduled although requests are running (all of them stuck inside their prompts
   with no page free), the youngest is preempted and the pass is repeated.

A request whose last token is computed in a step gets its next token sampled from that step's logits;
there is no separate prefill forward as in the reference (paged_engine.py:126-127), which also has no
token budget or portions (src/miniserve/engine.py:13-14).

Only decisions and bookkeeping live here: no tensors, so it runs (and is tested) without a GPU.
"""
from __future__ import annotations

import random
import threading
import time
from collections import deque
from typing import Callable, Deque, List, Optional

from ..cache.manager import CacheManager
from ..config.engine_config import EngineConfig
from .request import Request, Scheduled


class Scheduler:
    def __init__(self, manager: CacheManager, config: EngineConfig, clock: Callable[[], float] = time.perf_counter,
                 on_token: Optional[Callable[[Request, int], None]] = None,
                 on_finish: Optional[Callable[[Request], None]] = None):
        self.manager, self.config, self.clock = manager, config, clock
        self.on_token, self.on_finish = on_token, on_finish
        self.waiting: Deque[Request] = deque()
        self.running: List[Request] = []
        self.finished: List[Request] = []
        self.preemptions = 0
        self._next_id = 0
        self._admit_counter = 0
        self._seed_rng = random.Random()
        # add_request and cancel may be called from another thread than the one that steps
        # (src/miniserve/engine.py:136, 149): ids and the waiting queue change under this lock
        self._lock = threading.Lock()

    # ------------------------------------------------------------------ public
    def add_request(self, req: Request) -> Request:
        if not req.prompt_ids:
            raise ValueError("empty prompt")
        need = len(req.prompt_ids) + req.max_new_tokens
        if need > self.config.max_len:
            raise ValueError(f"request needs {need} cache positions but max_len is {self.config.max_len}")
        if need > self.manager.capacity_tokens():
            raise ValueError("request can never fit in the page pool")
        with self._lock:
            req.id = self._next_id
            self._next_id += 1
            req.arrival_time = self.clock()
            req.state = "waiting"
            req.sample_seed = req.seed if req.seed is not None else self._seed_rng.getrandbits(62)
            self.waiting.append(req)
        return req

    def has_work(self) -> bool:
        return bool(self.waiting) or bool(self.running)

    def cancel(self, req: Request) -> None:
        """Drop the request at the start of the next step (src/miniserve/engine.py:163-177)."""
        req.cancelled = True

    # ------------------------------------------------------------------ one step's decisions
    def schedule(self) -> List[Scheduled]:
        self._reap_cancelled()
        self.last_preempted = 0
        self.last_admitted = 0
        while True:
            out = self._schedule_once()
            if out or not self.running:
                return out
            self._preempt(max(self.running, key=lambda r: r.admit_seq))  # rule 4

    def _schedule_once(self) -> List[Scheduled]:
        m, cfg = self.manager, self.config
        budget = cfg.max_num_batched_tokens
        chunk = cfg.max_prefill_chunk or budget
        out: List[Scheduled] = []

        for r in sorted(self.running, key=lambda r: r.admit_seq):          # rule 1
            if r.state != "running" or r.num_tokens - r.num_computed != 1 or budget == 0:
                continue
            while r.state == "running" and not m.can_grow(r.id, r.num_computed + 1):
                self._preempt(max(self.running, key=lambda x: x.admit_seq))
            if r.state != "running":
                continue
            m.grow(r.id, r.num_computed + 1)
            out.append(Scheduled(r, r.num_computed, 1, True))
            budget -= 1

        for r in sorted(self.running, key=lambda r: r.admit_seq):          # rule 2
            left = r.num_tokens - r.num_computed
            if r.state != "running" or left <= 1 or budget == 0:
                continue
            n = min(left, budget, chunk, m.tokens_that_fit(r.id))
            if n <= 0:
                continue
            m.grow(r.id, r.num_computed + n)
            out.append(Scheduled(r, r.num_computed, n, n == left))
            budget -= n

        while self.waiting and len(self.running) < cfg.max_seqs and budget > 0 and m.free_rows() > 0:   # rule 3
            r = self.waiting[0]
            m.add(r.id)
            n = min(r.num_tokens, budget, chunk)
            if not m.can_grow(r.id, n, reserve=len(self.running)):
                m.free(r.id)
                break
            self.waiting.popleft()
            m.grow(r.id, n)
            r.state = "running"
            r.num_computed = 0
            if r.admitted_time is None:
                r.admitted_time = self.clock()
            self._admit_counter += 1
            r.admit_seq = self._admit_counter
            self.running.append(r)
            self.last_admitted += 1
            out.append(Scheduled(r, 0, n, n == r.num_tokens))
            budget -= n
        return out

    # ------------------------------------------------------------------ after the model ran
    def commit(self, scheduled: List[Scheduled], sampled: List[int]) -> int:
        """Advance the requests; ``sampled`` holds one token for every entry with ``sample`` set, in order.
        Returns how many requests got a token."""
        it = iter(sampled)
        useful = 0
        for s in scheduled:
            r = s.request
            r.num_computed = s.start + s.count
            if s.sample:
                self._emit(r, int(next(it)))
                useful += 1
        return useful

    def _emit(self, r: Request, tok: int) -> None:
        now = self.clock()
        if tok in r.eos_ids:                      # the stop id is not emitted (engine.py:281-283)
            self._finish(r, "stop", now)
            return
        r.output_ids.append(tok)
        r.token_times.append(now)
        if r.first_token_time is None:
            r.first_token_time = now
        if self.on_token:
            self.on_token(r, tok)
        if len(r.output_ids) >= r.max_new_tokens:
            self._finish(r, "length", now)

    def _finish(self, r: Request, reason: str, now: float) -> None:
        if r.state == "running":
            self.running.remove(r)
            self.manager.free(r.id)
        r.state, r.finish_reason, r.finish_time = "finished", reason, now
        if reason != "abort":
            self.finished.append(r)
        if self.on_finish:
            self.on_finish(r)

    def _preempt(self, victim: Request) -> None:
        self.running.remove(victim)
        self.manager.free(victim.id)
        victim.state = "waiting"
        victim.num_computed = 0
        victim.preemptions += 1
        self.preemptions += 1
        self.last_preempted += 1
        self.waiting.appendleft(victim)

    def _reap_cancelled(self) -> None:
        now = self.clock()
        with self._lock:
            dropped = [r for r in self.waiting if r.cancelled]
            for r in dropped:
                self.waiting.remove(r)
        for r in dropped:
            self._finish(r, "abort", now)
        for r in [r for r in self.running if r.cancelled]:
            self._finish(r, "abort", now)
