"""What a finished run looked like from outside: latencies of its requests, throughput, use of the decode rows.

Same figures and names as the reference's summary (src/miniserve/metrics.py:10-45), computed from the
``Request`` timing fields and the engine's ``StepRecord`` list.
"""
from __future__ import annotations

from typing import Dict, List, Sequence

from .request import Request, StepRecord

NAN = float("nan")


def percentile(values: Sequence[float], p: float) -> float:
    """The p-th percentile (0..100) with linear interpolation between the two nearest ranks; nan if there is
    no value (src/miniserve/metrics.py:10-17)."""
    if not 0.0 <= p <= 100.0:
        raise ValueError(f"a percentile lies between 0 and 100, not {p}")
    ordered = sorted(values)
    if not ordered:
        return NAN
    rank = p / 100.0 * (len(ordered) - 1)
    below = int(rank)
    above = min(below + 1, len(ordered) - 1)
    return ordered[below] + (rank - below) * (ordered[above] - ordered[below])


def _mean(values: List[float]) -> float:
    return sum(values) / len(values) if values else NAN


def _timings(done: Sequence[Request], field: str) -> List[float]:
    """One timing property of every finished request that has it."""
    return [v for v in (getattr(r, field) for r in done) if v is not None]


def summarize(requests: Sequence[Request], steps: Sequence[StepRecord], wall_time: float) -> Dict[str, float]:
    """Figures of a run over its finished requests (src/miniserve/metrics.py:20-45): tokens and tokens a second,
    time to the first token (mean, median, 95th percentile), waiting time, whole latency, time per output token,
    and how well the decode batches were used (``wasted_row_fraction``: rows that were computed but gave no
    token: with continuous batching only the steps that a launch of several ran past a request's stop id).  A
    record that covers several decode steps of one launch counts its rows for each of them."""
    done = [r for r in requests if r.state == "finished"]
    out: Dict[str, float] = {"requests": len(done), "output_tokens": sum(len(r.output_ids) for r in done),
                             "wall_time_s": wall_time, "steps": len(steps)}
    out["throughput_tok_s"] = out["output_tokens"] / wall_time if wall_time > 0 else 0.0

    first = _timings(done, "ttft")
    out.update(ttft_mean_s=_mean(first), ttft_p50_s=percentile(first, 50), ttft_p95_s=percentile(first, 95))
    out["queue_wait_mean_s"] = _mean(_timings(done, "queue_wait"))
    whole = _timings(done, "e2e")
    out.update(e2e_mean_s=_mean(whole), e2e_p95_s=percentile(whole, 95))
    out["tpot_mean_ms"] = 1000.0 * _mean(_timings(done, "tpot"))

    n_steps = rows = useful = 0
    for rec in steps:
        if rec.decode_batch <= 0:
            continue
        k = max(1, rec.decode_steps)              # decode steps this record covers
        n_steps += k
        rows += rec.decode_batch * k
        # a record's useful rows also count requests whose prompt ended in that step; those are no decode rows
        useful += min(rec.useful_rows, rec.decode_batch * k)
    out["mean_decode_batch"] = rows / n_steps if n_steps else 0.0
    out["wasted_row_fraction"] = 1.0 - useful / rows if rows else 0.0
    return out
