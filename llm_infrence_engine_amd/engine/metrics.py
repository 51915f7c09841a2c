"""What a finished run looked like from outside: latencies of its requests, throughput, use of the decode rows.

Same figures and names as the reference's summary (src/miniserve/metrics.py:10-45), computed from the
``Request`` timing fields and the engine's ``StepRecord`` list.
"""
from __future__ import annotations

from typing import Dict, Iterable, List, Optional, Sequence

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


def _known(values: Iterable[Optional[float]]) -> List[float]:
    return [v for v in values if v is not None]


def summarize(requests: Sequence[Request], steps: Sequence[StepRecord], wall_time: float) -> Dict[str, float]:
    """Figures of a run over its finished requests (src/miniserve/metrics.py:20-45): tokens and tokens a second,
    time to the first token (mean, median, 95th percentile), waiting time, whole latency, time per output token,
    and how well the decode batches were used (``wasted_row_fraction``: rows that were computed but gave no
    token: with continuous batching only the steps that a launch of several ran past a request's stop id).  A
    record that covers several decode steps of one launch counts its rows for each of them."""
    done = [r for r in requests if r.state == "finished"]
    tokens = sum(len(r.output_ids) for r in done)
    ttft, e2e = _known(r.ttft for r in done), _known(r.e2e for r in done)
    tpot, wait = _known(r.tpot for r in done), _known(r.queue_wait for r in done)
    decoding = [s for s in steps if s.decode_batch > 0]
    launches = sum(max(1, s.decode_steps) for s in decoding)     # decode steps, several to a record at times
    rows = sum(s.decode_batch * max(1, s.decode_steps) for s in decoding)
    # a record's useful rows also count requests whose prompt ended in that step; those are no decode rows
    useful = sum(min(s.useful_rows, s.decode_batch * max(1, s.decode_steps)) for s in decoding)
    return {
        "requests": len(done),
        "output_tokens": tokens,
        "wall_time_s": wall_time,
        "throughput_tok_s": tokens / wall_time if wall_time > 0 else 0.0,
        "ttft_mean_s": _mean(ttft),
        "ttft_p50_s": percentile(ttft, 50),
        "ttft_p95_s": percentile(ttft, 95),
        "queue_wait_mean_s": _mean(wait),
        "e2e_mean_s": _mean(e2e),
        "e2e_p95_s": percentile(e2e, 95),
        "tpot_mean_ms": 1000.0 * _mean(tpot),
        "steps": len(steps),
        "mean_decode_batch": rows / launches if launches else 0.0,
        "wasted_row_fraction": 1.0 - useful / rows if rows else 0.0,
    }
