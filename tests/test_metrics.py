"""The run summary: percentiles and the figures of a finished run, on hand-made records (no GPU)."""
import math

import pytest

from llm_infrence_engine_amd.engine.metrics import percentile, summarize
from llm_infrence_engine_amd.engine.request import Request, StepRecord


def test_percentile_interpolates_between_ranks():
    v = [4.0, 1.0, 3.0, 2.0]
    assert percentile(v, 0) == 1.0 and percentile(v, 100) == 4.0
    assert percentile(v, 50) == 2.5                    # halfway between the second and the third
    assert percentile(v, 95) == pytest.approx(3.85)    # rank 2.85 of 0..3
    assert percentile([7.0], 95) == 7.0
    assert math.isnan(percentile([], 50))
    with pytest.raises(ValueError, match="between 0 and 100"):
        percentile(v, 101)


def finished(arrival, admitted, token_times, n_prompt=3):
    r = Request([1] * n_prompt, max_new_tokens=len(token_times))
    r.state, r.finish_reason = "finished", "length"
    r.arrival_time, r.admitted_time = arrival, admitted
    r.output_ids = [5] * len(token_times)
    r.token_times = list(token_times)
    r.first_token_time, r.finish_time = token_times[0], token_times[-1]
    return r


def test_summary_arithmetic_on_hand_made_records():
    a = finished(0.0, 0.5, [1.0, 1.5, 2.0])           # ttft 1.0, e2e 2.0, tpot 0.5, wait 0.5
    b = finished(1.0, 1.0, [4.0, 4.25])               # ttft 3.0, e2e 3.25, tpot 0.25, wait 0
    waiting = Request([1, 2], max_new_tokens=4)        # never ran: not counted
    steps = [StepRecord(6, 0, 2, 0.1),                 # two prompts end here: two tokens, no decode rows
             StepRecord(0, 2, 2, 0.1, decode_steps=1),
             StepRecord(3, 1, 2, 0.1, decode_steps=1),  # a decode row beside a prompt's end
             StepRecord(0, 2, 5, 0.1, decode_steps=4)]  # four steps in one launch; a stop id cost three rows
    s = summarize([a, b, waiting], steps, wall_time=4.0)
    assert s["requests"] == 2 and s["output_tokens"] == 5
    assert s["throughput_tok_s"] == 1.25
    assert s["ttft_mean_s"] == 2.0 and s["ttft_p50_s"] == 2.0 and s["ttft_p95_s"] == pytest.approx(2.9)
    assert s["queue_wait_mean_s"] == 0.25
    assert s["e2e_mean_s"] == pytest.approx(2.625) and s["e2e_p95_s"] == pytest.approx(3.1875)
    assert s["tpot_mean_ms"] == pytest.approx(375.0)
    assert s["steps"] == 4
    assert s["mean_decode_batch"] == pytest.approx(11 / 6)         # rows 2 + 1 + 2 * 4 over 1 + 1 + 4 steps
    assert s["wasted_row_fraction"] == pytest.approx(1 - 8 / 11)   # 2 + 1 + 5 of them gave a token


def test_summary_of_nothing():
    s = summarize([], [], 0.0)
    assert s["requests"] == 0 and s["throughput_tok_s"] == 0.0 and s["wasted_row_fraction"] == 0.0
    assert math.isnan(s["ttft_mean_s"]) and math.isnan(s["tpot_mean_ms"])
