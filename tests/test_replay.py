"""Replay the same requests whole, with the last 32 tokens decoded one by one, in portions of changing
size, and mixed with other requests so that pages are used again, in 32-bit and in bfloat16, and compare
every written logit with the plain implementation."""
import io
import subprocess
import sys

import numpy as np
import pytest
import torch

from tests import traces
from tests.conftest import ROOT, TINY
from tests.plain import qwen2_plain as P

pytestmark = pytest.mark.gpu

# The oracle is the plain implementation in double with the stored weights.
# float32: the reference's own bound for equal paths (max |dlogit| < 1e-3, tests/test_kv_cache.py:39).
# bfloat16: no fixed number fits models whose softmax amplifies rounding differently, so the bound is
# measured per request: the plain implementation is run once more with every stored activation rounded to
# bfloat16, and the engine may stray from the exact logits at most BF16_NOISE times as far as that
# faithful computation does at its worst place (a wrong key, page or position strays much further).
F32_ATOL = 1e-3
BF16_NOISE = 3.0


def make_model(tmp_path_factory, name, std, dtype="bfloat16", seed=0):
    from llm_infrence_engine_amd.config import config_from_dict
    from llm_infrence_engine_amd.weights import write_random_model

    d = tmp_path_factory.mktemp(f"tiny{name}")
    return write_random_model(d, config_from_dict(TINY[name]), seed=seed, dtype=dtype, std=std)


def make_requests(vocab, lengths, seed):
    rng = np.random.default_rng(seed)
    return {f"r{i}": [int(t) for t in rng.integers(0, vocab, n)] for i, n in enumerate(lengths)}


class Oracle(dict):
    """request -> exact logits [T, V]; ``noise[request]``: worst deviation of a bfloat16-rounding plain run."""


def oracle(model_dir, requests):
    cfg = P.read_config(model_dir)
    w = P.read_weights(model_dir, torch.float64)
    out = Oracle()
    out.noise = {}
    for rid, toks in requests.items():
        out[rid] = P.forward(w, cfg, toks).numpy()
        out.noise[rid] = float(np.abs(P.forward(w, cfg, toks, act_dtype=torch.bfloat16).numpy() - out[rid]).max())
    return out


def run_replay(model_dir, dtype, steps, out, max_tokens, page_size=16):
    from llm_infrence_engine_amd.engine.trace import replay

    log = io.StringIO()
    runner = replay(model_dir, dtype, out, max_tokens, traces.to_lines(steps), log=log, page_size=page_size)
    assert log.getvalue().split() == [x for st in steps for x in ("done", str(st["step"]))]
    runner.manager.check_invariants()
    assert all(g.allocator.num_in_use() == 0 for g in runner.manager.groups), "a finished request kept pages"
    if dtype == "bfloat16":
        # the serving path: steps are replayed from captured graphs, single tokens and portions alike
        g = runner.graphs
        assert g is not None and g.launches > 0 and g.max_portion_tokens > 0
        n_steps = sum(1 for st in steps if st["entries"])
        small = sum(1 for st in steps if st["entries"] and (sum(len(e["tokens"]) for e in st["entries"]) <= g.max_portion_tokens
                                                            or all(len(e["tokens"]) == 1 for e in st["entries"])))
        assert g.launches == small, f"{g.launches} of {n_steps} steps were replayed from graphs, {small} could have been"
    else:
        assert runner.graphs is None
    return runner


def assert_pages_were_used_again(runner):
    """The pool was so small that pages given back by one request were handed out to another."""
    for g in runner.manager.groups:
        again = g.allocator.pages_granted_again()
        assert again > 0, f"no page of a pool of {g.allocator.num_pages} was handed out twice: the trace reuses nothing"


def compare(got, want, dtype, requests):
    assert got, "nothing was written"
    worst = 0.0
    for (rid, pos), row in got.items():
        ref = want[rid][pos]
        err = np.abs(row.astype(np.float64) - ref).max()
        bound = F32_ATOL if dtype == "float32" else BF16_NOISE * want.noise[rid]
        assert err < bound, f"request {rid} position {pos}: max |dlogit| {err:.3e} >= {bound:.3e}"
        if dtype == "float32":
            assert row.argmax() == ref.argmax() or np.sort(ref)[-1] - np.sort(ref)[-2] < 2 * F32_ATOL
        worst = max(worst, err / bound)
    return worst


LENGTHS = {"A": [5, 11, 17, 70, 129, 40, 200], "B": [1, 9, 23, 40, 150, 77, 64], "C": [33, 2, 96, 180, 50, 65, 31],
           "D": [70, 3, 160, 33, 97, 240, 64]}
# pages of 4 and 8 tokens go to the generic kernels in both types; with pages of 16 and 32, B (head size 32)
# and D (head size 64, 7 query heads per key/value head) run the matrix-core attention in bfloat16
SETUPS = {"A": ("A", 4), "B": ("B", 8), "C": ("C", 16), "B16": ("B", 16), "D": ("D", 16), "D32": ("D", 32)}
STD = {"A": 0.15, "B": 0.15, "C": 0.15, "D": 0.08}


@pytest.fixture(scope="module", params=list(SETUPS))
def setup(request, tmp_path_factory):
    name, page = SETUPS[request.param]
    # weights large enough for attention scores of order one, so that a wrong key, position or page changes the logits
    model_dir = make_model(tmp_path_factory, name, std=STD[name], seed={"A": 0, "B": 1, "C": 2, "D": 3}[name])
    reqs = make_requests(TINY[name]["vocab_size"], LENGTHS[name], seed=ord(name))
    return (name, page), model_dir, reqs, oracle(model_dir, reqs)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("mode", ["whole", "bulk_then_single", "changing_portions", "mixed"])
def test_replay_modes(setup, tmp_path, dtype, mode):
    (name, page), model_dir, reqs, want = setup
    up = lambda n: -(-n // 64) * 64
    if mode == "mixed":
        # room for the longest request and a little more: requests wait for pages, and freed pages are used again
        max_tokens = up(max(len(t) for t in reqs.values())) + 128
        steps = traces.mixed(reqs, max_tokens, seed=3)
    else:
        max_tokens = up(max(len(t) for t in reqs.values()))
        steps = getattr(traces, mode)(reqs)
    runner = run_replay(model_dir, dtype, steps, tmp_path, max_tokens, page_size=page)
    got = traces.collect(steps, tmp_path, TINY[name]["vocab_size"])
    if mode != "mixed":
        assert len(got) == sum(len(t) for t in reqs.values())
    else:
        assert_pages_were_used_again(runner)
        assert max(len(st["entries"]) for st in steps) >= 3, "the mixed trace never had three requests in a step"
    worst = compare(got, want, dtype, reqs)
    print(f"tiny {name} page {page} {dtype} {mode}: worst error is {worst:.3f} of its bound over {len(got)} places")


def test_baseline_distribution_weights_too(tmp_path_factory, tmp_path):
    """The stated distributions (N(0, 0.02) matrices and biases, norms 1 + N(0, 0.1)), stored in float."""
    model_dir = make_model(tmp_path_factory, "A", std=0.02, dtype="float32", seed=0)
    reqs = make_requests(256, [5, 11, 17], seed=0)
    want = oracle(model_dir, reqs)
    steps = traces.bulk_then_single(reqs, tail=8)
    run_replay(model_dir, "float32", steps, tmp_path, 64, page_size=4)
    compare(traces.collect(steps, tmp_path, 256), want, "float32", reqs)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(tmp_path_factory, tmp_path, dtype):
    """bin/trace_run as a user starts it: steps on standard input, files in --out, `done <step>` lines."""
    model_dir = make_model(tmp_path_factory, "B", std=0.15, seed=5)
    reqs = make_requests(384, [50, 20, 70], seed=9)
    want = oracle(model_dir, reqs)
    steps = traces.mixed(reqs, 128, seed=1)
    out = tmp_path / "out"
    r = subprocess.run([sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(model_dir), "--dtype", dtype,
                        "--out", str(out), "--max-tokens", "128"], input="\n".join(traces.to_lines(steps)) + "\n",
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr
    assert r.stdout.split() == [x for st in steps for x in ("done", str(st["step"]))]
    compare(traces.collect(steps, out, 384), want, dtype, reqs)


@pytest.fixture(scope="module")
def half_b(tmp_path_factory):
    """All 24 layers of the Qwen2.5-0.5B configuration with random weights, as a model folder."""
    from llm_infrence_engine_amd.config import config_from_dict, preset
    from llm_infrence_engine_amd.weights import write_random_model

    d = tmp_path_factory.mktemp("halfb")
    cfg = preset("0.5b")
    assert cfg["num_hidden_layers"] == 24 and cfg["vocab_size"] == 151936
    write_random_model(d, config_from_dict(cfg), seed=7, dtype="bfloat16", std=0.05)
    reqs = make_requests(151936, [90, 40, 150], seed=3)
    return d, reqs, oracle(d, reqs)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("mode", ["whole", "bulk_then_single", "changing_portions", "mixed"])
def test_replay_of_the_half_billion_model_at_its_real_depth(half_b, tmp_path, dtype, mode):
    """Qwen2.5-0.5B as config.json describes it (24 layers, hidden 896, 14 heads over 2 key/value heads of 64,
    intermediate 4864, vocabulary 151936, tied head) with random weights, in all four ways of cutting the work,
    as the reference checks its cache paths on the real model (tests/test_kv_cache.py:30-55,
    tests/test_paged.py:143-166): what 24 layers do to a rounding error is part of the comparison."""
    d, reqs, want = half_b
    # mixed: room for the two short requests together or the long one alone, so the long one takes over their pages
    max_tokens = 64 * 3
    steps = traces.mixed(reqs, max_tokens, seed=2) if mode == "mixed" else getattr(traces, mode)(reqs)
    # logits of every place would be 150 MB a request: ask for the last place of every portion only, and of
    # whole requests every sixteenth place as well
    for st in steps:
        for e in st["entries"]:
            n = len(e["tokens"])
            e["want"] = sorted(set(range(15, n, 16)) | {n - 1}) if mode == "whole" else [n - 1]
    runner = run_replay(d, dtype, steps, tmp_path, max_tokens, page_size=16)
    if mode == "mixed":
        assert_pages_were_used_again(runner)
    worst = compare(traces.collect(steps, tmp_path, 151936), want, dtype, reqs)
    print(f"0.5B, 24 layers, {dtype} {mode}: worst error is {worst:.3f} of its bound")
