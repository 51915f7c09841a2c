"""The engine above the step function, on the GPU: greedy generation through the entry points against the
plain implementation, the scheduler under page pressure, sampling options, long decoding and the first
tokens of a sequence."""
import json
import subprocess
import sys

import numpy as np
import pytest
import torch

from tests.conftest import ROOT, TINY
from tests.plain import qwen2_plain as P

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def eng():
    import llm_infrence_engine_amd as e

    return e


@pytest.fixture(scope="module", params=["A", "B"])
def tiny(request, tmp_path_factory, eng):
    from llm_infrence_engine_amd.config import config_from_dict

    name = request.param
    d = tmp_path_factory.mktemp(f"gen{name}")
    eng.write_random_model(d, config_from_dict(TINY[name]), seed=3, dtype="float32", std=0.1)
    cfg, w = P.read_config(d), P.read_weights(d, torch.float64)
    return name, str(d), cfg, w


def prompts_for(name, vocab):
    lengths = [5, 11, 17] if name == "A" else [1, 9, 23, 40]
    rng = np.random.default_rng(7)
    return [[int(t) for t in rng.integers(0, vocab, n)] for n in lengths]


def test_greedy_generation_matches_plain(tiny, eng):
    """The configurations' own workloads: A decodes 8 tokens per prompt with pages of 4; B 12 tokens with
    prompts cut into portions of 7 and pages of 8."""
    name, d, cfg, w = tiny
    prompts = prompts_for(name, cfg["vocab_size"])
    n_new = 8 if name == "A" else 12
    want = [P.greedy_generate(w, cfg, p, n_new) for p in prompts]
    kw = dict(block_size=4, max_len=64) if name == "A" else dict(block_size=8, max_len=64, max_prefill_chunk=7)
    llm = eng.LLM(d, dtype="float32", **kw)
    got = llm.generate(prompts, eng.SamplingParams(max_new_tokens=n_new))
    assert [o.token_ids for o in got] == want
    assert all(o.finish_reason == "length" for o in got)
    llm.engine.runner.manager.check_invariants()
    assert all(g.allocator.num_in_use() == 0 for g in llm.engine.runner.manager.groups)
    # one prompt alone through generate(), with the reference's option names
    r = eng.generate(llm.model, prompts[1], max_new_tokens=n_new)
    assert r.token_ids == want[1] and r.finish_reason == "length" and r.prompt_len == len(prompts[1])
    assert len(r.step_times) == n_new - 1 and r.cache_bytes > 0


def test_run_summary_of_continuous_batching(tiny, eng):
    """Requests of very different lengths: no decode row is computed for nothing (tests/test_batching.py:108-113
    of the reference); a launch of several steps that runs past a short request's end does waste rows."""
    import time

    from llm_infrence_engine_amd.engine import summarize

    name, d, cfg, w = tiny
    model = eng.load_model(d, "float32", "cuda:0")
    prompts = prompts_for(name, cfg["vocab_size"])
    lens = [3, 12, 5, 8][:len(prompts)]
    for per_launch in (1, 4):
        e = eng.Engine(model, block_size=8, max_len=64, max_seqs=4, hip_graphs=per_launch > 1,
                       decode_steps_per_launch=per_launch)
        reqs = [eng.Request(p, max_new_tokens=n) for p, n in zip(prompts, lens)]
        t0 = time.perf_counter()
        for r in reqs:
            e.add_request(r)
        e.run_until_idle()
        s = summarize(reqs, e.steps, time.perf_counter() - t0)
        assert s["requests"] == len(reqs) and s["output_tokens"] == sum(lens)
        assert s["wasted_row_fraction"] == 0.0        # launches of several steps never run past a request's budget
        assert 0 < s["ttft_p50_s"] <= s["ttft_p95_s"] <= s["e2e_p95_s"]
        assert s["throughput_tok_s"] > 0 and 1.0 <= s["mean_decode_batch"] <= len(reqs)


def test_stop_id_is_not_emitted(tiny, eng):
    name, d, cfg, w = tiny
    p = prompts_for(name, cfg["vocab_size"])[1]
    full = P.greedy_generate(w, cfg, p, 8)
    stop = full[3]
    model = eng.load_model(d, "float32")
    r = eng.generate(model, p, max_new_tokens=8, eos_ids=[stop])
    assert r.finish_reason == "stop" and r.token_ids == full[:full.index(stop)]


def test_preemption_under_page_pressure_keeps_outputs(tiny, eng):
    """A pool too small for everybody: requests are preempted and recomputed, outputs do not change, and
    every page comes back (the reference's tests/test_paged.py:247-259)."""
    name, d, cfg, w = tiny
    rng = np.random.default_rng(11)
    prompts = [[int(t) for t in rng.integers(0, cfg["vocab_size"], n)] for n in (9, 14, 6, 11, 8)]
    want = [P.greedy_generate(w, cfg, p, 10) for p in prompts]
    model = eng.load_model(d, "float32")
    e = eng.Engine(model, num_blocks=15, block_size=4, max_seqs=4, max_len=32, max_num_batched_tokens=12)
    reqs = [e.add_request(eng.Request(p, max_new_tokens=10)) for p in prompts]
    while e.has_work():
        e.step()
        e.runner.manager.check_invariants()
    assert e.preemptions > 0
    assert [r.output_ids for r in reqs] == want
    assert all(g.allocator.num_in_use() == 0 for g in e.runner.manager.groups)
    assert e.stats()["preemptions"] == e.preemptions


def test_mid_flight_join_and_cancel(tiny, eng):
    name, d, cfg, w = tiny
    ps = prompts_for(name, cfg["vocab_size"])
    want = [P.greedy_generate(w, cfg, p, 6) for p in ps[:2]]
    model = eng.load_model(d, "float32")
    e = eng.Engine(model, block_size=4, max_seqs=3, max_len=64)
    a = e.add_request(eng.Request(ps[0], max_new_tokens=6))
    e.step(); e.step()
    b = e.add_request(eng.Request(ps[1], max_new_tokens=6))   # joins while a is decoding
    c = e.add_request(eng.Request(ps[2], max_new_tokens=40))
    e.step()
    e.cancel(c)
    e.run_until_idle()
    assert a.output_ids == want[0] and b.output_ids == want[1]
    assert c.finish_reason == "abort" and c not in e.finished
    assert a.arrival_time <= a.admitted_time <= a.first_token_time <= a.finish_time
    assert all(g.allocator.num_in_use() == 0 for g in e.runner.manager.groups)


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_random_arrivals_cancels_and_scarce_pages_keep_outputs(tiny, eng, seed):
    """Requests of random lengths that arrive at random steps, some cancelled on the way, under a random token
    budget and a pool that cannot hold them all: whatever the scheduler does (portions, preemption, recomputation,
    pages used again), every request that finishes has the plain implementation's tokens, the cache manager's
    books balance after every step, and every page and slot comes back."""
    name, d, cfg, w = tiny
    rng = np.random.default_rng(100 + seed)
    n = 9
    prompts = [[int(t) for t in rng.integers(0, cfg["vocab_size"], int(rng.integers(1, 30)))] for _ in range(n)]
    new = [int(rng.integers(1, 14)) for _ in range(n)]
    arrive = sorted(int(rng.integers(0, 25)) for _ in range(n))
    cancel_at = {int(i): int(rng.integers(2, 30)) for i in rng.choice(n, 2, replace=False)}
    model = eng.load_model(d, "float32")
    block = int(rng.choice([2, 4, 8]))
    longest = max(len(p) + k for p, k in zip(prompts, new))
    pages_of_longest = -(-longest // block) + 1
    e = eng.Engine(model, num_blocks=pages_of_longest + int(rng.integers(1, 2 * pages_of_longest)), block_size=block,
                   max_seqs=int(rng.integers(2, 5)), max_len=64, max_num_batched_tokens=int(rng.integers(6, 40)))
    reqs, step = {}, 0
    while step < 400 and (len(reqs) < n or e.has_work()):
        for i in range(n):
            if i not in reqs and arrive[i] <= step:
                reqs[i] = e.add_request(eng.Request(prompts[i], max_new_tokens=new[i]))
        for i, at in cancel_at.items():
            if at == step and i in reqs:
                e.cancel(reqs[i])
        if e.has_work():
            e.step()
            e.runner.manager.check_invariants()
        step += 1
    assert len(reqs) == n and not e.has_work()
    for i, r in reqs.items():
        want = P.greedy_generate(w, cfg, prompts[i], new[i])
        if r.finish_reason == "abort":
            assert r.output_ids == want[:len(r.output_ids)]      # what it got before the cancel was right
        else:
            assert r.finish_reason == "length" and r.output_ids == want, (seed, i)
    assert sum(r.finish_reason != "abort" for r in reqs.values()) >= n - 2
    assert all(g.allocator.num_in_use() == 0 for g in e.runner.manager.groups)


def test_long_decoding_and_first_tokens(tiny, eng):
    """Decode 150 tokens one by one from a 3-token prompt in bfloat16 and float32: the first tokens of a
    sequence and positions far past several pages, checked against the plain logits along the way."""
    from llm_infrence_engine_amd.engine import StepEntry, load_runner

    name, d, cfg, w = tiny
    rng = np.random.default_rng(5)
    toks = [int(t) for t in rng.integers(0, cfg["vocab_size"], 153)]
    exact = P.forward(w, cfg, toks).numpy()
    noise = np.abs(P.forward(w, cfg, toks, act_dtype=torch.bfloat16).numpy() - exact).max()
    for dtype, bound in (("float32", 1e-3), ("bfloat16", 3.0 * noise)):
        r = load_runner(d, dtype=dtype, page_size=8, num_pages=24, max_requests=2, max_len=160)
        first = r.step([StepEntry("x", toks[:3], [0, 1, 2])]).cpu().numpy()
        assert np.abs(first - exact[:3]).max() < bound
        for p in range(3, len(toks)):
            row = r.step([StepEntry("x", [toks[p]], [0])]).cpu().numpy()[0]
            assert np.abs(row - exact[p]).max() < bound, f"{dtype} position {p}"


def test_sampling_through_the_engine(tiny, eng):
    name, d, cfg, w = tiny
    p = prompts_for(name, cfg["vocab_size"])[1]
    llm = eng.LLM(d, dtype="float32", block_size=4, max_len=64)
    sp = eng.SamplingParams(max_new_tokens=12, temperature=1.0, seed=42)
    a = llm.generate([p, p], [sp, sp])
    assert a[0].token_ids == a[1].token_ids                      # same seed, same tokens
    b = llm.generate([p], eng.SamplingParams(max_new_tokens=12, temperature=1.0, seed=43))
    assert b[0].token_ids != a[0].token_ids
    greedy = P.greedy_generate(w, cfg, p, 12)
    k1 = llm.generate([p], eng.SamplingParams(max_new_tokens=12, temperature=1.5, top_k=1, seed=1))
    assert k1[0].token_ids == greedy                             # top_k = 1 is greedy
    tiny_p = llm.generate([p], eng.SamplingParams(max_new_tokens=12, temperature=1.0, top_p=1e-6, seed=1))
    assert tiny_p[0].token_ids == greedy                         # the most likely token always stays


def test_rejects_impossible_requests(tiny, eng):
    name, d, cfg, w = tiny
    model = eng.load_model(d, "float32")
    e = eng.Engine(model, num_blocks=4, block_size=4, max_seqs=2, max_len=64)
    with pytest.raises(ValueError, match="empty"):
        e.add_request(eng.Request([]))
    with pytest.raises(ValueError, match="max_len"):
        e.add_request(eng.Request([1] * 60, max_new_tokens=10))
    with pytest.raises(ValueError, match="never fit"):
        e.add_request(eng.Request([1] * 10, max_new_tokens=10))
    with pytest.raises(ValueError, match="vocabulary"):
        e.add_request(eng.Request([cfg["vocab_size"]], max_new_tokens=1))


def test_command_line(tiny, tmp_path):
    name, d, cfg, w = tiny
    p = prompts_for(name, cfg["vocab_size"])[0]
    want = P.greedy_generate(w, cfg, p, 5)
    r = subprocess.run([sys.executable, "-m", "llm_infrence_engine_amd", "--model", d, "--dtype", "float32",
                        "--prompt-ids", ",".join(map(str, p)), "--max-new-tokens", "5", "--max-len", "64"],
                       capture_output=True, text=True, cwd=str(ROOT), timeout=300)
    assert r.returncode == 0, r.stderr
    assert json.loads(r.stdout.strip().splitlines()[-1])["token_ids"] == want


def test_engine_refuses_the_cpu(tiny, eng):
    name, d, cfg, w = tiny
    with pytest.raises(RuntimeError, match="no CPU path"):
        eng.load_model(d, "float32", device="cpu")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_hip_graph_decode_equals_eager(tiny, eng, dtype):
    """Decode steps replayed from captured graphs, with eager prompt portions, joins and finishes between the
    replays: every replay's logits equal the eager step's, and so do the generated tokens."""
    from llm_infrence_engine_amd.engine import StepEntry, load_runner

    name, d, cfg, w = tiny
    rng = np.random.default_rng(21)
    seqs = {i: [int(t) for t in rng.integers(0, cfg["vocab_size"], n)] for i, n in enumerate((40, 29, 37))}
    runs = {}
    for graphs in (False, True):
        # decode steps only: a portion replayed from its bucket's graph runs products of other row counts
        r = load_runner(d, dtype=dtype, page_size=16, num_pages=12, max_requests=4, max_len=64, hip_graphs=graphs,
                        graph_portion_tokens=0)
        out = []
        out.append(r.step([StepEntry(0, seqs[0][:20], [19])]).cpu())                       # eager: a prompt
        for p in range(20, 26):
            out.append(r.step([StepEntry(0, [seqs[0][p]], [0])]).cpu())                      # bucket of 1
        out.append(r.step([StepEntry(1, seqs[1][:17], [16]), StepEntry(0, [seqs[0][26]], [0])]).cpu())   # eager: mixed
        for p in range(6):
            out.append(r.step([StepEntry(0, [seqs[0][27 + p]], [0]), StepEntry(1, [seqs[1][17 + p]], [0])]).cpu())
        out.append(r.step([StepEntry(2, seqs[2][:30], [29])]).cpu())
        for p in range(4):                                                                   # bucket of 4, one row padding
            out.append(r.step([StepEntry(2, [seqs[2][30 + p]], [0]), StepEntry(0, [seqs[0][33 + p]], [0]),
                               StepEntry(1, [seqs[1][23 + p]], [0])]).cpu())
            if graphs:
                assert r.greedy_tokens.tolist() == out[-1].argmax(-1).tolist()
        r.free_request(1)
        for p in range(3):                                                                   # back to a bucket of 2
            out.append(r.step([StepEntry(2, [seqs[2][34 + p]], [0]), StepEntry(0, [seqs[0][37 + p]], [0])]).cpu())
        runs[graphs] = out
        if graphs:
            assert sorted(r.graphs.buckets) == [(1, False, 1), (2, False, 1), (4, False, 1)]
    for a, b in zip(runs[False], runs[True]):
        assert torch.equal(a, b)
    exact = P.forward(w, cfg, seqs[2]).numpy()
    noise = np.abs(P.forward(w, cfg, seqs[2], act_dtype=torch.bfloat16).numpy() - exact).max()
    assert np.abs(runs[True][-1][0].numpy() - exact[36]).max() < (1e-3 if dtype == "float32" else 3.0 * noise)


def test_generation_with_hip_graphs(tiny, eng):
    name, d, cfg, w = tiny
    prompts = prompts_for(name, cfg["vocab_size"])
    want = [P.greedy_generate(w, cfg, p, 10) for p in prompts]
    llm = eng.LLM(d, dtype="float32", block_size=16, max_len=64, max_seqs=4, hip_graphs=True)
    got = llm.generate(prompts, eng.SamplingParams(max_new_tokens=10))
    assert [o.token_ids for o in got] == want
    assert llm.engine.runner.graphs.buckets


def test_graph_capture_while_an_old_engine_waits_for_the_collector(tiny, eng):
    """An engine with graphs of its own that went out of use inside a reference cycle is finalised before the
    next capture starts, never during it (the collector is kept off while the stream captures)."""
    import gc

    name, d, cfg, w = tiny
    prompts = prompts_for(name, cfg["vocab_size"])
    want = eng.LLM(d, dtype="float32", block_size=8, max_len=64).generate(prompts, eng.SamplingParams(max_new_tokens=6))
    old = gc.get_threshold()
    try:
        for _ in range(2):
            llm = eng.LLM(d, dtype="float32", block_size=8, max_len=64, hip_graphs=True)
            got = llm.generate(prompts, eng.SamplingParams(max_new_tokens=6))
            assert [o.token_ids for o in got] == [o.token_ids for o in want]
            llm.cycle = llm            # only the collector can free it and its graphs now
            del llm, got
            gc.set_threshold(50, 2, 2)   # the collector runs often from here on, the oldest generation too
    finally:
        gc.set_threshold(*old)
        gc.collect()


def test_long_context_decode_splits_keys_and_matches_plain(eng, tmp_path):
    """Past 2,048 keys a small decode batch spreads each request's keys over several blocks (and, with graphs,
    switches to the long-context graphs): logits still follow the plain implementation."""
    from llm_infrence_engine_amd.config import config_from_dict
    from llm_infrence_engine_amd.engine import StepEntry, load_runner
    from llm_infrence_engine_amd.kernels import ops

    d = tmp_path / "m"
    eng.write_random_model(d, config_from_dict(TINY["D"]), seed=5, dtype="bfloat16", std=0.08)
    cfg, w = P.read_config(d), P.read_weights(d, torch.float64)
    rng = np.random.default_rng(4)
    n = ops.LONG_CONTEXT + 40
    seqs = {r: [int(t) for t in rng.integers(0, cfg["vocab_size"], m)] for r, m in (("a", n), ("b", 300))}
    exact = {r: P.forward(w, cfg, t).numpy() for r, t in seqs.items()}
    noise = {r: np.abs(P.forward(w, cfg, t, act_dtype=torch.bfloat16).numpy() - exact[r]).max() for r, t in seqs.items()}
    for graphs in (False, True):
        r = load_runner(d, dtype="bfloat16", page_size=16, num_pages=160, max_requests=2, max_len=n + 16, hip_graphs=graphs)
        cut = {"a": n - 60, "b": 240}
        r.step([StepEntry("a", seqs["a"][:cut["a"]], []), StepEntry("b", seqs["b"][:cut["b"]], [])])
        for i in range(60):
            lg = r.step([StepEntry(q, [seqs[q][cut[q] + i]], [0]) for q in ("a", "b")]).cpu().numpy()
            for row, q in zip(lg, ("a", "b")):
                assert np.abs(row - exact[q][cut[q] + i]).max() < 3.0 * noise[q], (graphs, q, i)
        if graphs:
            assert sorted(r.graphs.buckets) == [(2, False, 1), (2, True, 1)]   # it crossed from short to long on the way


def test_large_uneven_decode_batch_matches_plain(eng, tmp_path):
    """36 requests with contexts of 20 to 1,150 tokens decode together at the layer widths of the half-billion
    model (two layers, a vocabulary of 4,128): the products for 17 to 64 tokens, attention over many requests of
    which some pass the length from which keys are split over blocks, prompts in portions beside each other."""
    from llm_infrence_engine_amd.config import config_from_dict
    from llm_infrence_engine_amd.engine import StepEntry, load_runner

    cfg = {"architectures": ["Qwen2ForCausalLM"], "num_hidden_layers": 2, "hidden_size": 896, "num_attention_heads": 14,
           "num_key_value_heads": 2, "intermediate_size": 4864, "vocab_size": 4128, "rope_theta": 1000000.0,
           "rms_norm_eps": 1e-6, "tie_word_embeddings": True}
    d = tmp_path / "m"
    eng.write_random_model(d, config_from_dict(cfg), seed=1, dtype="bfloat16", std=0.05)
    pc, w = P.read_config(d), P.read_weights(d, torch.float64)
    rng = np.random.default_rng(1)
    R, tail = 36, 2
    seqs = {f"r{i}": [int(t) for t in rng.integers(0, 4128, n)] for i, n in enumerate(rng.integers(20, 1151, R))}
    seqs["r5"] = seqs["r5"] + seqs["r6"][:1150 - len(seqs["r5"])]   # one of them as long as it gets
    exact = {r: P.forward(w, pc, t)[-tail:].numpy() for r, t in seqs.items()}
    noise = {r: np.abs(P.forward(w, pc, t, act_dtype=torch.bfloat16)[-tail:].numpy() - exact[r]).max() for r, t in seqs.items()}
    runner = load_runner(d, dtype="bfloat16", page_size=16, max_requests=R, max_len=1168)
    done = {r: 0 for r in seqs}
    while any(done[r] < len(seqs[r]) - tail for r in seqs):     # portions of up to 500 tokens, 2,048 to a step
        entries, left = [], 2048
        for r, t in seqs.items():
            n = min(len(t) - tail - done[r], left, int(rng.integers(1, 500)))
            if n > 0:
                entries.append(StepEntry(r, t[done[r]:done[r] + n], []))
                done[r] += n
                left -= n
        runner.step(entries)
    for k in range(tail):
        lg = runner.step([StepEntry(r, [t[len(t) - tail + k]], [0]) for r, t in seqs.items()]).float().cpu().numpy()
        for row, r in zip(lg, seqs):
            assert np.abs(row - exact[r][k]).max() < 3.0 * noise[r], (r, len(seqs[r]), k)


def test_decode_batch_at_the_widths_of_the_seven_billion_model(eng, tmp_path):
    """22 requests decode together at the layer widths of Qwen2.5-7B (two layers, a vocabulary of 4,100): rows too
    long to lie in LDS whole go through it in chunks, the down projection splits its columns over blocks, head
    size 128 with seven query heads to a key/value head."""
    from llm_infrence_engine_amd.config import config_from_dict
    from llm_infrence_engine_amd.engine import StepEntry, load_runner

    cfg = {"architectures": ["Qwen2ForCausalLM"], "num_hidden_layers": 2, "hidden_size": 3584, "num_attention_heads": 28,
           "num_key_value_heads": 4, "intermediate_size": 18944, "vocab_size": 4100, "rope_theta": 1000000.0,
           "rms_norm_eps": 1e-6, "tie_word_embeddings": False}
    d = tmp_path / "m"
    eng.write_random_model(d, config_from_dict(cfg), seed=7, dtype="bfloat16", std=0.02)
    pc, w = P.read_config(d), P.read_weights(d, torch.float64)
    rng = np.random.default_rng(7)
    R, tail = 22, 2
    seqs = {f"r{i}": [int(t) for t in rng.integers(0, 4100, n)] for i, n in enumerate(rng.integers(20, 121, R))}
    exact = {r: P.forward(w, pc, t)[-tail:].numpy() for r, t in seqs.items()}
    noise = {r: np.abs(P.forward(w, pc, t, act_dtype=torch.bfloat16)[-tail:].numpy() - exact[r]).max() for r, t in seqs.items()}
    runner = load_runner(d, dtype="bfloat16", page_size=16, max_requests=R, max_len=128)
    runner.step([StepEntry(r, t[:-tail], []) for r, t in seqs.items()])
    for k in range(tail):
        lg = runner.step([StepEntry(r, [t[len(t) - tail + k]], [0]) for r, t in seqs.items()]).float().cpu().numpy()
        for row, r in zip(lg, seqs):
            assert np.abs(row - exact[r][k]).max() < 3.0 * noise[r], (r, len(seqs[r]), k)


def test_several_decode_steps_per_launch_change_nothing(tiny, eng):
    """Up to 8 decode steps queued in one graph launch (tokens fed back on the device): the same outputs as step
    by step, also when a stop id arrives in the middle of a launch, a request joins, or pages are scarce."""
    name, d, cfg, w = tiny
    rng = np.random.default_rng(31)
    prompts = [[int(t) for t in rng.integers(0, cfg["vocab_size"], n)] for n in (9, 21, 5, 14)]
    full = [P.greedy_generate(w, cfg, p, 30) for p in prompts]
    stops = [(), (full[1][11],), (), (full[3][4],)]
    want = [P.greedy_generate(w, cfg, p, 30, eos_ids=s) for p, s in zip(prompts, stops)]
    model = eng.load_model(d, "float32")
    launches = {}
    for kw in (dict(num_blocks=None), dict(num_blocks=6)):            # plenty of pages; so few that launches shrink
        e = eng.Engine(model, block_size=16, max_seqs=4, max_len=64, hip_graphs=True, decode_steps_per_launch=8, **kw)
        reqs = [e.add_request(eng.Request(p, max_new_tokens=30, eos_ids=s)) for p, s in zip(prompts[:3], stops[:3])]
        for _ in range(3):
            e.step()
        reqs.append(e.add_request(eng.Request(prompts[3], max_new_tokens=30, eos_ids=stops[3])))   # joins on the way
        while e.has_work():
            e.step()
            e.runner.manager.check_invariants()
        assert [r.output_ids for r in reqs] == want
        assert [r.finish_reason for r in reqs] == ["length", "stop", "length", "stop"]
        assert any(rec.decode_steps > 1 for rec in e.steps)
        assert all(g.allocator.num_in_use() == 0 for g in e.runner.manager.groups)
        launches[kw["num_blocks"]] = ([rec.decode_steps for rec in e.steps if rec.decode_steps], e.preemptions)
    (plenty, none_preempted), (scarce, preempted) = launches[None], launches[6]
    assert none_preempted == 0 and 8 in plenty
    # six pages for four requests of up to four pages each: somebody had to wait, shrink a launch or be preempted
    assert preempted > 0 or len(scarce) > len(plenty), (plenty, scarce, preempted)
