"""The scheduler's decisions, without a GPU: a stand-in model whose next token is a function of the whole
prefix, so that any scheduling must give the same outputs."""
import random
import zlib

import pytest

from llm_infrence_engine_amd.cache import CacheLayout, CacheManager
from llm_infrence_engine_amd.config import EngineConfig
from llm_infrence_engine_amd.engine.request import Request
from llm_infrence_engine_amd.engine.scheduler import Scheduler
from llm_infrence_engine_amd.parts.base import KVNeed

VOCAB = 97


def next_token(prefix):
    return zlib.crc32(bytes(str(list(prefix)), "ascii")) % VOCAB


def alone(prompt, n, eos=()):
    out, toks = [], list(prompt)
    for _ in range(n):
        t = next_token(toks)
        if t in eos:
            break
        out.append(t); toks.append(t)
    return out


def make(num_pages=64, page_size=4, max_seqs=4, max_len=64, budget=32, chunk=None, window=None):
    layout = CacheLayout([(KVNeed(2, 16, None), None, None), (KVNeed(2, 16, window), None, None)])
    m = CacheManager(layout, page_size, num_pages, max_seqs, max_len)
    cfg = EngineConfig(block_size=page_size, num_blocks=num_pages, max_seqs=max_seqs, max_len=max_len,
                       max_num_batched_tokens=budget, max_prefill_chunk=chunk)
    return Scheduler(m, cfg, clock=lambda: 0.0), m


def one_step(s, m):
    sched = s.schedule()
    seen = set()
    for e in sched:
        assert e.request.id not in seen, "a request twice in one step"
        seen.add(e.request.id)
        assert e.start == m.computed(e.request.id) == e.request.num_computed
        assert e.sample == (e.start + e.count == e.request.num_tokens)
        m.advance(e.request.id, e.start + e.count)
    s.commit(sched, [next_token(e.request.tokens[:e.start + e.count]) for e in sched if e.sample])
    m.check_invariants()
    return sched


def drain(s, m, limit=10000):
    steps = []
    while s.has_work():
        steps.append(one_step(s, m))
        assert len(steps) < limit, "no end"
    return steps


def prompts(seed, lengths):
    rng = random.Random(seed)
    return [[rng.randrange(VOCAB) for _ in range(n)] for n in lengths]


def test_outputs_do_not_depend_on_budget_portions_or_pool():
    ps = prompts(0, [5, 11, 17, 1, 23, 9])
    want = [alone(p, 12) for p in ps]
    for kw in (dict(), dict(budget=7), dict(budget=9, chunk=4), dict(num_pages=12, budget=10), dict(max_seqs=1),
               dict(num_pages=11, page_size=4, budget=5, chunk=3, window=6)):
        s, m = make(**kw)
        reqs = [s.add_request(Request(p, max_new_tokens=12)) for p in ps]
        drain(s, m)
        assert [r.output_ids for r in reqs] == want, kw
        assert all(r.finish_reason == "length" for r in reqs) and s.finished == sorted(s.finished, key=lambda r: r.finish_time)
        assert all(g.allocator.num_in_use() == 0 for g in m.groups) and m.free_rows() == m.max_requests


def test_budget_and_portion_limit_hold_and_decodes_go_first():
    s, m = make(budget=10, chunk=6, max_seqs=4)
    a = s.add_request(Request(prompts(1, [3])[0], max_new_tokens=8))
    one_step(s, m)                       # a's whole prompt; it now decodes
    b = s.add_request(Request(prompts(2, [20])[0], max_new_tokens=4))
    c = s.add_request(Request(prompts(3, [9])[0], max_new_tokens=4))
    for _ in range(6):
        sched = one_step(s, m)
        assert sum(e.count for e in sched) <= 10
        assert all(e.count <= 6 for e in sched)
        if a.state == "running" or a in [e.request for e in sched]:
            assert sched[0].request is a and sched[0].count == 1      # the decoding request is placed first
    # b was cut: 6 + 6 + 6 + 2; c had to share the budget with it
    assert b.output_ids and c.output_ids


def test_first_come_first_served_without_skipping():
    s, m = make(num_pages=8, page_size=4, budget=64, max_len=32)
    big = s.add_request(Request(prompts(4, [20])[0], max_new_tokens=4))
    big2 = s.add_request(Request(prompts(5, [20])[0], max_new_tokens=4))
    small = s.add_request(Request(prompts(6, [2])[0], max_new_tokens=2))
    sched = one_step(s, m)
    # big takes 5 of 8 pages; big2 needs 5 (+1 spare for the running one) and must wait; small fits but may not overtake
    assert [e.request for e in sched] == [big] and list(s.waiting) == [big2, small]
    drain(s, m)
    assert big.admit_seq < big2.admit_seq < small.admit_seq


def test_spare_page_per_running_request_at_admission():
    s, m = make(num_pages=6, page_size=4, budget=64, max_len=24)
    a = s.add_request(Request(prompts(7, [8])[0], max_new_tokens=8))
    b = s.add_request(Request(prompts(8, [13])[0], max_new_tokens=4))
    sched = one_step(s, m)
    # a holds 2 pages, 4 are free; b's prompt needs 4 but one must stay spare for a
    assert [e.request for e in sched] == [a] and b.state == "waiting"


def test_youngest_is_preempted_when_a_decode_finds_no_page():
    s, m = make(num_pages=4, page_size=4, budget=64, max_len=16, max_seqs=3)
    old = s.add_request(Request(prompts(9, [7])[0], max_new_tokens=9))
    one_step(s, m)
    young = s.add_request(Request(prompts(10, [4])[0], max_new_tokens=9))
    want_old, want_young = alone(old.prompt_ids, 9), alone(young.prompt_ids, 9)
    steps = []
    while s.has_work():
        before = s.preemptions
        sched = one_step(s, m)
        steps.append(sched)
        if s.preemptions > before:
            # the victim is the youngest, it lost everything, and it waits at the front of the queue
            assert young.preemptions >= 1 and old.preemptions == 0
    assert s.preemptions > 0 and young.preemptions > 0
    assert old.output_ids == want_old and young.output_ids == want_young
    # after its preemption the victim was recomputed from prompt + output so far in one piece
    recompute = [e for sched in steps for e in sched if e.request is young and e.start == 0 and e.count > 4]
    assert recompute and all(e.sample for e in recompute)


def test_requests_stuck_in_their_prompts_do_not_deadlock():
    # two prompts admitted on their first portions; together they can never hold their whole prompts
    s, m = make(num_pages=6, page_size=4, budget=8, chunk=4, max_len=24, max_seqs=2)
    a = s.add_request(Request(prompts(11, [18])[0], max_new_tokens=2))
    b = s.add_request(Request(prompts(12, [18])[0], max_new_tokens=2))
    drain(s, m, limit=200)
    assert a.output_ids == alone(a.prompt_ids, 2) and b.output_ids == alone(b.prompt_ids, 2)
    assert s.preemptions > 0


def test_stop_id_length_and_cancel():
    p = prompts(13, [6])[0]
    full = alone(p, 8)
    s, m = make()
    r = s.add_request(Request(p, max_new_tokens=8, eos_ids=(full[3],)))
    drain(s, m)
    assert r.finish_reason == "stop" and r.output_ids == full[:full.index(full[3])]
    s, m = make()
    a = s.add_request(Request(p, max_new_tokens=30))
    b = s.add_request(Request(p, max_new_tokens=3))
    one_step(s, m)
    s.cancel(a)
    w = s.add_request(Request(p, max_new_tokens=3))
    s.cancel(w)                                   # cancelled while waiting: holds nothing
    drain(s, m)
    assert a.finish_reason == "abort" and w.finish_reason == "abort" and s.finished == [b]
    assert all(g.allocator.num_in_use() == 0 for g in m.groups)


def test_impossible_requests_are_refused():
    s, m = make(num_pages=4, page_size=4, max_len=64)
    with pytest.raises(ValueError, match="empty"):
        s.add_request(Request([]))
    with pytest.raises(ValueError, match="max_len"):
        s.add_request(Request([1] * 60, max_new_tokens=5))
    with pytest.raises(ValueError, match="never fit"):
        s.add_request(Request([1] * 10, max_new_tokens=7))
    for bad in (dict(max_new_tokens=0), dict(top_k=-1), dict(top_p=0.0), dict(top_p=1.5)):
        with pytest.raises(ValueError):
            Request([1], **bad)


@pytest.mark.parametrize("seed", range(5))
def test_random_arrivals_under_pressure(seed):
    rng = random.Random(seed)
    s, m = make(num_pages=rng.choice([9, 14, 30]), page_size=rng.choice([2, 4, 8]), budget=rng.choice([4, 9, 33]),
                chunk=rng.choice([None, 2, 5]), max_seqs=rng.choice([2, 4]), max_len=36, window=rng.choice([None, 7]))
    pool = m.num_pages * m.page_size
    reqs, want = [], []
    for i in range(14):
        n, k = rng.randrange(1, 16), rng.randrange(1, 12)
        if n + k > min(36, pool):
            continue
        p = [rng.randrange(VOCAB) for _ in range(n)]
        for _ in range(rng.randrange(3)):
            if s.has_work():
                one_step(s, m)
        reqs.append(s.add_request(Request(p, max_new_tokens=k)))
        want.append(alone(p, k))
    drain(s, m)
    assert [r.output_ids for r in reqs] == want
    assert all(g.allocator.num_in_use() == 0 for g in m.groups)


def test_requests_may_arrive_and_be_cancelled_from_other_threads():
    """add_request and cancel from threads of their own while this one steps (the reference's server does so,
    src/miniserve/engine.py:136-161): ids stay unique, nothing is lost, outputs are those of each request alone."""
    import threading
    import time

    s, m = make(num_pages=40, page_size=4, max_seqs=4, max_len=48, budget=16)
    ps = prompts(3, [5, 9, 2, 14, 7, 3, 11, 6] * 5)
    reqs, stop = [], threading.Event()
    lock = threading.Lock()

    def feed(mine):
        for p in mine:
            r = s.add_request(Request(p, max_new_tokens=6))
            with lock:
                reqs.append(r)

    feeders = [threading.Thread(target=feed, args=(ps[i::4],)) for i in range(4)]
    for t in feeders:
        t.start()
    steps = 0
    while any(t.is_alive() for t in feeders) or s.has_work():
        if s.has_work():
            one_step(s, m)
            steps += 1
            if steps == 3:
                while True:     # a feeder may have been interrupted between add_request and its note of it
                    with lock:
                        if reqs:
                            victim = reqs[-1]
                            break
                    time.sleep(0.001)
                threading.Thread(target=s.cancel, args=(victim,)).start()
        assert steps < 5000
    for t in feeders:
        t.join()
    assert len(reqs) == len(ps) and sorted(r.id for r in reqs) == list(range(len(ps)))
    for r in reqs:
        if r.finish_reason == "abort":
            assert r is victim
        else:
            assert r.output_ids == alone(r.prompt_ids, 6)
    assert all(g.allocator.num_in_use() == 0 for g in m.groups)


def test_a_portion_may_leave_one_prompt_token_which_then_runs_as_a_single_token_row():
    """A 5-token prompt under a budget of 4: first four tokens, then the last one alone, with its start past 0,
    one token and a sample, before the request has any output: what feeds such a row must be the prompt's
    last token."""
    s, m = make(budget=4)
    r = s.add_request(Request(prompts(3, [5])[0], max_new_tokens=3))
    first = one_step(s, m)
    assert [(e.start, e.count, e.sample) for e in first] == [(0, 4, False)]
    second = s.schedule()
    assert [(e.start, e.count, e.sample) for e in second] == [(4, 1, True)]
    assert not r.output_ids and r.tokens[second[0].start] == r.prompt_ids[-1]
    assert (r.output_ids or r.prompt_ids)[-1] == r.tokens[second[0].start]


def test_pool_size_from_a_memory_budget():
    """Without num_blocks: max_seqs requests of max_len, or what the stated share of the device's memory has
    room for beside what is held already; too little for one request is refused."""
    per_token = 24 * 2 * 2 * 64 * 2                       # the half-billion shape in bfloat16: 12,288 bytes a token
    cfg = EngineConfig(block_size=16, max_seqs=64, max_len=8192)
    assert cfg.resolved_num_blocks() == 64 * 512
    assert EngineConfig(block_size=16, num_blocks=7, max_seqs=64, max_len=8192, gpu_memory_fraction=0.5) \
        .resolved_num_blocks(per_token, 1 << 30, 0) == 7   # given by hand wins
    gib = 1 << 30
    small = EngineConfig(block_size=16, max_seqs=64, max_len=8192, gpu_memory_fraction=0.5)
    # half of 8 GiB, 1 GiB of it held by the weights: 3 GiB of pages of 16 * 12,288 bytes, one of them the null page
    assert small.resolved_num_blocks(per_token, 8 * gib, 1 * gib) == 3 * gib // (16 * per_token) - 1
    # plenty of memory: never more pages than the requests can fill
    assert small.resolved_num_blocks(per_token, 288 * gib, 1 * gib) == 64 * 512
    with pytest.raises(ValueError, match="less than one request"):
        small.resolved_num_blocks(per_token, 2 * gib, 1 * gib - 50 * 16 * per_token)
    with pytest.raises(ValueError, match="gpu_memory_fraction"):
        EngineConfig(gpu_memory_fraction=1.5)
    assert EngineConfig(dtype="bfloat16").hip_graphs is True and EngineConfig(dtype="float32").hip_graphs is False
    assert EngineConfig(dtype="float32", hip_graphs=True).hip_graphs is True


def test_batch_size_buckets_of_the_decode_graphs():
    """The reference's own vectors (tests/test_cuda_graph.py:45-48) and the edges around them."""
    from llm_infrence_engine_amd.engine.graph import default_batch_sizes

    assert default_batch_sizes(8) == [1, 2, 4, 8]
    assert default_batch_sizes(6) == [1, 2, 4, 6]
    assert default_batch_sizes(1) == [1]
    assert default_batch_sizes(2) == [1, 2]
    assert default_batch_sizes(9) == [1, 2, 4, 8, 9]
    assert default_batch_sizes(64) == [1, 2, 4, 8, 16, 32, 64]
    with pytest.raises(ValueError):
        default_batch_sizes(0)


def test_memory_beside_the_pages_is_taken_off_the_budget():
    """The pool sized from a share of the device's memory leaves room for what the engine holds beside weights and
    pages: state slots (one more than requests), block tables, the logits of the graph buckets and activations."""
    import torch

    from llm_infrence_engine_amd.config import config_from_dict, preset
    from llm_infrence_engine_amd.engine.engine import memory_beside_the_pages
    from llm_infrence_engine_amd.parts.base import Runtime, StateNeed
    from llm_infrence_engine_amd.parts.model import Model

    model = Model(config_from_dict(preset("tinyB")).to_spec())
    model.rt = Runtime(torch.device("cpu"), torch.bfloat16)
    plain = CacheLayout(model.run_needs())
    stateful = CacheLayout([(kv, (StateNeed((1000,), torch.float32), StateNeed((), torch.int32)) if i == 0 else None, c)
                            for i, (kv, _, c) in enumerate(model.run_needs())])
    cfg = EngineConfig(dtype="bfloat16", max_seqs=7, max_len=64, block_size=16, max_num_batched_tokens=128,
                       gpu_memory_fraction=0.5, hip_graphs=False)
    a, b = memory_beside_the_pages(cfg, model, plain), memory_beside_the_pages(cfg, model, stateful)
    assert b - a == 8 * (1000 * 4 + 4)                      # eight slots of 1,000 floats and an int
    tables = 1 * 8 * 4 * 4                                  # one group, eight rows of four pages
    widest = max(320 * 2, 192 * 4)                          # the widest checkpoint matrix's rows in bfloat16, or the float stream
    assert a == tables + 10 * 128 * widest
    with_graphs = EngineConfig(dtype="bfloat16", max_seqs=7, max_len=64, block_size=16, max_num_batched_tokens=128,
                               gpu_memory_fraction=0.5, hip_graphs=True)
    assert memory_beside_the_pages(with_graphs, model, plain) == tables + (1 + 2 + 4 + 7) * 384 * 4 + 10 * (128 + 7) * widest
    # and it comes off the pool
    per_token = plain.bytes_per_token(2)
    total = 1 << 24
    free_pool = cfg.resolved_num_blocks(per_token, total, 0)
    assert cfg.resolved_num_blocks(per_token, total, 0, other_bytes=b) <= free_pool
    tight = EngineConfig(dtype="bfloat16", max_seqs=64, max_len=4096, block_size=16, gpu_memory_fraction=0.5)
    most = tight.resolved_num_blocks(per_token, total, 0)
    assert tight.resolved_num_blocks(per_token, total, 0, other_bytes=1 << 20) == most - (1 << 20) // (per_token * 16)
