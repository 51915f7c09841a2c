"""The path that serving and the bench take: bfloat16, decode steps replayed from HIP graphs that were all
captured before the first request, several steps to a launch with the chosen token fed back on the device.
Compared with the plain implementation by teacher forcing: the plain logits of (prompt + the engine's own
tokens) say at every place which token a faithful computation would have chosen there."""
import numpy as np
import pytest
import torch

from tests.conftest import TINY
from tests.plain import qwen2_plain as P

pytestmark = pytest.mark.gpu

BF16_NOISE = 3.0    # as in test_replay.py: the engine may stray this many times further than a faithful bfloat16 run

HALF_B_WIDTHS = {"architectures": ["Qwen2ForCausalLM"], "num_hidden_layers": 2, "hidden_size": 896,
                 "num_attention_heads": 14, "num_key_value_heads": 2, "intermediate_size": 4864, "vocab_size": 4128,
                 "rope_theta": 1000000.0, "rms_norm_eps": 1e-6, "tie_word_embeddings": True}


@pytest.fixture(scope="module")
def eng():
    import llm_infrence_engine_amd as e

    return e


def plain_rows(w, cfg, prompt, out):
    """Exact logits at the places the engine chose ``out`` from, and the noise of a faithful bfloat16 run there."""
    seq = list(prompt) + list(out)
    first = len(prompt) - 1
    exact = P.forward(w, cfg, seq[:-1])[first:].numpy()
    noisy = P.forward(w, cfg, seq[:-1], act_dtype=torch.bfloat16)[first:].numpy()
    return exact, float(np.abs(noisy - exact).max())


def assert_tokens_follow_plain(w, cfg, prompt, out, min_agreement=0.6):
    """Every token is the plain implementation's choice for the same prefix, unless the plain logits of the two
    candidates lie closer together than reduced precision can tell apart."""
    exact, noise = plain_rows(w, cfg, prompt, out)
    assert len(exact) == len(out)
    same = 0
    for i, tok in enumerate(out):
        top = int(exact[i].argmax())
        if tok == top:
            same += 1
            continue
        gap = exact[i][top] - exact[i][tok]
        assert gap < 2 * BF16_NOISE * noise, f"token {i}: chose {tok}, plain chooses {top}, {gap:.3e} apart (noise {noise:.3e})"
    assert same >= min_agreement * len(out), f"only {same} of {len(out)} tokens are the plain implementation's"
    return exact, noise


@pytest.fixture(scope="module")
def half_b(tmp_path_factory, eng):
    from llm_infrence_engine_amd.config import config_from_dict

    d = tmp_path_factory.mktemp("halfb_serving")
    eng.write_random_model(d, config_from_dict(HALF_B_WIDTHS), seed=11, dtype="bfloat16", std=0.05)
    return str(d), P.read_config(d), P.read_weights(d, torch.float64)


def test_the_path_the_bench_times_follows_plain(half_b, eng):
    """Eight requests with contexts past 512 at the layer widths of the half-billion model: graphs, eight steps
    to a launch.  Tokens follow the plain implementation; no graph is captured while serving; and the same runner
    stepped once per launch over the same tokens gives logits within the bfloat16 bound at every place."""
    from llm_infrence_engine_amd.engine import StepEntry

    d, cfg, w = half_b
    rng = np.random.default_rng(2)
    prompts = [[int(t) for t in rng.integers(0, cfg["vocab_size"], n)] for n in (520, 531, 544, 560, 577, 590, 513, 601)]
    n_new = 21                                    # launches of 8, 8, 4 and 1 steps after the first token
    model = eng.load_model(d, "bfloat16")
    e = eng.Engine(model, block_size=16, max_seqs=8, max_len=640, max_num_batched_tokens=4096, hip_graphs=True,
                   decode_steps_per_launch=8)
    graphs = e.runner.graphs
    held = len(graphs.buckets)
    assert held == 4 * 1 * 4                      # buckets 1, 2, 4, 8; one context class; 1, 2, 4, 8 steps
    reqs = [e.add_request(eng.Request(p, max_new_tokens=n_new)) for p in prompts]
    e.run_until_idle()
    assert len(graphs.buckets) == held, "a graph was captured while serving"
    assert 8 in {rec.decode_steps for rec in e.steps}, [rec.decode_steps for rec in e.steps]
    rows = {}
    for i, (p, r) in enumerate(zip(prompts, reqs)):
        assert len(r.output_ids) == n_new
        rows[i] = assert_tokens_follow_plain(w, cfg, p, r.output_ids)
    # one step per launch on the same runner, fed the same tokens
    runner = e.runner
    runner.step([StepEntry(("again", i), p[:-1], []) for i, p in enumerate(prompts)])
    for k in range(n_new):
        toks = [(p + r.output_ids)[len(p) - 1 + k] for p, r in zip(prompts, reqs)]
        lg = runner.step([StepEntry(("again", i), [t], [0]) for i, t in enumerate(toks)]).float().cpu().numpy()
        assert runner.greedy_tokens is not None      # it was a graph replay
        for i in range(len(prompts)):
            exact, noise = rows[i]
            err = np.abs(lg[i] - exact[k]).max()
            assert err < BF16_NOISE * noise, f"request {i} step {k}: {err:.3e} >= {BF16_NOISE * noise:.3e}"
    assert len(graphs.buckets) == held


def test_a_launch_that_crosses_into_long_contexts(eng, tmp_path):
    """A launch of eight steps that starts below the length from which a decode batch splits its keys over
    blocks and ends above it takes the long-context graph for all its steps."""
    from llm_infrence_engine_amd.config import config_from_dict
    from llm_infrence_engine_amd.kernels import ops

    d = tmp_path / "m"
    eng.write_random_model(d, config_from_dict(TINY["D"]), seed=5, dtype="bfloat16", std=0.08)
    cfg, w = P.read_config(d), P.read_weights(d, torch.float64)
    rng = np.random.default_rng(8)
    prompts = [[int(t) for t in rng.integers(0, cfg["vocab_size"], n)] for n in (ops.LONG_CONTEXT - 4, 300)]
    model = eng.load_model(str(d), "bfloat16")
    e = eng.Engine(model, block_size=16, max_seqs=2, max_len=ops.LONG_CONTEXT + 64, hip_graphs=True,
                   decode_steps_per_launch=8)
    held = len(e.runner.graphs.buckets)
    assert held == 2 * 2 * 4                      # buckets 1, 2; short and long contexts; 1, 2, 4, 8 steps
    reqs = [e.add_request(eng.Request(p, max_new_tokens=25)) for p in prompts]
    launches = []
    while e.has_work():
        before = max(r.num_computed for r in e.running) if e.running else 0
        rec = e.step()
        launches.append((before, rec.decode_steps))
    assert any(b < ops.LONG_CONTEXT < b + k and k == 8 for b, k in launches), launches
    assert len(e.runner.graphs.buckets) == held
    for p, r in zip(prompts, reqs):
        assert_tokens_follow_plain(w, cfg, p, r.output_ids)


@pytest.mark.parametrize("per_launch", [1, 8])
def test_a_portion_that_leaves_one_prompt_token(eng, tmp_path, per_launch):
    """A prompt one token longer than the portion limit: its last token runs as a single-token row before any
    output exists, in a launch of several steps too."""
    from llm_infrence_engine_amd.config import config_from_dict

    d = tmp_path / "m"
    eng.write_random_model(d, config_from_dict(TINY["B"]), seed=3, dtype="float32", std=0.1)
    cfg, w = P.read_config(d), P.read_weights(d, torch.float64)
    rng = np.random.default_rng(13)
    prompts = [[int(t) for t in rng.integers(0, cfg["vocab_size"], n)] for n in (17, 9)]
    want = [P.greedy_generate(w, cfg, p, 12) for p in prompts]
    model = eng.load_model(str(d), "float32")
    e = eng.Engine(model, block_size=8, max_seqs=2, max_len=64, max_prefill_chunk=16, max_num_batched_tokens=16,
                   hip_graphs=True, decode_steps_per_launch=per_launch)
    a = e.add_request(eng.Request(prompts[0], max_new_tokens=12))
    e.step()                                          # 16 of the 17 tokens
    assert a.num_computed == 16 and not a.output_ids
    e.run_until_idle()
    b = e.add_request(eng.Request(prompts[1], max_new_tokens=12))
    e.run_until_idle()
    assert [a.output_ids, b.output_ids] == want
    if per_launch > 1:
        assert any(rec.decode_steps > 1 for rec in e.steps)


@pytest.mark.parametrize("name", ["A", "B", "D"])
def test_generation_in_bfloat16_follows_plain(eng, tmp_path, name):
    """``LLM.generate`` with its defaults in bfloat16 (graphs on): tokens follow the plain implementation."""
    from llm_infrence_engine_amd.config import config_from_dict

    d = tmp_path / "m"
    eng.write_random_model(d, config_from_dict(TINY[name]), seed=4, dtype="bfloat16", std=0.1)
    cfg, w = P.read_config(d), P.read_weights(d, torch.float64)
    rng = np.random.default_rng(5)
    prompts = [[int(t) for t in rng.integers(0, cfg["vocab_size"], n)] for n in (5, 11, 17, 40)]
    llm = eng.LLM(str(d), dtype="bfloat16", block_size=16, max_len=96, max_seqs=4, max_prefill_chunk=7)
    assert llm.engine.runner.graphs is not None and llm.engine.runner.graphs.buckets
    got = llm.generate(prompts, eng.SamplingParams(max_new_tokens=24))
    for p, o in zip(prompts, got):
        assert len(o.token_ids) == 24
        assert_tokens_follow_plain(w, cfg, p, o.token_ids)


@pytest.fixture(scope="module")
def tiny_d(tmp_path_factory, eng):
    """Configuration D (head size 64, seven query heads to a key/value head: the matrix-core kernels) in bfloat16."""
    from llm_infrence_engine_amd.config import config_from_dict

    d = tmp_path_factory.mktemp("tinyD_serving")
    eng.write_random_model(d, config_from_dict(TINY["D"]), seed=6, dtype="bfloat16", std=0.08)
    return eng.load_model(str(d), "bfloat16"), P.read_config(d), P.read_weights(d, torch.float64)


def test_sampled_tokens_do_not_depend_on_graphs(tiny_d, eng):
    """bfloat16 with temperature, top-k and top-p: the sampler reads a view of a graph's static logits when graphs
    are on.  The same seeds give the same tokens with graphs on and off; top_k = 1 is the greedy choice, which
    with graphs comes from launches of eight steps."""
    model, cfg, w = tiny_d
    rng = np.random.default_rng(17)
    prompts = [[int(t) for t in rng.integers(0, cfg["vocab_size"], n)] for n in (21, 34, 9, 50)]
    sp = [eng.SamplingParams(max_new_tokens=20, temperature=0.8, top_k=20, top_p=0.9, seed=100 + i) for i in range(4)]
    kw = dict(block_size=16, max_len=96, max_seqs=4)
    with_graphs = eng.LLM(model, hip_graphs=True, decode_steps_per_launch=8, **kw)
    without = eng.LLM(model, hip_graphs=False, **kw)
    a = with_graphs.generate(prompts, sp)
    # the draws happened on the device, eight steps to a launch, from graphs that hold the sampling kernels
    assert any(rec.decode_steps == 8 for rec in with_graphs.engine.steps)
    assert (4, False, 8, "sampled", True, True) in with_graphs.engine.runner.graphs.buckets
    b = without.generate(prompts, sp)
    assert [o.token_ids for o in a] == [o.token_ids for o in b]
    assert len({tuple(o.token_ids) for o in a}) == 4
    assert with_graphs.engine.runner.graphs.launches > 0
    other = with_graphs.generate(prompts[:1], eng.SamplingParams(max_new_tokens=20, temperature=0.8, top_k=20, top_p=0.9, seed=7))
    assert other[0].token_ids != a[0].token_ids
    t_only = eng.SamplingParams(max_new_tokens=20, temperature=0.9, seed=3)
    assert [o.token_ids for o in with_graphs.generate(prompts, t_only)] == [o.token_ids for o in without.generate(prompts, t_only)]
    assert (4, False, 8, "sampled", False, False) in with_graphs.engine.runner.graphs.buckets
    greedy = with_graphs.generate(prompts, eng.SamplingParams(max_new_tokens=20))
    assert any(rec.decode_steps == 8 for rec in with_graphs.engine.steps)
    k1 = with_graphs.generate(prompts, eng.SamplingParams(max_new_tokens=20, temperature=1.3, top_k=1, seed=5))
    assert [o.token_ids for o in k1] == [o.token_ids for o in greedy]
    for p, o in zip(prompts, greedy):
        assert_tokens_follow_plain(w, cfg, p, o.token_ids)


def test_preemption_with_graphs_and_eight_steps_to_a_launch(tiny_d, eng):
    """bfloat16, graphs, eight steps to a launch and ten pages for four requests that need five each: requests are
    preempted and their prefixes recomputed as prompt portions (other kernels than the decode steps that first
    produced them); tokens still follow the plain implementation and every page comes back."""
    model, cfg, w = tiny_d
    rng = np.random.default_rng(23)
    prompts = [[int(t) for t in rng.integers(0, cfg["vocab_size"], n)] for n in (30, 27, 31, 25, 29)]
    e = eng.Engine(model, num_blocks=10, block_size=16, max_seqs=4, max_len=80, max_num_batched_tokens=64,
                   hip_graphs=True, decode_steps_per_launch=8)
    reqs = [e.add_request(eng.Request(p, max_new_tokens=40)) for p in prompts]
    while e.has_work():
        e.step()
        e.runner.manager.check_invariants()
    assert e.preemptions > 0 and any(r.preemptions > 0 for r in reqs)
    assert any(rec.decode_steps > 1 for rec in e.steps)
    assert all(g.allocator.num_in_use() == 0 for g in e.runner.manager.groups)
    assert all(g.allocator.pages_granted_again() > 0 for g in e.runner.manager.groups)
    for p, r in zip(prompts, reqs):
        assert len(r.output_ids) == 40 and r.finish_reason == "length"
        assert_tokens_follow_plain(w, cfg, p, r.output_ids)


def test_cancel_that_arrives_inside_a_launch_of_eight_steps(tiny_d, eng):
    """``cancel`` called while a launch of eight steps is being handed out (from the token callback, as a server's
    thread would): the request keeps the tokens of that launch, is dropped before the next one, its pages come
    back, and the others' outputs are what they are without it."""
    model, cfg, w = tiny_d
    rng = np.random.default_rng(29)
    prompts = [[int(t) for t in rng.integers(0, cfg["vocab_size"], n)] for n in (18, 40, 26)]
    kw = dict(block_size=16, max_seqs=4, max_len=96, hip_graphs=True, decode_steps_per_launch=8)
    alone = eng.Engine(model, **kw)
    full = [alone.add_request(eng.Request(p, max_new_tokens=36)) for p in prompts]
    alone.run_until_idle()

    state = {}

    def on_token(req, tok):
        if req is state.get("first") and len(req.output_ids) == 12:     # the third token of the second launch
            state["engine"].cancel(state["victim"])

    e = eng.Engine(model, on_token=on_token, **kw)
    state["engine"] = e
    reqs = [e.add_request(eng.Request(p, max_new_tokens=36)) for p in prompts]
    state["first"], state["victim"] = reqs[0], reqs[1]
    before = None
    while e.has_work():
        rec = e.step()
        e.runner.manager.check_invariants()
        if reqs[1].cancelled and before is None:
            before = (rec.decode_steps, len(reqs[1].output_ids))
    assert before is not None and before[0] == 8, before
    assert reqs[1].finish_reason == "abort" and reqs[1] not in e.finished
    n = len(reqs[1].output_ids)
    assert n == before[1] and 12 <= n < 36 and reqs[1].output_ids == full[1].output_ids[:n]
    assert reqs[0].output_ids == full[0].output_ids and reqs[2].output_ids == full[2].output_ids
    assert all(g.allocator.num_in_use() == 0 for g in e.runner.manager.groups)


def test_random_weights_drawn_on_the_device(eng):
    """Seeded draws straight into the kept types: distributions per role, repeatable from the seed, different
    for another seed and from tensor to tensor."""
    from llm_infrence_engine_amd.config import config_from_dict
    from llm_infrence_engine_amd.parts.model import Model
    from llm_infrence_engine_amd.weights import RandomSource

    cfg = config_from_dict(HALF_B_WIDTHS)
    specs = Model(cfg.to_spec()).tensor_specs()
    src = RandomSource(specs, seed=3, run_dtype=torch.bfloat16, device="cuda:0", std=0.02, norm_std=0.1, piece=1 << 20)
    again = RandomSource(specs, seed=3, run_dtype=torch.bfloat16, device="cuda:0", std=0.02, norm_std=0.1, piece=1 << 20)
    other = RandomSource(specs, seed=4, run_dtype=torch.bfloat16, device="cuda:0", std=0.02, norm_std=0.1)
    seen = {}
    for s in specs:
        t = src.get(s.name)
        assert tuple(t.shape) == tuple(s.shape) and t.is_cuda
        assert torch.equal(t, again.get(s.name))
        assert not torch.equal(t, other.get(s.name))
        f = t.float()
        if s.role == "matrix":
            assert t.dtype == torch.bfloat16
            assert abs(f.mean().item()) < 4 * 0.02 / f.numel() ** 0.5 + 1e-5
            assert abs(f.std().item() / 0.02 - 1) < 0.02
        elif s.role == "bias":
            assert t.dtype == torch.float32 and abs(f.std().item() / 0.02 - 1) < 0.25 and abs(f.mean().item()) < 0.01
        elif s.role == "norm":
            assert t.dtype == torch.float32 and abs(f.mean().item() - 1) < 0.02 and abs(f.std().item() / 0.1 - 1) < 0.2
        seen.setdefault(tuple(s.shape), []).append(f)
    for same_shape in seen.values():                 # tensors of one shape are not copies of each other
        for a, b in zip(same_shape, same_shape[1:]):
            assert not torch.equal(a, b)
    m1 = eng.load_random_model(cfg, seed=9)
    m2 = eng.load_random_model(cfg, seed=9)
    assert torch.equal(m1.layers[0].mixer.w_qkv, m2.layers[0].mixer.w_qkv)
    assert m1.layers[0].mixer.w_qkv.dtype == torch.bfloat16 and m1.layers[0].mixer.b_qkv.dtype == torch.float32


WIDE = {"architectures": ["Qwen2ForCausalLM"], "num_hidden_layers": 2, "hidden_size": 1536,
        "num_attention_heads": 24, "num_key_value_heads": 12, "intermediate_size": 2304, "vocab_size": 1184,
        "rope_theta": 1000000.0, "rms_norm_eps": 1e-6, "tie_word_embeddings": False}


def test_many_rows_of_wide_layers_take_the_norm_kernel_and_follow_plain(eng, tmp_path):
    """48 decode rows of width 1,536: the products no longer fold the norm in (they read bfloat16 rows that a norm
    kernel leaves) and the q/k/v projection, rotation and cache store run as kernels of their own.  With 8 rows the
    same layers take the fused kernels.  Both follow the plain implementation."""
    from llm_infrence_engine_amd.config import config_from_dict
    from llm_infrence_engine_amd.engine import StepEntry
    from llm_infrence_engine_amd.kernels import ops

    n_rows = 48
    x = torch.empty(n_rows, WIDE["hidden_size"], device="cuda:0")
    w_qkv = torch.empty((24 + 2 * 12) * 64, WIDE["hidden_size"], dtype=torch.bfloat16, device="cuda:0")
    assert not ops.fold_norm_pays(n_rows, WIDE["hidden_size"]) and ops.fold_norm_pays(8, WIDE["hidden_size"])
    assert not ops.qkv_rope_store_pays(x, w_qkv) and ops.qkv_rope_store_pays(x[:8], w_qkv)
    d = tmp_path / "m"
    eng.write_random_model(d, config_from_dict(WIDE), seed=21, dtype="bfloat16", std=0.04)
    cfg, w = P.read_config(d), P.read_weights(d, torch.float64)
    rng = np.random.default_rng(4)
    prompts = [[int(t) for t in rng.integers(0, cfg["vocab_size"], 20 + i % 7)] for i in range(n_rows)]
    model = eng.load_model(str(d), "bfloat16")
    e = eng.Engine(model, block_size=16, max_seqs=n_rows, max_len=64, max_num_batched_tokens=2048, hip_graphs=True,
                   capture_at_start=False)
    runner = e.runner
    runner.step([StepEntry(i, p[:-1], []) for i, p in enumerate(prompts)])
    checked = 0
    for rows in (n_rows, 8):                       # all rows in a step, then the first eight alone
        lg = runner.step([StepEntry(i, [prompts[i][-1]] if rows == n_rows else [7], [0]) for i in range(rows)])
        lg = lg.float().cpu().numpy()
        for i in range(0, rows, 5):
            seq = prompts[i] + ([7] if rows == 8 else [])
            exact = P.forward(w, cfg, seq)[-1].numpy()
            noise = float(np.abs(P.forward(w, cfg, seq, act_dtype=torch.bfloat16)[-1].numpy() - exact).max())
            err = np.abs(lg[i] - exact).max()
            assert err < BF16_NOISE * noise, f"{rows} rows, request {i}: {err:.3e} >= {BF16_NOISE * noise:.3e}"
            checked += 1
    assert checked == 12
