"""Decode and prefill throughput of the engine on one MI355X, with roofline fractions.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Default run: the layer sizes of the Qwen2.5-0.5B configuration with random weights in bfloat16, a batch
of 8 requests with 512-token prompts, K timed decode steps through the whole engine (scheduler, step
function, sampler).  One JSON line is printed: ``value`` is decoded tokens a second; ``prefill`` is one
2,048-token prompt in one step; ``roofline`` prices the decode step against HBM bandwidth (every weight it
uses once plus the cache of the live requests); ``points`` holds decode throughput at batch 1 and 64;
``launch`` says how many decode steps one graph launch holds and what it costs the host to enqueue it against
the whole launch (a step bound by launching would show the two close together).  Every graph is captured
when the engine is built, before any timer starts; ``launch.graphs_captured_while_timed`` is asserted to be 0.
``roofline.measured_peak`` is the bandwidth a plain streaming read of 2 GiB reaches on this device and
``prefill.measured_peak_tflops`` the rate of a large square bfloat16 product on its matrix cores (the reference
measures its own denominators the same way, benchmarks/diag_gpu_launch.py:29-40, benchmarks/bench_micro.py:49-51);
fractions are against the published peaks.  After the headline the default run measures the two larger shapes
the same way, all their layers with weights drawn on the GPU: ``shapes["7b"]`` (decode at batch 8 and 64, the
2,048-token prompt, a queue of 64 requests with prompts of 128 to 4,096 tokens and 256 decoded each) and
``shapes["32b"]`` (the prompt, decode at batch 1, 8 and 64 after 1,024-token prompts); ``--no-shapes`` leaves
them out.  ``--only sample`` times the sampler alone at the real vocabulary.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# MI355X published peaks
HBM_GBS = 8000.0
PEAK_TFLOPS = {"bf16": 2500.0, "fp16": 2500.0, "fp8": 5000.0, "fp32": 157.3}

PROMPT_LEN = 512
CONTEXT_LIMIT = 8192
BLOCK_SIZE = 16
PREFILL_TOKENS = 2048
LONG_PROMPT = 7600          # a further point: decoding behind prompts of this length
LONG_PREFILL = 8192         # and a prompt step of this many tokens
DECODE_STEPS_PER_LAUNCH = 8   # decode steps queued in one graph launch (a stop id is noticed that many steps late at most)
# the reference's own decode at batch 8: CUDA-graph step of 6.0 ms on an A10, context 128 (docs/RESULTS.md:38)
REFERENCE_TOKS = 8 / 6.0e-3


def decode_bytes(cfg, batch, context, bytes_per_value=2):
    """Bytes a decode step has to read: every weight it uses once (the embedding table counts once, as the
    tied head) and the keys and values of the live requests."""
    H, I, V, d = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size, cfg.head_dim
    nh, nkv, L = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.num_hidden_layers
    per_layer = (nh + 2 * nkv) * d * H + H * nh * d + 3 * H * I
    weights = (L * per_layer + V * H) * bytes_per_value + (L * ((nh + 2 * nkv) * d + 2 * H) + H) * 4
    return weights + batch * context * cfg.kv_bytes_per_token(bytes_per_value)


def prefill_flops(cfg, tokens):
    H, I, V, d = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size, cfg.head_dim
    nh, nkv, L = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.num_hidden_layers
    linear = 2 * tokens * L * ((nh + 2 * nkv) * d * H + H * nh * d + 3 * H * I) + 2 * V * H  # head: one row
    attention = L * 4 * nh * d * tokens * (tokens + 1) // 2
    return linear + attention


def run_decode(eng_mod, model, batch, steps, warmup, vocab, seed, prompt_len=PROMPT_LEN, sampling=None):
    """Prefill ``batch`` prompts, then time ``steps`` decode steps of the engine.  Returns seconds per step, the
    mean context length of the timed steps, and what a graph launch cost the host against the whole launch."""
    import numpy as np
    import torch

    rng = np.random.default_rng(seed)
    budget = max(4096, batch)
    extra = -(-batch * prompt_len // budget) + 2     # requests admitted first decode while the others prefill
    need = prompt_len + warmup + steps + extra
    pages = batch * (-(-need // BLOCK_SIZE) + 1)
    e = eng_mod.Engine(model, num_blocks=pages, block_size=BLOCK_SIZE, max_seqs=batch, max_len=CONTEXT_LIMIT,
                       max_num_batched_tokens=budget, hip_graphs=True, decode_steps_per_launch=DECODE_STEPS_PER_LAUNCH,
                       capture_at_start=False)
    # every graph this run can reach, before any timer: all requests stay alive, so the one bucket of ``batch``
    # rows, in both context classes and every launch size (an engine that serves captures all buckets itself)
    e.runner.graphs.warm_up(e.launch_sizes(), batch_sizes=[batch], portion_tokens=())
    for i in range(batch):
        e.add_request(eng_mod.Request([int(t) for t in rng.integers(0, vocab, prompt_len)],
                                      max_new_tokens=warmup + steps + extra, **dict(sampling or {}, **({"seed": i} if sampling else {}))))
    while any(r.num_tokens - r.num_computed > 1 for r in e.running) or e.waiting:
        e.step()                                   # prompts in portions under the budget; first tokens sampled
    def run(n):   # exactly n decode steps, several to a graph launch
        done, first = 0, len(e.steps)
        while done < n:
            done += e.step(max_decode_steps=n - done).decode_steps
        assert done == n and all(rec.decode_batch == batch and rec.n_prefill_tokens == 0 for rec in e.steps[first:])

    run(warmup)
    assert len(e.running) == batch and all(r.num_tokens - r.num_computed == 1 for r in e.running)
    graphs = e.runner.graphs
    held = len(graphs.buckets)      # (graphs that draw tokens are captured at their first use: the warm-up steps)
    torch.cuda.synchronize()
    q0, n0 = graphs.enqueue_seconds, graphs.launches
    t0 = time.perf_counter()
    run(steps)
    torch.cuda.synchronize()
    total = time.perf_counter() - t0
    if len(graphs.buckets) != held:
        raise AssertionError("a graph was captured inside the timed region")
    dt = total / steps
    mean_context = prompt_len + warmup + (steps + 1) / 2
    launches = graphs.launches - n0
    # the host's share: filling the static buffers and enqueuing the graph, against the whole launch
    launch = {"steps_per_launch": round(steps / launches, 2),
              "enqueue_ms": round((graphs.enqueue_seconds - q0) / launches * 1e3, 4),
              "total_ms": round(total / launches * 1e3, 4), "graphs_held": held, "graphs_captured_while_timed": 0}
    return dt, mean_context, launch


def measure_read_gbs(repeats=5):
    """GB/s of a plain streaming read of 2 GiB by a kernel that does nothing else, best of ``repeats``."""
    import torch

    from llm_infrence_engine_amd.kernels import ops

    x = torch.ones(1 << 30, dtype=torch.bfloat16, device="cuda:0")
    best = None
    for i in range(repeats + 1):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        ops.read_probe(x)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        if i > 0:
            best = dt if best is None else min(best, dt)
    return x.numel() * 2 / best / 1e9


def measure_matrix_tflops(n=8192, repeats=5):
    """TFLOP/s of one n x n x n bfloat16 product on the matrix cores (the tiled kernel of this library and the
    library's own, whichever is faster), best of ``repeats``."""
    import torch

    from llm_infrence_engine_amd.kernels import ops

    g = torch.Generator(device="cuda:0").manual_seed(0)
    a = torch.randn(n, n, generator=g, device="cuda:0").bfloat16()
    w = torch.randn(n, n, generator=g, device="cuda:0").bfloat16()
    best = None
    for fn in (lambda: ops.gemm_tiled(a, w), lambda: torch.mm(a, w.t())):
        for i in range(repeats + 1):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            fn()
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
            if i > 0:
                best = dt if best is None else min(best, dt)
    return 2.0 * n ** 3 / best / 1e12


def run_sampler(vocab, batches=(8, 64), repeats=20):
    """Microseconds one call of the sampling kernel takes for a batch of rows at the real vocabulary: greedy, and
    temperature 0.8 with top-k 50 and top-p 0.9."""
    import torch

    from llm_infrence_engine_amd.kernels import ops

    out = {}
    g = torch.Generator(device="cuda:0").manual_seed(1)
    for b in batches:
        logits = torch.randn(b, vocab, generator=g, device="cuda:0") * 3.0
        tok = torch.empty(b, dtype=torch.int32, device="cuda:0")
        temp = torch.full((b,), 0.8, device="cuda:0")
        top_k = torch.full((b,), 50, dtype=torch.int32, device="cuda:0")
        top_p = torch.full((b,), 0.9, device="cuda:0")
        seeds = torch.arange(b, dtype=torch.int64, device="cuda:0") + 7
        draw = torch.zeros(b, dtype=torch.int32, device="cuda:0")
        for name, fn in (("greedy", lambda: ops.sample(logits, tok)),
                         ("top_k50_top_p0.9", lambda: ops.sample(logits, tok, temp, top_k, top_p, seeds, draw)),
                         ("temperature_only", lambda: ops.sample(logits, tok, temp, None, None, seeds, draw))):
            fn()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(repeats):
                fn()
            torch.cuda.synchronize()
            out[f"b{b}_{name}_us"] = round((time.perf_counter() - t0) / repeats * 1e6, 1)
    return out


def run_prefill(eng_mod, model, vocab, seed, repeats=5, tokens=PREFILL_TOKENS):
    import numpy as np
    import torch

    from llm_infrence_engine_amd.engine import ModelRunner, StepEntry

    rng = np.random.default_rng(seed)
    runner = ModelRunner(model, BLOCK_SIZE, tokens // BLOCK_SIZE + 1, 1, tokens + BLOCK_SIZE)
    best = None
    for i in range(repeats + 1):
        toks = [int(t) for t in rng.integers(0, vocab, tokens)]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        runner.step([StepEntry("p", toks, [tokens - 1])])
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        runner.free_request("p")
        if i > 0:                                   # the first run warms up
            best = dt if best is None else min(best, dt)
    return best


def run_serving(eng_mod, model, vocab, seed, n_requests=64, new_tokens=256, lo=128, hi=4096, max_seqs=64,
                budget=4096):
    """The whole engine on a queue of requests: prompts of lo..hi tokens (uniform), ``new_tokens`` decoded for
    each, admitted as pages and slots allow, prompts in portions beside the decoding of earlier requests."""
    import numpy as np
    import torch

    rng = np.random.default_rng(seed)
    lens = [int(n) for n in rng.integers(lo, hi + 1, n_requests)]
    pages = max_seqs * (-(-(hi + new_tokens) // BLOCK_SIZE) + 1)
    e = eng_mod.Engine(model, num_blocks=pages, block_size=BLOCK_SIZE, max_seqs=max_seqs, max_len=CONTEXT_LIMIT,
                       max_num_batched_tokens=budget, hip_graphs=True, decode_steps_per_launch=DECODE_STEPS_PER_LAUNCH)
    reqs = [eng_mod.Request([int(t) for t in rng.integers(0, vocab, n)], max_new_tokens=new_tokens) for n in lens]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for r in reqs:
        e.add_request(r)
    while e.has_work():
        e.step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    made = sum(len(r.output_ids) for r in reqs)
    mixed = sum(1 for rec in e.steps if rec.n_prefill_tokens and rec.decode_batch)
    s = eng_mod.engine.summarize(reqs, e.steps, dt)
    return {"seconds": round(dt, 3), "requests": n_requests, "prompt_tokens": sum(lens), "new_tokens": made,
            "new_tokens_per_s": round(made / dt, 1), "all_tokens_per_s": round((sum(lens) + made) / dt, 1),
            "launches": len(e.steps), "mixed_launches": mixed, "preemptions": e.preemptions,
            "ttft_p50_s": round(s["ttft_p50_s"], 4), "ttft_p95_s": round(s["ttft_p95_s"], 4),
            "tpot_mean_ms": round(s["tpot_mean_ms"], 3), "mean_decode_batch": round(s["mean_decode_batch"], 1),
            "wasted_row_fraction": round(s["wasted_row_fraction"], 4)}


def main() -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--shape", choices=["0.5b", "7b", "32b"], default="0.5b",
                    help="layer sizes: the default is the configuration the headline numbers are quoted on")
    ap.add_argument("--layers", type=int, default=None,
                    help="fewer layers than the configuration has, if memory or time needs it (both numbers are reported)")
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 and 64 decode points and the prefill")
    ap.add_argument("--prompt-len", type=int, default=PROMPT_LEN, help="prompt length of the decode run (default 512)")
    ap.add_argument("--no-shapes", action="store_true", help="skip the 7B and 32B shapes that follow the headline")
    ap.add_argument("--only", choices=["prefill", "serve", "sample"],
                    help="run one part alone: the 2,048-token prefill (for profiles), a queue of 64 requests with "
                         "prompts of 128 to 4,096 tokens and 256 decoded tokens each through the scheduler, or the "
                         "sampling kernel at the real vocabulary")
    a = ap.parse_args()
    if a.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print(f"bench.py measures one GPU; --gpus {a.gpus} is not supported by this single-GPU engine")
        return 2

    import torch

    import llm_infrence_engine_amd as eng
    from llm_infrence_engine_amd.config import config_from_dict, preset

    shape = preset(a.shape)
    if a.layers is None:
        a.layers = shape["num_hidden_layers"]
    d = dict(shape)
    d["num_hidden_layers"] = a.layers
    cfg = config_from_dict(d)
    model = eng.load_random_model(cfg, seed=0, dtype="bfloat16", device="cuda:0")   # drawn on the GPU: no file
    vocab = cfg.vocab_size
    if a.only == "prefill":
        pt = run_prefill(eng, model, vocab, seed=2, repeats=3)
        print(json.dumps({"prefill": {"value": round(PREFILL_TOKENS / pt, 1), "tokens": PREFILL_TOKENS,
                                      "ms": round(pt * 1e3, 3)}}), flush=True)
        return 0

    if a.only == "serve":
        run_serving(eng, model, vocab, seed=4, n_requests=8, new_tokens=16)       # warms up graphs and the library
        print(json.dumps({"serving": run_serving(eng, model, vocab, seed=5)}), flush=True)
        return 0

    if a.only == "sample":
        print(json.dumps({"sampler": run_sampler(vocab)}), flush=True)
        return 0

    dt, ctx, launch = run_decode(eng, model, a.batch, a.steps, a.warmup, vocab, seed=1, prompt_len=a.prompt_len)
    value = a.batch / dt
    gbs = decode_bytes(cfg, a.batch, ctx) / dt / 1e9
    measured = measure_read_gbs()
    out = {
        "metric": "decode_tokens_per_s", "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1,
        "steps": a.steps, "warmup": a.warmup, "ms_per_step": round(dt * 1e3, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": round(value / REFERENCE_TOKS, 2) if a.shape == "0.5b" else None,
        "dtype": "bf16", "data": "synthetic",
        "config": {
            "model": f"Qwen2.5-{a.shape.upper()} shape, random weights", "layers": a.layers,
            "layers_of_config": shape["num_hidden_layers"],
            "hidden": cfg.hidden_size, "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads,
            "head_dim": cfg.head_dim, "intermediate": cfg.intermediate_size, "vocab": vocab, "tied": cfg.tie_word_embeddings,
            "global_batch": a.batch, "prompt_len": a.prompt_len, "seq_len": CONTEXT_LIMIT, "block_size": BLOCK_SIZE,
            "prefill_tokens": PREFILL_TOKENS, "parallelism": "single_gpu",
            "decode_steps_per_launch": DECODE_STEPS_PER_LAUNCH,
            "baseline": "reference CUDA-graph decode, batch 8, ctx 128, A10 bf16: 6.0 ms/step",
        },
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_GBS, 4), "measured_peak": round(measured, 1),
                     "frac_of_measured": round(gbs / measured, 4)},
        "launch": launch,
    }
    if not a.no_points:
        out["prefill"] = prefill_point(eng, model, cfg, vocab)
        out["prefill"]["measured_peak_tflops"] = round(measure_matrix_tflops(), 1)
        out["points"] = {}
        for b in (1, 64):
            out["points"].update(decode_point(eng, model, cfg, b, min(a.steps, 128), min(a.warmup, 8), vocab, a.prompt_len))
        # the same batch as the headline with every request drawing its tokens (temperature 0.8, top-k 50, top-p 0.9)
        dts, _, _ = run_decode(eng, model, a.batch, min(a.steps, 128), 16, vocab, seed=9, prompt_len=a.prompt_len,
                               sampling=dict(temperature=0.8, top_k=50, top_p=0.9))
        out["points"][f"decode_b{a.batch}_sampled"] = round(a.batch / dts, 1)
        if a.shape == "0.5b":       # a long context: decoding behind 7,600-token prompts, and a prompt of 8,192 tokens
            dtl, ctxl, _ = run_decode(eng, model, a.batch, 64, 8, vocab, seed=11, prompt_len=LONG_PROMPT)
            out["points"].update({f"decode_b{a.batch}_ctx{LONG_PROMPT}_ms_per_step": round(dtl * 1e3, 4),
                                  f"decode_b{a.batch}_ctx{LONG_PROMPT}_frac":
                                      round(decode_bytes(cfg, a.batch, ctxl) / dtl / 1e9 / HBM_GBS, 4)})
            ptl = run_prefill(eng, model, vocab, seed=12, repeats=3, tokens=LONG_PREFILL)
            out["points"].update({f"prefill_{LONG_PREFILL}_ms": round(ptl * 1e3, 3),
                                  f"prefill_{LONG_PREFILL}_frac":
                                      round(prefill_flops(cfg, LONG_PREFILL) / ptl / 1e12 / PEAK_TFLOPS["bf16"], 4)})
        out["sampler"] = run_sampler(vocab)
    if a.shape == "0.5b" and not a.no_points and not a.no_shapes and a.layers == shape["num_hidden_layers"]:
        del model
        out["shapes"] = {}
        for name, prompt_len, batches, serve in (("7b", PROMPT_LEN, (8, 64), True), ("32b", 1024, (1, 8, 64), False)):
            out["shapes"][name] = measure_shape(eng, name, prompt_len, batches, serve)
    print(json.dumps(out), flush=True)
    return 0


def prefill_point(eng, model, cfg, vocab):
    pt = run_prefill(eng, model, vocab, seed=2)
    tf = prefill_flops(cfg, PREFILL_TOKENS) / pt / 1e12
    return {"value": round(PREFILL_TOKENS / pt, 1), "tokens": PREFILL_TOKENS, "ms": round(pt * 1e3, 3),
            "frac": round(tf / PEAK_TFLOPS["bf16"], 4)}


def decode_point(eng, model, cfg, batch, steps, warmup, vocab, prompt_len):
    """decode_b<batch>: tokens a second, with the step's time and its fraction of the published HBM bandwidth."""
    dt, ctx, _ = run_decode(eng, model, batch, steps, warmup, vocab, seed=3 + batch, prompt_len=prompt_len)
    gbs = decode_bytes(cfg, batch, ctx) / dt / 1e9
    return {f"decode_b{batch}": round(batch / dt, 1), f"decode_b{batch}_ms_per_step": round(dt * 1e3, 4),
            f"decode_b{batch}_frac": round(gbs / HBM_GBS, 4)}


def measure_shape(eng, name, prompt_len, batches, serve):
    """Another shape measured as the headline is: all its layers, weights drawn on the GPU."""
    import gc

    import torch

    from llm_infrence_engine_amd.config import config_from_dict, preset

    gc.collect()
    torch.cuda.empty_cache()
    cfg = config_from_dict(preset(name))
    t0 = time.perf_counter()
    model = eng.load_random_model(cfg, seed=0, dtype="bfloat16", device="cuda:0")
    torch.cuda.synchronize()
    out = {"layers": cfg.num_hidden_layers, "hidden": cfg.hidden_size, "prompt_len": prompt_len,
           "load_s": round(time.perf_counter() - t0, 1), "roofline_bound": "hbm", "roofline_peak_gbs": HBM_GBS}
    out["prefill"] = prefill_point(eng, model, cfg, cfg.vocab_size)
    for b in batches:
        out.update(decode_point(eng, model, cfg, b, 64, 8, cfg.vocab_size, prompt_len))
    if serve:
        run_serving(eng, model, cfg.vocab_size, seed=4, n_requests=8, new_tokens=16)       # warms up graphs and the library
        sv = run_serving(eng, model, cfg.vocab_size, seed=5)
        out["serve_64_mixed"] = {k: sv[k] for k in ("seconds", "prompt_tokens", "new_tokens", "all_tokens_per_s",
                                                    "new_tokens_per_s", "preemptions", "ttft_p50_s", "tpot_mean_ms")}
    del model
    gc.collect()
    torch.cuda.empty_cache()
    return out


if __name__ == "__main__":
    sys.exit(main())
