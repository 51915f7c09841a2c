"""Trace replay: feed given token ids through the model step by step and write logits.  Nothing is sampled.

It drives the same model, step function, cache manager and kernels that generation uses.  Steps come as
one JSON object a line:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

All entries of a step are one batch.  ``end`` names requests that are finished after the step; what they
hold is given back.  For a step that wants logits, ``<out>/<step>.f32`` holds them as little-endian floats
[wanted places, vocabulary] in the order of the entries and of ``want``.  After every step a line
``done <step>`` is printed and flushed.
"""
from __future__ import annotations

import argparse
import json
import sys
from pathlib import Path

PAGE_SIZE = 16        # tokens per page
ROUND_TO = 64         # --max-tokens counts each live request rounded up to this many tokens
MAX_LIVE = 8          # request rows (the format allows up to four live requests; leave room)


def replay(model_dir, dtype: str, out_dir, max_tokens: int, lines, log=sys.stdout, page_size: int = PAGE_SIZE,
           device: str = "cuda:0"):
    """Runs the steps of ``lines`` and returns the runner they ran on (its cache manager tells how pages were used)."""
    import numpy as np

    from .batch import StepEntry
    from .runner import load_runner

    out = Path(out_dir)
    out.mkdir(parents=True, exist_ok=True)
    unit = max(ROUND_TO, page_size)
    if ROUND_TO % page_size and page_size % ROUND_TO:
        raise ValueError(f"page size {page_size} neither divides nor is a multiple of {ROUND_TO}")
    if max_tokens <= 0:
        raise ValueError("--max-tokens must be positive")
    tokens = -(-max_tokens // unit) * unit
    # bfloat16 is the serving path, and serving replays its steps from captured graphs
    runner = load_runner(model_dir, dtype=dtype, device=device, page_size=page_size, num_pages=tokens // page_size,
                         max_requests=MAX_LIVE, max_len=tokens, hip_graphs=dtype == "bfloat16")
    for line in lines:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        step = rec["step"]
        entries = [StepEntry(e["id"], [int(t) for t in e["tokens"]], [int(w) for w in e.get("want", ())])
                   for e in rec.get("entries", ())]
        if entries:
            logits = runner.step(entries)
            if logits.shape[0]:
                arr = logits.to("cpu").numpy().astype("<f4", copy=False)
                np.ascontiguousarray(arr).tofile(out / f"{step}.f32")
        for rid in rec.get("end", ()):
            if runner.manager.has(rid):
                runner.free_request(rid)
        print(f"done {step}", file=log, flush=True)
    return runner


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"],
                    help="bfloat16: the kernels and precisions that serving uses; float32: everything in true 32-bit")
    ap.add_argument("--out", required=True, help="folder for <step>.f32")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens that live requests hold at any time (each rounded up to a multiple of 64); "
                         "the cache pool is made for this many")
    ap.add_argument("--page-size", type=int, default=PAGE_SIZE, help=argparse.SUPPRESS)
    a = ap.parse_args(argv)
    replay(a.model, a.dtype, a.out, a.max_tokens, sys.stdin, page_size=a.page_size)
    return 0
