"""Trace builders for the replay tests: the same requests whole, with the last 32 tokens one by one, in
portions of changing size, and mixed with other requests in a pool so small that pages are used again.
A trace is a list of step dicts in the replay tool's format; ``collect`` maps the written files back to
(request, position) -> logits."""
import json
import random
from pathlib import Path

import numpy as np


def whole(requests):
    """Each request alone and whole, all places wanted."""
    steps = []
    for i, (rid, toks) in enumerate(requests.items()):
        steps.append({"step": i, "entries": [{"id": rid, "tokens": toks, "want": list(range(len(toks)))}], "end": [rid]})
    return steps


def bulk_then_single(requests, tail=32):
    """Most of it in one step and the last ``tail`` tokens one by one."""
    steps, s = [], 0
    for rid, toks in requests.items():
        cut = max(1, len(toks) - tail)
        steps.append({"step": s, "entries": [{"id": rid, "tokens": toks[:cut], "want": list(range(cut))}], "end": []})
        s += 1
        for p in range(cut, len(toks)):
            steps.append({"step": s, "entries": [{"id": rid, "tokens": [toks[p]], "want": [0]}],
                          "end": [rid] if p == len(toks) - 1 else []})
            s += 1
        if cut == len(toks):
            steps[-1]["end"] = [rid]
    return steps


def changing_portions(requests, seed=0, sizes=(2, 3, 5, 7, 16, 17, 33, 64, 2, 9)):
    """Portions of changing size, down to two tokens, crossing page edges."""
    rng = random.Random(seed)
    steps, s = [], 0
    for rid, toks in requests.items():
        p = 0
        order = list(sizes)
        rng.shuffle(order)
        i = 0
        while p < len(toks):
            n = min(order[i % len(order)], len(toks) - p)
            if len(toks) - p - n == 1:  # never leave a single token over: portions go down to two
                n += 1
            i += 1
            steps.append({"step": s, "entries": [{"id": rid, "tokens": toks[p:p + n], "want": list(range(n))}],
                          "end": [rid] if p + n == len(toks) else []})
            p += n
            s += 1
    return steps


def mixed(requests, max_tokens, seed=0, max_live=4, tail=32, round_to=64):
    """Up to ``max_live`` live requests: portions of some beside decoded tokens of others, some left out of a
    step, admitted only while the rounded-up totals fit ``max_tokens`` so that freed pages are used again."""
    rng = random.Random(seed)
    up = lambda n: -(-n // round_to) * round_to
    waiting = list(requests.items())
    live = {}  # rid -> position
    steps, s = [], 0
    while waiting or live:
        while waiting and len(live) < max_live and \
                sum(up(len(requests[r])) for r in live) + up(len(waiting[0][1])) <= max_tokens:
            live[waiting.pop(0)[0]] = 0
        assert live, "max_tokens is too small for the next request"
        entries, ended = [], []
        chosen = [r for r in live if rng.random() < 0.8] or [next(iter(live))]
        for rid in chosen:
            toks, p = requests[rid], live[rid]
            if p < len(toks) - tail:
                n = min(rng.choice((2, 3, 4, 7, 13, 16, 21, 40)), len(toks) - tail - p)
                if len(toks) - tail - p - n == 1:
                    n += 1
            else:
                n = 1
            want = list(range(n)) if rng.random() < 0.7 else [n - 1]
            entries.append({"id": rid, "tokens": toks[p:p + n], "want": want})
            live[rid] = p + n
            if p + n == len(toks):
                ended.append(rid)
        for rid in ended:
            del live[rid]
        steps.append({"step": s, "entries": entries, "end": ended})
        s += 1
    return steps


def to_lines(steps):
    return [json.dumps(st) for st in steps]


def collect(steps, out_dir, vocab):
    """(request id, position) -> float32 logits, from the files the replay wrote."""
    got, pos = {}, {}
    for st in steps:
        wanted = [(e["id"], pos.get(e["id"], 0) + w) for e in st["entries"] for w in e["want"]]
        for e in st["entries"]:
            pos[e["id"]] = pos.get(e["id"], 0) + len(e["tokens"])
        for rid in st["end"]:
            pos.pop(rid, None)
        f = Path(out_dir) / f"{st['step']}.f32"
        if not wanted:
            assert not f.exists()
            continue
        arr = np.fromfile(f, dtype="<f4").reshape(len(wanted), vocab)
        for key, row in zip(wanted, arr):
            assert key not in got, f"{key} written twice"
            got[key] = row
    return got
