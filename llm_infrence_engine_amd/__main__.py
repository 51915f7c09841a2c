"""``python -m llm_infrence_engine_amd``: generate from token ids on one GPU.

Option names follow the reference's only command line (``python -m miniserve.server``,
src/miniserve/server.py:435-448) where it has them: --model --dtype --device --max-len --max-seqs
--num-blocks --cuda-graphs (on by default in bfloat16; --no-hip-graphs turns it off); the request options are those of its ``Request``
(src/miniserve/engine.py:32-38).  There is no HTTP server here: prompts come from the command line.
"""
from __future__ import annotations

import argparse
import json
import sys


def _ids(text: str):
    return [int(t) for t in text.replace(",", " ").split()]


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="python -m llm_infrence_engine_amd", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", help="folder with config.json and *.safetensors")
    ap.add_argument("--random-config", help="instead of --model: a preset (tinyA, tinyB, 0.5b, 7b, 32b) or the path of a "
                                            "config.json, filled with random weights drawn on the GPU")
    ap.add_argument("--seed", type=int, default=0, help="seed of the random weights")
    ap.add_argument("--dtype", default="bfloat16", choices=["float32", "bfloat16"])
    ap.add_argument("--device", default="cuda:0")
    ap.add_argument("--prompt-ids", action="append", default=[], help="token ids, e.g. 1,2,3 (repeatable)")
    ap.add_argument("--prompt-file", help="a file with one prompt a line: token ids separated by commas or blanks")
    ap.add_argument("--prompt", action="append", default=[], help="text; needs tokenizer.json in the model folder")
    ap.add_argument("--max-new-tokens", type=int, default=64)
    ap.add_argument("--temperature", type=float, default=0.0)
    ap.add_argument("--top-k", type=int, default=0)
    ap.add_argument("--top-p", type=float, default=1.0)
    ap.add_argument("--sample-seed", type=int, default=None)
    ap.add_argument("--eos-ids", default="", help="stop ids, e.g. 151645,151643")
    ap.add_argument("--max-len", type=int, default=1024)
    ap.add_argument("--max-seqs", "--max-num-seqs", dest="max_seqs", type=int, default=32)
    ap.add_argument("--num-blocks", type=int, default=None)
    ap.add_argument("--block-size", type=int, default=16)
    ap.add_argument("--max-num-batched-tokens", type=int, default=2048)
    ap.add_argument("--gpu-memory-fraction", type=float, default=None,
                    help="without --num-blocks: size the page pool to this share of the device's memory, weights included")
    ap.add_argument("--cuda-graphs", "--hip-graphs", "--hip-graph", dest="hip_graphs", action="store_true", default=None,
                    help="replay decode-only steps from captured HIP graphs (the default in bfloat16)")
    ap.add_argument("--no-hip-graphs", dest="hip_graphs", action="store_false", help="launch every kernel of a decode step")
    ap.add_argument("--decode-steps-per-launch", type=int, default=1,
                    help="with graphs: decode steps queued in one launch while every request decodes greedily")
    a = ap.parse_args(argv)
    if bool(a.model) == bool(a.random_config):
        ap.error("give exactly one of --model and --random-config")

    from . import LLM, SamplingParams, load_random_model
    from .config import PRESETS, config_from_dict, preset

    model_dir = model = a.model
    if a.random_config:
        if a.random_config in PRESETS:
            cfg = config_from_dict(preset(a.random_config))
        else:
            with open(a.random_config) as fh:
                cfg = config_from_dict(json.load(fh))
        model = load_random_model(cfg, seed=a.seed, dtype=a.dtype, device=a.device)
    prompts = [_ids(p) for p in a.prompt_ids]
    if a.prompt_file:
        with open(a.prompt_file) as fh:
            prompts += [_ids(line) for line in fh if line.strip()]
    tok = None
    if a.prompt:
        from pathlib import Path

        tj = Path(model_dir or ".") / "tokenizer.json"
        if not model_dir or not tj.is_file():
            ap.error(f"--prompt needs {tj}; give --prompt-ids instead")
        from tokenizers import Tokenizer

        tok = Tokenizer.from_file(str(tj))
        prompts += [tok.encode(p).ids for p in a.prompt]
    if not prompts:
        ap.error("give at least one --prompt-ids, --prompt-file or --prompt")
    llm = LLM(model, dtype=a.dtype, device=a.device, num_blocks=a.num_blocks, block_size=a.block_size,
              max_seqs=a.max_seqs, max_len=a.max_len, max_num_batched_tokens=a.max_num_batched_tokens,
              hip_graphs=a.hip_graphs, decode_steps_per_launch=a.decode_steps_per_launch,
              gpu_memory_fraction=a.gpu_memory_fraction)
    params = SamplingParams(a.max_new_tokens, a.temperature, a.top_k, a.top_p, a.sample_seed, tuple(_ids(a.eos_ids)))
    for i, out in enumerate(llm.generate(prompts, params)):
        rec = {"prompt": i, "token_ids": out.token_ids, "finish_reason": out.finish_reason}
        if tok is not None:
            rec["text"] = tok.decode(out.token_ids)
        print(json.dumps(rec), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
