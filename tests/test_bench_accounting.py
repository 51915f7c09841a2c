"""The byte and flop counts that bench.py prices its roofline fractions with (no GPU)."""
import importlib.util
import os

from llm_infrence_engine_amd.config import config_from_dict, preset

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
spec = importlib.util.spec_from_file_location("bench", os.path.join(ROOT, "bench.py"))
bench = importlib.util.module_from_spec(spec)
spec.loader.exec_module(bench)


def test_decode_bytes_of_the_half_billion_shape():
    cfg = config_from_dict(preset("0.5b"))
    # the reference counts 494,032,768 parameters = 988,065,536 bytes in bfloat16 (results/raw/gpu_launch_diag.json)
    assert cfg.num_params == 494_032_768
    weights = bench.decode_bytes(cfg, batch=0, context=0)
    small = (24 * ((14 + 4) * 64 + 2 * 896) + 896) * 2     # biases and norm scales are read as float: 2 bytes more each
    assert weights == 988_065_536 + small
    # keys and values: 12,288 bytes a token (tests/test_kv_cache.py:93 of the reference)
    assert bench.decode_bytes(cfg, batch=8, context=640) - weights == 8 * 640 * 12_288


def test_prefill_flops_of_the_half_billion_shape():
    cfg = config_from_dict(preset("0.5b"))
    f = bench.prefill_flops(cfg, 2048)
    linear = 2 * 2048 * 24 * 14_912_384 - 2 * 2048 * 24 * (18 * 64 + 2 * 896)   # per-layer parameters without biases and norms
    attention = 24 * 4 * 14 * 64 * 2048 * 2049 // 2
    assert f == linear + attention + 2 * 151_936 * 896
    assert 1.6e12 < f < 1.7e12


def test_further_shapes_have_their_published_sizes():
    assert config_from_dict(preset("7b")).num_params == 7_615_616_512
    assert config_from_dict(preset("32b")).kv_bytes_per_token(2) == 262_144


def test_more_than_one_gpu_is_refused(capsys):
    import sys
    argv = sys.argv
    sys.argv = ["bench.py", "--gpus", "2"]
    try:
        assert bench.main() == 2
    finally:
        sys.argv = argv
    assert "one GPU" in capsys.readouterr().out
