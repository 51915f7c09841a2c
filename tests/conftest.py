"""Shared fixtures: the ``gpu`` marker and the tiny configurations every test uses."""
import json
import sys
from pathlib import Path

import pytest
import torch

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


# Two tiny Qwen2 configurations that differ in every size and option, and a third with an
# explicit head_dim, an odd vocabulary, one key/value head and a width that is no power of two.
TINY_A = {
    "architectures": ["Qwen2ForCausalLM"],
    "num_hidden_layers": 2, "hidden_size": 64, "num_attention_heads": 4, "num_key_value_heads": 2,
    "intermediate_size": 128, "vocab_size": 256, "rope_theta": 10000.0, "rms_norm_eps": 1e-6,
    "tie_word_embeddings": True,
}
TINY_B = {
    "architectures": ["Qwen2ForCausalLM"],
    "num_hidden_layers": 3, "hidden_size": 192, "num_attention_heads": 6, "num_key_value_heads": 2,
    "intermediate_size": 320, "vocab_size": 384, "rope_theta": 1000000.0, "rms_norm_eps": 1e-5,
    "tie_word_embeddings": False,
}
TINY_C = {
    "architectures": ["Qwen2ForCausalLM"],
    "num_hidden_layers": 2, "hidden_size": 120, "num_attention_heads": 5, "num_key_value_heads": 1,
    "head_dim": 48, "intermediate_size": 200, "vocab_size": 331, "rope_theta": 50000.0,
    "rms_norm_eps": 3e-6, "tie_word_embeddings": False,
}
# head size 64 and 7 query heads per key/value head, as the 0.5B model has: the sizes the matrix-core kernels serve
TINY_D = {
    "architectures": ["Qwen2ForCausalLM"],
    "num_hidden_layers": 2, "hidden_size": 448, "num_attention_heads": 7, "num_key_value_heads": 1,
    "intermediate_size": 264, "vocab_size": 509, "rope_theta": 1000000.0, "rms_norm_eps": 1e-6,
    "tie_word_embeddings": True,
}
TINY = {"A": TINY_A, "B": TINY_B, "C": TINY_C, "D": TINY_D}


def plain_random_weights(cfg: dict, seed: int, std: float = 0.02, dtype=torch.float32) -> dict:
    """Random tensors under the checkpoint's names, made here (not by the product's writer) so the
    plain implementation's own tests need nothing from the package."""
    g = torch.Generator().manual_seed(seed)
    H, I, V = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    nh, nkv = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    d = cfg.get("head_dim") or H // nh

    def mat(*shape):
        return (torch.randn(*shape, generator=g) * std).to(dtype)

    def norm(n):
        return (1.0 + 0.1 * torch.randn(n, generator=g)).to(dtype)

    w = {"model.embed_tokens.weight": mat(V, H)}
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        w[p + "self_attn.q_proj.weight"] = mat(nh * d, H)
        w[p + "self_attn.q_proj.bias"] = mat(nh * d)
        w[p + "self_attn.k_proj.weight"] = mat(nkv * d, H)
        w[p + "self_attn.k_proj.bias"] = mat(nkv * d)
        w[p + "self_attn.v_proj.weight"] = mat(nkv * d, H)
        w[p + "self_attn.v_proj.bias"] = mat(nkv * d)
        w[p + "self_attn.o_proj.weight"] = mat(H, nh * d)
        w[p + "mlp.gate_proj.weight"] = mat(I, H)
        w[p + "mlp.up_proj.weight"] = mat(I, H)
        w[p + "mlp.down_proj.weight"] = mat(H, I)
        w[p + "input_layernorm.weight"] = norm(H)
        w[p + "post_attention_layernorm.weight"] = norm(H)
    w["model.norm.weight"] = norm(H)
    if not cfg.get("tie_word_embeddings", False):
        w["lm_head.weight"] = mat(V, H)
    return w


def write_plain_model(folder, cfg: dict, weights: dict) -> Path:
    from safetensors.torch import save_file

    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in weights.items()}, str(folder / "model.safetensors"))
    return folder


@pytest.fixture
def tiny_configs():
    return {k: dict(v) for k, v in TINY.items()}
