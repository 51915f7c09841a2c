"""Named config.json contents for the random-weights mode: the shapes the published Qwen2.5 checkpoints
have and the two tiny ones the tests use, so that ``--random-config 0.5b`` needs no file.  These are data
of the kind a config.json holds; no part or kernel reads them.
"""
from __future__ import annotations

_QWEN2 = {"architectures": ["Qwen2ForCausalLM"], "rope_theta": 1000000.0, "rms_norm_eps": 1e-6}

PRESETS = {
    "tinyA": {**_QWEN2, "num_hidden_layers": 2, "hidden_size": 64, "num_attention_heads": 4, "num_key_value_heads": 2,
              "intermediate_size": 128, "vocab_size": 256, "rope_theta": 10000.0, "tie_word_embeddings": True},
    "tinyB": {**_QWEN2, "num_hidden_layers": 3, "hidden_size": 192, "num_attention_heads": 6, "num_key_value_heads": 2,
              "intermediate_size": 320, "vocab_size": 384, "rms_norm_eps": 1e-5, "tie_word_embeddings": False},
    "0.5b": {**_QWEN2, "num_hidden_layers": 24, "hidden_size": 896, "num_attention_heads": 14,
             "num_key_value_heads": 2, "intermediate_size": 4864, "vocab_size": 151936, "tie_word_embeddings": True},
    "7b": {**_QWEN2, "num_hidden_layers": 28, "hidden_size": 3584, "num_attention_heads": 28,
           "num_key_value_heads": 4, "intermediate_size": 18944, "vocab_size": 152064, "tie_word_embeddings": False},
    "32b": {**_QWEN2, "num_hidden_layers": 64, "hidden_size": 5120, "num_attention_heads": 40,
            "num_key_value_heads": 8, "intermediate_size": 27648, "vocab_size": 152064, "tie_word_embeddings": False},
}


def preset(name: str) -> dict:
    if name not in PRESETS:
        raise KeyError(f"no preset {name!r}; there are {', '.join(sorted(PRESETS))}")
    return dict(PRESETS[name])
