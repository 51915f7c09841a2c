"""Typed configuration of the Qwen2 dense decoder and its translation into a ``ModelSpec``.

Keys and defaults follow the reference's ``ModelConfig.from_json`` (src/miniserve/model.py:42-58):
``rope_theta`` falls back to ``rope_parameters.rope_theta`` and then to 10000.0, and
``tie_word_embeddings`` defaults to False.  ``head_dim`` is hidden_size // num_attention_heads
unless config.json states it (model.py:38-40 always derives it).  Fixed by the reference's code
and therefore constants of this architecture: q/k/v projections with bias and the output
projection without (model.py:108-111), SiLU as the gate's activation and no feed-forward bias
(model.py:160-165), full rotary dimension with half-split pairing (model.py:83-98), scores scaled
by 1/sqrt(head_dim) (model.py:143), pre-norm residual layers (model.py:184-185).
"""
from __future__ import annotations

import math
from dataclasses import asdict, dataclass

from .registry import ConfigError, register_architecture, require
from .spec import ModelSpec, PartSpec, Run, layer


@dataclass(frozen=True)
class Qwen2Config:
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    rms_norm_eps: float
    rope_theta: float = 10000.0
    tie_word_embeddings: bool = False
    head_dim: int = 0  # 0: hidden_size // num_attention_heads

    architecture = "Qwen2ForCausalLM"

    def __post_init__(self):
        for k in ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                  "num_attention_heads", "num_key_value_heads"):
            if getattr(self, k) <= 0:
                raise ConfigError(f"{k} must be positive, got {getattr(self, k)}")
        if self.head_dim == 0:
            if self.hidden_size % self.num_attention_heads:
                raise ConfigError(f"hidden_size {self.hidden_size} is not a multiple of num_attention_heads "
                                  f"{self.num_attention_heads} and config.json gives no head_dim")
            object.__setattr__(self, "head_dim", self.hidden_size // self.num_attention_heads)
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(f"num_attention_heads {self.num_attention_heads} is not a multiple of "
                              f"num_key_value_heads {self.num_key_value_heads}")
        if self.head_dim % 2:
            raise ConfigError(f"head_dim {self.head_dim} must be even for the rotary pairing")
        if not self.rms_norm_eps >= 0:
            raise ConfigError(f"rms_norm_eps must be >= 0, got {self.rms_norm_eps}")
        if not self.rope_theta > 0:
            raise ConfigError(f"rope_theta must be > 0, got {self.rope_theta}")

    # ------------------------------------------------------------------ config.json
    @classmethod
    def from_dict(cls, d: dict) -> "Qwen2Config":
        rope = d.get("rope_theta")
        if rope is None:
            rope = (d.get("rope_parameters") or {}).get("rope_theta", 10000.0)
        scaling = d.get("rope_scaling")
        if scaling not in (None, {}):
            raise ConfigError(f"rope_scaling={scaling!r} is not supported (the reference never scales the rotation)")
        if d.get("use_sliding_window"):
            raise ConfigError("use_sliding_window=true is not supported (the reference attends to every key)")
        return cls(
            vocab_size=require(d, "vocab_size", int),
            hidden_size=require(d, "hidden_size", int),
            intermediate_size=require(d, "intermediate_size", int),
            num_hidden_layers=require(d, "num_hidden_layers", int),
            num_attention_heads=require(d, "num_attention_heads", int),
            num_key_value_heads=require(d, "num_key_value_heads", int),
            rms_norm_eps=require(d, "rms_norm_eps", float),
            rope_theta=float(rope),
            tie_word_embeddings=bool(d.get("tie_word_embeddings", False)),
            head_dim=int(d.get("head_dim") or 0),
        )

    def to_dict(self) -> dict:
        d = asdict(self)
        d["architectures"] = [self.architecture]
        d["model_type"] = "qwen2"
        return d

    # ------------------------------------------------------------------ derived sizes
    @property
    def num_params(self) -> int:
        H, I, V, d = self.hidden_size, self.intermediate_size, self.vocab_size, self.head_dim
        nh, nkv = self.num_attention_heads, self.num_key_value_heads
        layer = (nh + 2 * nkv) * d * (H + 1) + H * nh * d + 3 * H * I + 2 * H
        return V * H * (1 if self.tie_word_embeddings else 2) + self.num_hidden_layers * layer + H

    def kv_bytes_per_token(self, bytes_per_value: int = 2) -> int:
        """layers x 2 x kv heads x head_dim x bytes (src/miniserve/cache.py:27-29)."""
        return self.num_hidden_layers * 2 * self.num_key_value_heads * self.head_dim * bytes_per_value

    # ------------------------------------------------------------------ the model as data
    def to_spec(self) -> ModelSpec:
        H = self.hidden_size
        norm = {"size": H, "eps": self.rms_norm_eps}
        layers = []
        for i in range(self.num_hidden_layers):
            p = f"model.layers.{i}."
            layers.append(layer(
                "pre_norm_residual",
                mixer=PartSpec("gqa_attention", p + "self_attn.", {
                    "hidden_size": H, "num_heads": self.num_attention_heads,
                    "num_kv_heads": self.num_key_value_heads, "head_dim": self.head_dim,
                    "scale": 1.0 / math.sqrt(self.head_dim), "qkv_bias": True, "out_bias": False,
                    "window": None}),
                position=PartSpec("rotary_half", "", {"head_dim": self.head_dim, "rotary_dim": self.head_dim,
                                                      "theta": self.rope_theta}),
                feed_forward=PartSpec("swiglu", p + "mlp.", {"hidden_size": H,
                                                              "intermediate_size": self.intermediate_size}),
                mixer_norm=PartSpec("rms_norm", p + "input_layernorm.", norm),
                feed_forward_norm=PartSpec("rms_norm", p + "post_attention_layernorm.", norm),
            ))
        head = {"hidden_size": H, "vocab_size": self.vocab_size,
                "tied_to": "model.embed_tokens.weight" if self.tie_word_embeddings else None}
        return ModelSpec(
            architecture=self.architecture, hidden_size=H, vocab_size=self.vocab_size,
            embedding=PartSpec("token_embedding", "model.embed_tokens.", {"vocab_size": self.vocab_size, "hidden_size": H}),
            layers=tuple(layers), order=tuple(Run(i) for i in range(self.num_hidden_layers)),
            final_norm=PartSpec("rms_norm", "model.norm.", norm),
            head=PartSpec("lm_head", "lm_head.", head),
        )


register_architecture(Qwen2Config.architecture, Qwen2Config, model_type="qwen2")
