"""Random-weights mode: write a model folder (config.json, model.safetensors) from a configuration and a seed.

The reference has no such mode (its loader only reads checkpoints, src/miniserve/loader.py:29-51).
Tensors are drawn in the order the model's parts list them, in float on the CPU from one seeded
generator: matrices and biases N(0, std), norm scales 1 + N(0, 0.1); then stored in ``dtype``.
"""
from __future__ import annotations

import json
from pathlib import Path

import torch
from safetensors.torch import save_file

_STORE = {"float32": torch.float32, "bfloat16": torch.bfloat16, "float16": torch.float16}


def random_tensors(specs, seed: int, std: float = 0.02, norm_std: float = 0.1, dtype: str = "bfloat16") -> dict:
    if dtype not in _STORE:
        raise ValueError(f"dtype must be one of {sorted(_STORE)}, got {dtype!r}")
    g = torch.Generator().manual_seed(seed)
    out = {}
    for s in specs:
        if s.role == "table":
            out[s.name] = torch.zeros(s.shape, dtype=torch.int32)
            continue
        t = torch.randn(s.shape, generator=g, dtype=torch.float32)
        t = 1.0 + norm_std * t if s.role == "norm" else std * t
        out[s.name] = t.to(_STORE[dtype]).contiguous()
    return out


def write_random_model(folder, config, seed: int = 0, dtype: str = "bfloat16", std: float = 0.02,
                       norm_std: float = 0.1) -> Path:
    """``config`` is a typed configuration of a registered architecture."""
    from ..parts.model import Model

    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    model = Model(config.to_spec())
    tensors = random_tensors(model.tensor_specs(), seed, std, norm_std, dtype)
    d = config.to_dict()
    d["torch_dtype"] = dtype
    (folder / "config.json").write_text(json.dumps(d, indent=1))
    save_file(tensors, str(folder / "model.safetensors"))
    return folder
