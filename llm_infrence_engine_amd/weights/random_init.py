"""Random-weights mode: write a model folder (config.json, model.safetensors) from a configuration and a seed.

The reference has no such mode (its loader only reads checkpoints, src/miniserve/loader.py:29-51).
Tensors are drawn in the order the model's parts list them, in float on the CPU from one seeded
generator: matrices and biases N(0, std), norm scales 1 + N(0, 0.1); then stored in ``dtype``.

``load_random_model`` is the same mode without the folder, for models too large to pass through host
memory and a file: every tensor is drawn on the GPU, piece by piece, straight in the type it is kept in.
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


class RandomSource:
    """Stands where a ``CheckpointReader`` stands in ``Model.load``: ``get(name)`` draws the tensor on the device.

    Every tensor has a generator of its own, seeded from ``seed`` and the tensor's place in the model's list, so
    a tensor's values depend on nothing but the seed, the list, its shape and the piece size.  Matrices are drawn in pieces of
    at most ``piece`` values in float and rounded into the kept type at once, so the largest table costs its own
    size plus one piece, not a float copy of itself."""

    def __init__(self, specs, seed: int, run_dtype: torch.dtype, device, std: float = 0.02, norm_std: float = 0.1,
                 piece: int = 1 << 26):
        self.specs = {s.name: (i, s) for i, s in enumerate(specs)}
        self.seed, self.run_dtype, self.device = int(seed), run_dtype, torch.device(device)
        self.std, self.norm_std, self.piece = float(std), float(norm_std), int(piece)

    def check(self, wanted, ignorable=()) -> None:
        missing = [s.name for s in wanted if s.name not in self.specs]
        if missing:
            raise KeyError(f"the random source was made for another model; it does not know {missing}")

    def get(self, name: str) -> torch.Tensor:
        i, s = self.specs[name]
        if s.role == "table":
            return torch.zeros(s.shape, dtype=torch.int32, device=self.device)
        g = torch.Generator(device=self.device).manual_seed((self.seed * 1000003 + i) & ((1 << 62) - 1))
        keep = torch.float32 if s.role in ("bias", "norm") or s.keep32 else self.run_dtype
        out = torch.empty(s.shape, dtype=keep, device=self.device)
        flat = out.view(-1)
        for a in range(0, flat.numel(), self.piece):
            b = min(flat.numel(), a + self.piece)
            t = torch.randn(b - a, generator=g, dtype=torch.float32, device=self.device)
            t = t.mul_(self.norm_std).add_(1.0) if s.role == "norm" else t.mul_(self.std)
            flat[a:b].copy_(t)
        return out

    def close(self) -> None:
        pass


def load_random_model(config, seed: int = 0, dtype: str = "bfloat16", device: str = "cuda:0", std: float = 0.02,
                      norm_std: float = 0.1):
    """A model of ``config`` (a typed configuration of a registered architecture) with seeded random weights
    drawn on the GPU: no folder, no file and no copy in host memory.  The distributions are
    ``write_random_model``'s; the values are not (another generator)."""
    from ..parts.base import Runtime
    from ..parts.model import Model

    if dtype not in ("float32", "bfloat16"):
        raise ValueError(f"dtype must be 'bfloat16' or 'float32', got {dtype!r}")
    dev = torch.device(device)
    if dev.type != "cuda" or not torch.cuda.is_available():
        raise RuntimeError("random weights are drawn on the GPU; no GPU is visible (the engine has no CPU path)")
    model = Model(config.to_spec())
    model.config = config
    run_dtype = _STORE[dtype]
    model.load(RandomSource(model.tensor_specs(), seed, run_dtype, dev, std, norm_std), Runtime(dev, run_dtype))
    return model
