"""Model folder -> a model with its weights on the GPU.  The class is chosen by config.json.

After the reference's ``load_model(name_or_path, dtype, device)`` (src/miniserve/loader.py:29-51); only local
folders are read (there is no download) and token ids, not text, go in and out, so no tokenizer is returned.
"""
from __future__ import annotations

import torch

from .config import load_config
from .parts.base import Runtime
from .parts.model import Model
from .weights import CheckpointReader

DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def load_model(model_dir, dtype: str = "bfloat16", device: str = "cuda:0") -> Model:
    if isinstance(dtype, torch.dtype):
        dtype = {v: k for k, v in DTYPES.items()}.get(dtype, str(dtype))
    if dtype not in DTYPES:
        raise ValueError(f"dtype must be 'bfloat16' or 'float32', got {dtype!r}")
    dev = torch.device(device)
    if dev.type != "cuda":
        raise RuntimeError(f"the engine runs on the GPU only (device {device!r} was asked for); there is no CPU path")
    if not torch.cuda.is_available():
        raise RuntimeError("no GPU is visible to this process; the engine has no CPU path")
    config = load_config(model_dir)
    model = Model(config.to_spec())
    model.config = config
    model.load(CheckpointReader(model_dir), Runtime(dev, DTYPES[dtype]))
    return model
