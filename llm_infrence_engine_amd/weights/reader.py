"""Weights from safetensors files, by tensor name.

Like the reference's loader (src/miniserve/loader.py:41-43) every ``*.safetensors`` file of the folder
is read and merged by name, with no renaming; ``model.safetensors.index.json`` is consulted only to name
the files of a sharded checkpoint that are not in the folder.  Unlike it (``strict=False`` at loader.py:45 drops
mismatches silently) the names and shapes are checked against what the model's parts ask for, and one
error lists everything that is missing, unexpected or of the wrong shape or type.
"""
from __future__ import annotations

import json
from pathlib import Path
from typing import Dict, Iterable, List

import torch
from safetensors import safe_open

from .spec import TensorSpec

INDEX_NAME = "model.safetensors.index.json"
_FLOAT_TYPES = {"F32", "BF16", "F16", "F64"}
_INT_TYPES = {"I8", "I16", "I32", "I64", "U8"}


class WeightsError(ValueError):
    """The checkpoint does not hold what the model needs."""

    def __init__(self, folder, missing=(), unexpected=(), wrong_shape=(), wrong_type=()):
        self.missing, self.unexpected = list(missing), list(unexpected)
        self.wrong_shape, self.wrong_type = list(wrong_shape), list(wrong_type)
        lines = [f"weights in {folder} do not fit the model:"]
        if self.missing:
            lines.append(f"  missing ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        for name, want, got in self.wrong_shape:
            lines.append(f"  wrong shape: {name} is {list(got)}, the model needs {list(want)}")
        for name, got, want in self.wrong_type:
            lines.append(f"  wrong type: {name} is stored as {got}, the model needs {want}")
        super().__init__("\n".join(lines))


class CheckpointReader:
    """Index of every tensor in a model folder; tensors are read one at a time when asked for."""

    def __init__(self, model_dir):
        self.folder = Path(model_dir)
        files = sorted(self.folder.glob("*.safetensors"))
        if not files:
            raise WeightsError(self.folder, missing=["(no *.safetensors file in the folder)"])
        # a sharded checkpoint's index is read only to say which of its files are not there: the tensors
        # themselves are found by reading every file's own header
        absent = sorted(self._shards_named_by_index() - {f.name for f in files})
        if absent:
            raise WeightsError(self.folder, missing=[f"(file {n}, named by {INDEX_NAME})" for n in absent])
        self._where: Dict[str, Path] = {}
        self._shape: Dict[str, tuple] = {}
        self._dtype: Dict[str, str] = {}
        for f in files:
            with safe_open(str(f), framework="pt") as fh:
                for name in fh.keys():
                    sl = fh.get_slice(name)
                    self._where[name] = f
                    self._shape[name] = tuple(sl.get_shape())
                    self._dtype[name] = str(sl.get_dtype())
        self._open: Dict[Path, object] = {}

    def _shards_named_by_index(self) -> set:
        index = self.folder / INDEX_NAME
        if not index.is_file():
            return set()
        try:
            weight_map = json.loads(index.read_text()).get("weight_map", {})
        except (ValueError, AttributeError) as e:
            raise WeightsError(self.folder, missing=[f"({INDEX_NAME} cannot be read: {e})"]) from e
        return {str(v) for v in weight_map.values()} if isinstance(weight_map, dict) else set()

    def names(self) -> List[str]:
        return sorted(self._where)

    def shape(self, name: str) -> tuple:
        return self._shape[name]

    def stored_type(self, name: str) -> str:
        return self._dtype[name]

    def check(self, wanted: Iterable[TensorSpec], ignorable: Iterable[str] = ()) -> None:
        """Raise one ``WeightsError`` naming every missing, unexpected, misshapen or mistyped tensor.
        ``ignorable`` names may be present without being used (a tied head's own copy)."""
        wanted = list(wanted)
        names = {s.name for s in wanted}
        missing = [s.name for s in wanted if s.name not in self._where]
        unexpected = [n for n in self.names() if n not in names and n not in set(ignorable)]
        wrong_shape, wrong_type = [], []
        for s in wanted:
            if s.name not in self._where:
                continue
            if tuple(s.shape) != self._shape[s.name]:
                wrong_shape.append((s.name, tuple(s.shape), self._shape[s.name]))
            t = self._dtype[s.name]
            if s.role == "table":
                if t not in _INT_TYPES:
                    wrong_type.append((s.name, t, "an integer type"))
            elif t not in _FLOAT_TYPES:
                wrong_type.append((s.name, t, "F32, BF16 or F16"))
        if missing or unexpected or wrong_shape or wrong_type:
            raise WeightsError(self.folder, missing, unexpected, wrong_shape, wrong_type)

    def get(self, name: str) -> torch.Tensor:
        """The tensor as stored (on the CPU)."""
        f = self._where[name]
        fh = self._open.get(f)
        if fh is None:
            fh = self._open[f] = safe_open(str(f), framework="pt")
        return fh.get_tensor(name)

    def close(self) -> None:
        self._open.clear()


def place(t: torch.Tensor, spec: TensorSpec, run_dtype: torch.dtype, device) -> torch.Tensor:
    """Move a stored tensor to the device in the type it is kept in: matrices in the run's type (a matrix
    stored in 32-bit float stays so when its part says ``keep32``), vectors in float, integer tables as int32."""
    if spec.role == "table":
        return t.to(device=device, dtype=torch.int32).contiguous()
    if spec.role in ("bias", "norm"):
        return t.to(device=device, dtype=torch.float32).contiguous()
    if spec.keep32 and t.dtype == torch.float32:
        return t.to(device=device).contiguous()
    return t.to(device=device, dtype=run_dtype).contiguous()
