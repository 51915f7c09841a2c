"""What a part says about each tensor it wants from the checkpoint."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Tuple


@dataclass(frozen=True)
class TensorSpec:
    """``role`` decides how the tensor is kept and how the random-weights mode draws it:

    ``matrix``  a projection or embedding table: kept in the run's type (bfloat16 when serving); N(0, std)
    ``bias``    a vector added to a projection: kept in float; N(0, std)
    ``norm``    a norm's scale: kept in float; 1 + N(0, 0.1)
    ``table``   an integer table: kept as int32; zeros in the random-weights mode

    A tensor that the file stores in 32-bit float is never narrowed when the part asks for ``keep32``.
    """

    name: str
    shape: Tuple[int, ...]
    role: str = "matrix"
    keep32: bool = False

    def __post_init__(self):
        if self.role not in ("matrix", "bias", "norm", "table"):
            raise ValueError(f"unknown tensor role {self.role!r}")
