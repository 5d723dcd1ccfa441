"""The linear-layer interface every weight format implements (hibana/weights/linear.py:25-40 of the reference):
`lin(x)` for BF16 rows, `out_features`, `in_features`, `bytes`, `dequantize()` -> FP32 [N, K], and `w3`, the optional
3-bit decode copy. A model lists its projections with `linears()` -> iterable of (name, linear)."""
from __future__ import annotations

from typing import Protocol, runtime_checkable

import torch


@runtime_checkable
class Linear(Protocol):
    w3: object

    @property
    def out_features(self) -> int: ...

    @property
    def in_features(self) -> int: ...

    @property
    def bytes(self) -> int: ...

    def dequantize(self) -> torch.Tensor: ...

    def __call__(self, x: torch.Tensor) -> torch.Tensor: ...
