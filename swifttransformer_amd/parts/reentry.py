"""What happens to the residual stream before a marked run of a layer.

``InputInjection``: a pass over a group of layers starts from a mix of the stream and the step's
embedding,  x <- W [x ; e] + s,  W [hidden, 2 hidden] (the stream's half first), s one row of a
table [passes, hidden] chosen by the pass number.  Both halves enter the product in the engine's
storage type; the sum and the result are float.
``AdditiveEntry``: the pass starts from the plain sum  x <- x (+ e) + s,  all float.
The reference has no such parts."""
from __future__ import annotations

from typing import Dict, List

import torch

from ..ops import kernels as K
from ..weights.loader import TensorSpec
from .base import Part


class InputInjection(Part):
    """params: index (int: the row of the table this pass adds), passes (int: rows of the table)."""

    def __init__(self, spec, hidden_size, dtype):
        super().__init__(spec, hidden_size, dtype)
        self.index = int(self.param("index", 0) if "index" in spec.params else 0)
        self.passes = int(self.param("passes"))
        if not 0 <= self.index < self.passes:
            raise ValueError(f"pass {self.index} of {self.passes}")
        self.weight = self.shift = None

    def tensor_specs(self) -> List[TensorSpec]:
        H = self.hidden_size
        return [TensorSpec(self.name("weight"), (H, 2 * H), "matrix"),
                TensorSpec(self.name("shift"), (self.passes, H), "vector")]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.weight = tensors[self.name("weight")]
        self.shift = tensors[self.name("shift")][self.index].contiguous()

    def forward(self, x32: torch.Tensor, first32: torch.Tensor, ctx) -> torch.Tensor:
        both = K.concat_cast(x32, first32, self.dtype)
        return K.gemm(both, self.weight, bias=self.shift, out_f32=True)


class AdditiveEntry(Part):
    """params: index (int: the row of the table this pass adds), passes (int: rows of the table),
    add_first (bool: the step's embedding is added too)."""

    def __init__(self, spec, hidden_size, dtype):
        super().__init__(spec, hidden_size, dtype)
        self.index = int(spec.params.get("index", 0))
        self.passes = int(self.param("passes"))
        self.add_first = bool(spec.params.get("add_first", False))
        if not 0 <= self.index < self.passes:
            raise ValueError(f"pass {self.index} of {self.passes}")
        self.shift = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec(self.name("shift"), (self.passes, self.hidden_size), "vector")]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.shift = tensors[self.name("shift")][self.index].contiguous()

    def forward(self, x32: torch.Tensor, first32: torch.Tensor, ctx) -> torch.Tensor:
        return K.row_add(x32, first32 if self.add_first else None, self.shift)
