"""A per-layer input of the token's own: a second, narrow embedding whose row gates a projection of the
stream and re-enters it at unit root mean square.

    e = E[token, index * dim : (index + 1) * dim]         one table for all layers, a part of a row a layer
    g = gelu_tanh(G x) * e;  y = P g;  x <- x + y / rms(y) * s

The two matrices and the table are of the engine's storage type; the stream's row, the sums, the gated
vector, the unit norm and the sum into the stream are float.  One kernel a row does all of it (``token_side``: the row in LDS, a wave a gate feature, a thread
an output feature); a stream wider than that kernel's LDS takes the separate kernels.  The reference has
no such part."""
from __future__ import annotations

from typing import Dict, List

import torch

from ..ops import kernels as K
from ..weights.loader import TensorSpec
from .base import Part


class TokenSideInput(Part):
    """params: vocab_size, dim (the layer's part of a table row), index (which part), parts (how many parts a
    row has), eps (float, of the unit norm).  names: table, gate, proj, norm."""

    def __init__(self, spec, hidden_size, dtype):
        super().__init__(spec, hidden_size, dtype)
        self.vocab_size = int(self.param("vocab_size"))
        self.dim = int(self.param("dim"))
        self.index = int(spec.params.get("index", 0))
        self.parts = int(self.param("parts"))
        self.eps = float(self.param("eps"))
        if not 0 <= self.index < self.parts:
            raise ValueError(f"part {self.index} of {self.parts}")

    def tensor_specs(self) -> List[TensorSpec]:
        H = self.hidden_size
        return [TensorSpec(self.name("table"), (self.vocab_size, self.parts * self.dim), "table"),
                TensorSpec(self.name("gate"), (self.dim, H), "matrix"),
                TensorSpec(self.name("proj"), (H, self.dim), "matrix"),
                TensorSpec(self.name("norm"), (H,), "vector", init="gain")]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        lo = self.index * self.dim
        self.table = tensors[self.name("table")][:, lo:lo + self.dim]     # this layer's columns of the shared table
        self.fused = K.token_side_fits(self.hidden_size, self.dim)
        if not self.fused:
            self.table = self.table.contiguous()
        self.w_gate, self.w_proj, self.gain = (tensors[self.name(n)] for n in ("gate", "proj", "norm"))

    def forward(self, x32: torch.Tensor, ctx, x_t: torch.Tensor = None) -> torch.Tensor:
        """``x_t``: the stream in the storage type, where the caller has it already."""
        if self.fused:
            return K.token_side(x32, ctx.token_ids, ctx.token_item, self.table, self.w_gate, self.w_proj, self.gain,
                                self.eps)
        T = x32.shape[0]
        if x_t is None:
            x_t = x32 if self.dtype == torch.float32 else K.cast(x32, self.dtype)
        e = K.empty((T, self.dim), self.dtype, x32.device)
        K.lookup(ctx.token_ids, self.table, out_f32=e if self.dtype == torch.float32 else None,
                 out_t=None if self.dtype == torch.float32 else e)
        g = K.activation_multiply(K.gemm(x_t, self.w_gate), e, "gelu_tanh")
        y32 = K.gemm(g, self.w_proj, out_f32=True)
        return K.unit_add(x32, y32, self.gain, self.eps)
