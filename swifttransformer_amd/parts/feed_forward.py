"""Dense feed-forward: y = act(x W1^T + b1) W2^T + b2, returned added to the residual.

Reference src/csrc/layer/ffn.cc:71-124: FC1 product, fused bias+activation kernel,
FC2 product, bias kernel; the residual add is a further kernel
(src/csrc/model/gpt/gpt.cc:496-501).  Here bias+ReLU is the FC1 product's epilogue and
bias+residual the FC2 product's."""
from __future__ import annotations

from typing import Dict, List

import torch

from ..ops import kernels as K
from ..weights.loader import TensorSpec
from .base import Part, fold_output_scale



class DenseFeedForward(Part):
    """params: inner (int), activation (a name the products' epilogues know), bias (bool),
    residual_scale (float, default 1: the factor with which the result enters the residual stream), out_scale
    (bool: the file holds a per-feature factor on the result; it is folded into the second matrix and bias)."""

    def __init__(self, spec, hidden_size, dtype):
        super().__init__(spec, hidden_size, dtype)
        self.inner = int(self.param("inner"))
        self.activation = str(self.param("activation", "relu"))
        if self.activation not in K.ACTIVATIONS:
            raise ValueError(f"feed-forward activation {self.activation!r} has no kernel; "
                             f"available: {sorted(K.ACTIVATIONS)}")
        self.bias = bool(self.param("bias", True))
        self.residual_scale = float(spec.params.get("residual_scale", 1.0))
        self.out_scale = bool(spec.params.get("out_scale", False))
        self.w1 = self.b1 = self.w2 = self.b2 = None

    def tensor_specs(self) -> List[TensorSpec]:
        H, F = self.hidden_size, self.inner
        specs = [TensorSpec(self.name("fc1.weight"), (F, H), "matrix"),
                 TensorSpec(self.name("fc2.weight"), (H, F), "matrix")]
        if self.bias:
            specs += [TensorSpec(self.name("fc1.bias"), (F,), "vector"),
                      TensorSpec(self.name("fc2.bias"), (H,), "vector")]
        if self.out_scale:
            specs.append(TensorSpec(self.name("out_scale"), (H,), "vector", init="gain"))
        return specs

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.w1 = tensors[self.name("fc1.weight")]
        self.w2 = tensors[self.name("fc2.weight")]
        if self.bias:
            self.b1 = tensors[self.name("fc1.bias")]
            self.b2 = tensors[self.name("fc2.bias")]
        if self.out_scale:
            self.w2, self.b2 = fold_output_scale(self.w2, self.b2, tensors[self.name("out_scale")])

    accepts_norm = True     # forward(..., norm=part) normalises residual32 itself

    def forward(self, x_t, residual32: torch.Tensor, ctx, norm=None) -> torch.Tensor:
        x_in = norm.as_input(residual32) if norm is not None else x_t
        h = K.gemm(x_in, self.w1, bias=self.b1, activation=self.activation)
        return K.gemm(h, self.w2, bias=self.b2, residual=residual32, out_f32=True, out_scale=self.residual_scale)


class GatedFeedForward(Part):
    """y = Wd (act(Wg x) * (Wu x)), no biases.  params: inner (int), activation (a name the elementwise kernels
    know), residual_scale (float, default 1).  names: gate, up [inner, hidden], down [hidden, inner].
    Gate and up are one product; ``forward(..., residual32=None)`` returns the float result alone.
    The reference has no gated feed-forward."""

    raw_output_ok = True

    def __init__(self, spec, hidden_size, dtype):
        super().__init__(spec, hidden_size, dtype)
        self.inner = int(self.param("inner"))
        self.activation = str(self.param("activation", "silu"))
        if self.activation not in K.ACTIVATIONS:
            raise ValueError(f"feed-forward activation {self.activation!r} has no kernel; "
                             f"available: {sorted(K.ACTIVATIONS)}")
        self.residual_scale = float(spec.params.get("residual_scale", 1.0))
        self.w_gate_up = self.w_down = None

    def tensor_specs(self) -> List[TensorSpec]:
        H, F = self.hidden_size, self.inner
        return [TensorSpec(self.name("gate"), (F, H), "matrix"), TensorSpec(self.name("up"), (F, H), "matrix"),
                TensorSpec(self.name("down"), (H, F), "matrix")]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.w_gate_up = torch.cat([tensors[self.name("gate")], tensors[self.name("up")]], dim=0).contiguous()
        self.w_down = tensors[self.name("down")]

    def forward(self, x_t, residual32, ctx, norm=None):
        F = self.inner
        gu = K.gemm(x_t, self.w_gate_up)
        h = K.activation_multiply(gu[:, :F], gu[:, F:], self.activation)
        return K.gemm(h, self.w_down, residual=residual32, out_f32=True, out_scale=self.residual_scale)
