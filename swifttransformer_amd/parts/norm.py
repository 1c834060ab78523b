"""LayerNorm over the hidden dimension.

Formula (reference src/csrc/kernel/layernorm.cu:35-97): mean and variance over
the row, y = (x - mean) * rsqrt(var + eps) * gamma + beta.  The reference forms
the two sums in float and normalises in the storage type; here the whole
computation is in float on the float residual stream, with the variance taken
from centred values.  The parameter ``center`` = False gives the form that takes no mean
off, y = x * rsqrt(mean(x^2) + eps) * gamma (+ beta) (reference src/csrc/kernel/rmsnorm.cu):
the same kernels and the same fusion into a product, by a flag.

``DynamicTanh`` is a norm that takes no statistics of the row at all: y = tanh(alpha x) * w + b per
element, alpha one learned number.  It can also add its result to a stream on the way
(``forward_onto``), which is how a branch's result is normalised as it enters the residual stream.
The reference has no such part."""
from __future__ import annotations

from typing import Dict, List, Optional, Tuple

import torch

from ..ops import kernels as K
from ..ops.tuning import tuning
from ..weights.loader import TensorSpec
from .base import Part

class LayerNorm(Part):
    """params: eps (float), affine (bool), center (bool, default True; False: root-mean-square norm),
    bias (bool, default = affine: whether the affine part has a bias), width (int, default hidden_size),
    scalar_gain (bool, default False: the file holds one number that multiplies every coordinate)."""

    def __init__(self, spec, hidden_size, dtype):
        super().__init__(spec, hidden_size, dtype)
        self.eps = float(self.param("eps"))
        self.affine = bool(self.param("affine", True))
        self.center = bool(spec.params.get("center", True))
        self.has_bias = bool(spec.params.get("bias", self.affine)) and self.affine
        self.width = int(self.param("width", hidden_size))
        self.scalar_gain = bool(spec.params.get("scalar_gain", False))
        self.gamma: Optional[torch.Tensor] = None
        self.beta: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        if not self.affine:
            return []
        specs = [TensorSpec(self.name("weight"), () if self.scalar_gain else (self.width,), "vector", init="gain")]
        if self.has_bias:
            specs.append(TensorSpec(self.name("bias"), (self.width,), "vector"))
        return specs

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        if self.affine:
            self.gamma = tensors[self.name("weight")]
            if self.scalar_gain:       # the kernels take a gain per coordinate
                self.gamma = self.gamma.reshape(1).expand(self.width).contiguous()
            self.beta = tensors[self.name("bias")] if self.has_bias else None

    def fusable(self, rows: int, out_features: int) -> bool:
        """Whether a product with ``out_features`` outputs can take this norm as its prologue."""
        return (rows <= tuning.fused_norm_max_rows and self.width <= tuning.fused_norm_max_width and
                K.can_fuse_norm(rows, out_features, self.width, self.dtype))

    def as_input(self, x32: torch.Tensor, rows: Optional[torch.Tensor] = None) -> "K.NormInput":
        """This norm of ``x32`` (of its rows ``rows``, int32 on the device) as the input of a product."""
        return K.NormInput(x32, self.gamma, self.beta, self.eps, rows, self.center)

    def forward(self, x32: torch.Tensor, *, out_t: bool = True, out_f32: bool = False,
                rows: Optional[torch.Tensor] = None) -> Tuple[Optional[torch.Tensor], Optional[torch.Tensor]]:
        n = rows.shape[0] if rows is not None else x32.shape[0]
        yt = K.empty((n, self.width), self.dtype, x32.device) if out_t else None
        y32 = K.empty((n, self.width), torch.float32, x32.device) if out_f32 else None
        if self.dtype == torch.float32 and out_t and out_f32:
            # one float result serves as both
            K.layernorm(x32, self.gamma, self.beta, self.eps, rows=rows, out_f32=y32, center=self.center)
            return y32, y32
        K.layernorm(x32, self.gamma, self.beta, self.eps, rows=rows, out_t=yt, out_f32=y32, center=self.center)
        return yt, y32


class DynamicTanh(Part):
    """params: width (int, default hidden_size), bias (bool, default True).  names: weight, bias, alpha
    (a tensor of no dimensions)."""

    chains_onto = True      # forward_onto(..., then=another of this kind / cast=True) makes a second result in its pass

    def __init__(self, spec, hidden_size, dtype):
        super().__init__(spec, hidden_size, dtype)
        self.width = int(self.param("width", hidden_size))
        self.has_bias = bool(spec.params.get("bias", True))
        self.gamma = self.beta = self.alpha = None

    def tensor_specs(self) -> List[TensorSpec]:
        specs = [TensorSpec(self.name("weight"), (self.width,), "vector", init="gain"),
                 TensorSpec(self.name("alpha"), (), "vector", init="gain")]
        if self.has_bias:
            specs.append(TensorSpec(self.name("bias"), (self.width,), "vector"))
        return specs

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.gamma = tensors[self.name("weight")]
        self.alpha = tensors[self.name("alpha")].reshape(1).contiguous()
        self.beta = tensors[self.name("bias")] if self.has_bias else None

    def forward(self, x32: torch.Tensor, *, out_t: bool = True, out_f32: bool = False,
                rows: Optional[torch.Tensor] = None) -> Tuple[Optional[torch.Tensor], Optional[torch.Tensor]]:
        n = rows.shape[0] if rows is not None else x32.shape[0]
        if self.dtype == torch.float32 and out_t and out_f32:
            out_t = False                                   # one float result serves as both
            both = True
        else:
            both = False
        yt = K.empty((n, self.width), self.dtype, x32.device) if out_t else None
        y32 = K.empty((n, self.width), torch.float32, x32.device) if out_f32 else None
        K.dynamic_tanh(x32, self.gamma, self.beta, self.alpha, rows=rows, out_t=yt, out_f32=y32)
        return (y32, y32) if both else (yt, y32)

    def forward_onto(self, y32: torch.Tensor, stream32: torch.Tensor, then=None, cast: bool = False):
        """stream32 + norm(y32), float, a new tensor.  ``then`` (another ``DynamicTanh``): returns (the sum, that
        norm of the sum in the storage type), made in the same pass; ``cast``: (the sum, the sum in the storage
        type)."""
        out = K.empty(tuple(stream32.shape), torch.float32, stream32.device)
        if then is None and not cast:
            K.dynamic_tanh(y32, self.gamma, self.beta, self.alpha, out_f32=out, base=stream32)
            return out
        if self.dtype == torch.float32 and then is None:
            K.dynamic_tanh(y32, self.gamma, self.beta, self.alpha, out_f32=out, base=stream32)
            return out, out
        out_t = K.empty(tuple(stream32.shape), self.dtype, stream32.device)
        K.dynamic_tanh(y32, self.gamma, self.beta, self.alpha, out_f32=out, out_t=out_t, base=stream32,
                       then=None if then is None else (then.gamma, then.beta, then.alpha))
        return out, out_t
