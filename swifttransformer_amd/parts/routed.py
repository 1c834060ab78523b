"""A feed-forward of routed experts: every token passes through ``top`` of ``experts`` small gated
layers, chosen by a router.

    z = Wr x (float);  s = sigmoid(z);  the ``top`` largest s choose the experts
    expert e on its input u = s_e x:  g = min(Wg u, limit),  h = clamp(Wu u, -limit, limit),
                                      y = g * sigmoid(1.702 g) * (h + 1),  result Wd y
    the token's result is the sum over its experts (the weights are not renormalised and multiply
    the expert's input, not its output)

or, ``style`` "softmax_output":

    z = Wr x + br (float);  the ``top`` largest z choose the experts;  s = softmax over the chosen z alone
    expert e:  Wd (silu(Wg x) * (Wu x));  the token's result is sum_e s_e expert_e(x)

or, ``style`` "softmax_all":

    z = Wr x (float);  s = softmax(z) over all experts;  experts form ``groups`` equal groups of neighbours, a
    group ranks by its largest s, and the ``top`` largest s among the experts of the ``keep`` best groups choose
    the experts;  the token's result is sum_e s_e expert_e(x) with s as it is (not renormalised)

Routing, sorting by expert and the experts' products all run on the device with launch shapes
that depend on the number of rows only, so steps with this part are recorded like any other
(``csrc/moe.hip``).  The reference has no such part."""
from __future__ import annotations

from typing import Dict, List

import torch

from ..ops import kernels as K
from ..weights.loader import TensorSpec
from .base import Part


class RoutedExperts(Part):
    """params: experts (int), top (int), inner (int: width inside an expert), limit (float, of the
    "scaled_input" style), residual_scale (float, default 1), style ("scaled_input", the default, or
    "softmax_output" or "softmax_all"), groups and keep (ints, default 1: of the "softmax_all" style),
    router_bias (bool, default False).  names: ``router`` (``router_bias``) and the
    patterns ``gate``, ``up``, ``down`` with ``{e}`` for the expert's number."""

    raw_output_ok = True     # with the softmax styles, forward(..., residual32=None) returns the sum alone

    def __init__(self, spec, hidden_size, dtype):
        super().__init__(spec, hidden_size, dtype)
        self.experts = int(self.param("experts"))
        self.top = int(self.param("top"))
        self.inner = int(self.param("inner"))
        self.style = str(spec.params.get("style", "scaled_input"))
        self.limit = float(self.param("limit")) if self.style == "scaled_input" else 0.0
        self.router_bias = bool(spec.params.get("router_bias", False))
        self.groups = int(spec.params.get("groups", 1) or 1)
        self.keep = int(spec.params.get("keep", self.groups) or self.groups)
        if self.experts % self.groups or not 1 <= self.keep <= self.groups or self.groups > 64:
            raise ValueError(f"{self.experts} experts in {self.groups} equal groups (up to 64) of which {self.keep} are kept")
        if self.style == "softmax_all" and int(self.param("top")) > self.keep * (self.experts // self.groups):
            raise ValueError(f"{self.param('top')} experts a token do not fit {self.keep} groups")
        self.residual_scale = float(spec.params.get("residual_scale", 1.0))
        if not 1 <= self.top <= min(self.experts, 16):
            raise ValueError(f"1 to 16 of {self.experts} experts a token, not {self.top}")

    def _expert(self, which: str, e: int) -> str:
        return self.name(which).format(e=e)

    def tensor_specs(self) -> List[TensorSpec]:
        H, F = self.hidden_size, self.inner
        specs = [TensorSpec(self.name("router"), (self.experts, H), "matrix")]
        if self.router_bias:
            specs.append(TensorSpec(self.name("router_bias"), (self.experts,), "vector"))
        for e in range(self.experts):
            specs += [TensorSpec(self._expert("gate", e), (F, H), "matrix"),
                      TensorSpec(self._expert("up", e), (F, H), "matrix"),
                      TensorSpec(self._expert("down", e), (H, F), "matrix")]
        return specs

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.w_router = tensors[self.name("router")]
        self.b_router = tensors[self.name("router_bias")] if self.router_bias else None
        stack = lambda which: torch.stack([tensors[self._expert(which, e)] for e in range(self.experts)]).contiguous()
        self.w_gate, self.w_up, self.w_down = stack("gate"), stack("up"), stack("down")

    def forward(self, x_t: torch.Tensor, residual32: torch.Tensor, ctx) -> torch.Tensor:
        logits = K.gemm(x_t, self.w_router, bias=self.b_router, out_f32=True)
        return K.routed_experts(x_t, logits, self.w_gate, self.w_up, self.w_down, residual32, top=self.top,
                                limit=self.limit, out_scale=self.residual_scale, token_item=ctx.token_item,
                                style=self.style, groups=self.groups, keep=self.keep)
