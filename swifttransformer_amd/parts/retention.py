"""Retention: linear attention with one fixed decay a head and neither softmax nor denominator.

    q = Wq x, k = Wk x * key_dim^-1/2, v = Wv x              (heads x key_dim, heads x value_dim)
    S_t = decay_h S_(t-1) + k_t v_t^T;  o_t = S_t^T q_t      (S float, one per request and head)
    y = Wo (concat_h(o_h / rms(o_h)) * silu(Wg x))

The state lives in the request's state slot and is carried from step to step.  Steps of single tokens and
small steps run ``state_scan`` in its additive form (its two gates one row of constants: key_dim^-1/2 and
the head's decay); steps of ``chunked_from`` rows or more that hold prompts or portions run
``retention_chunks``: because the decay does not change over time, a chunk's own sums need no state and the
chunks run side by side, with a carry of the state between them.  q, k and v leave their product as floats; the state,
the sums over it and the heads' unit norm are float.

Variants by parameter: an activation on q, k and v right after their product (``qkv_activation``), another
factor on the keys (``key_scale``), the norm over all heads' read-outs together with a gain an element in
the place of a unit norm a head (``norm`` = "all"), and a sigmoid gate in silu's place (``gate``).  With
silu(q), silu(k), silu(v), no key factor, the norm over all heads and a sigmoid gate this is lightning
attention with a fixed decay a head.  The reference has no such mixer."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..ops import kernels as K
from ..weights.loader import TensorSpec
from .base import CacheNeed, Mixer


class Retention(Mixer):
    """params: num_heads, key_dim, value_dim, decay (list of floats, one a head), eps (float, of the heads'
    unit norm), out_scale (float, default 1: a factor on the result), qkv_activation (default "none"), key_scale
    (float, default key_dim^-1/2), norm ("head", the default: each head's read-out at unit root mean square; "all":
    the heads' read-outs normalised together, times the tensor ``norm`` [heads * value_dim]), gate ("silu", the
    default, or "sigmoid")."""

    raw_output_ok = True
    chunked_from = 64          # rows of a step from which prompts and portions take the chunked kernels

    def __init__(self, spec, hidden_size, dtype):
        super().__init__(spec, hidden_size, dtype)
        self.num_heads = int(self.param("num_heads"))
        self.key_dim = int(self.param("key_dim"))
        self.value_dim = int(self.param("value_dim"))
        self.decay = [float(d) for d in self.param("decay")]
        self.eps = float(self.param("eps"))
        self.out_scale = float(spec.params.get("out_scale", 1.0))
        self.qkv_activation = str(spec.params.get("qkv_activation", "none"))
        self.key_scale = float(spec.params.get("key_scale", float(self.key_dim) ** -0.5))
        self.norm_over = str(spec.params.get("norm", "head"))
        self.gate_kind = str(spec.params.get("gate", "silu"))
        if self.qkv_activation not in K.ACTIVATIONS or self.norm_over not in ("head", "all") or \
                self.gate_kind not in ("silu", "sigmoid"):
            raise ValueError(f"retention: activation {self.qkv_activation!r}, norm {self.norm_over!r}, gate {self.gate_kind!r}")
        if len(self.decay) != self.num_heads:
            raise ValueError(f"{len(self.decay)} decays for {self.num_heads} heads")
        if self.key_dim > 256:
            raise ValueError(f"the scan takes up to 256 key channels a head, not {self.key_dim}")
        self.qk_size = self.num_heads * self.key_dim
        self.v_size = self.num_heads * self.value_dim

    def tensor_specs(self) -> List[TensorSpec]:
        H = self.hidden_size
        return [TensorSpec(self.name("q"), (self.qk_size, H), "matrix"),
                TensorSpec(self.name("k"), (self.qk_size, H), "matrix"),
                TensorSpec(self.name("v"), (self.v_size, H), "matrix"),
                TensorSpec(self.name("gate"), (self.v_size, H), "matrix"),
                TensorSpec(self.name("out"), (H, self.v_size), "matrix")] + (
                   [TensorSpec(self.name("norm"), (self.v_size,), "vector", init="gain")] if self.norm_over == "all" else [])

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        t = lambda n: tensors[self.name(n)]
        # q | k | v in one product whose results stay float; the gate in one of the storage type
        self.w_qkv = torch.cat([t("q"), t("k"), t("v")], dim=0).contiguous()
        self.w_gate, self.w_out = t("gate"), t("out")
        dev = self.w_out.device
        self.key_factor = torch.full((1, self.num_heads), self.key_scale, dtype=torch.float32, device=dev)
        self.decays = torch.tensor([self.decay], dtype=torch.float64).to(torch.float32).to(dev)
        self.decay_row = self.decays[0].contiguous()
        self.gain = (t("norm") if self.norm_over == "all" else
                     torch.ones(self.value_dim, dtype=torch.float32, device=dev))

    def cache_need(self) -> CacheNeed:
        return CacheNeed("state", state_shape=(self.num_heads, self.key_dim, self.value_dim),
                         state_dtype=torch.float32)

    def forward(self, x_t: torch.Tensor, residual32: Optional[torch.Tensor], ctx, cache, write: bool = True) -> torch.Tensor:
        if not write:
            raise ValueError("a recurrent mixer has no read-only run: its state moves with every token")
        qk = self.qk_size
        items = (ctx.token_item, ctx.item_len, ctx.item_tok_off, ctx.item_slot)
        qkv = K.gemm(x_t, self.w_qkv, out_f32=True, activation=self.qkv_activation)
        gate = K.gemm(x_t, self.w_gate)
        if not ctx.all_single and x_t.shape[0] >= self.chunked_from:
            o = K.retention_chunks(qkv[:, :qk], qkv[:, qk:2 * qk], qkv[:, 2 * qk:], self.decay_row,
                                   self.key_scale, cache.state, items, self.num_heads)
        else:
            o = K.state_scan(qkv[:, :qk], qkv[:, qk:2 * qk], qkv[:, 2 * qk:], self.key_factor, self.decays, cache.state,
                             items, self.num_heads, "additive", max_item_rows=1 if ctx.all_single else 0)
        y = K.gated_group_norm(o, gate, self.gain, self.num_heads if self.norm_over == "head" else 1, self.eps,
                               self.dtype, gate_kind=self.gate_kind)
        return K.gemm(y, self.w_out, residual=residual32, out_f32=True, out_scale=self.out_scale)
