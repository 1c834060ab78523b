"""Grouped softmax attention with a short causal filter over time on its queries, keys and values, partial
rotary positions, a sliding window that keeps the first tokens, and a gate on the heads' outputs.

    q, k, v = conv(Wq x), conv(Wk x), conv(Wv x)            one filter a channel, no bias; optional
    q, k turned by the rotary part (v is not)
    p(i, j) = softmax_j(scale * q_h(i) . k_c(h)(j))         over j <= i with i - j < window or j < keep_first
    y = Wo (concat_h(sum_j p(i, j) v_c(h)(j)) * sigmoid(Wg x))

Keys and values live in pages of their own sizes; the filters' last ``taps - 1`` inputs a request are a
fixed-size state.  The two caches are named "kv" and "conv" (``cache_parts``).  A windowed cache gives
pages back as the window passes, except those of the first ``keep_first`` tokens.  One route serves
prompts, portions and decoded tokens: filter, turn, write the step's keys and values, then every row
attends over the cache (``sink_attention`` without sink and head mix).  Scores and the softmax are
float.  The reference has no such mixer (its attention is src/csrc/layer/attention.cc)."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..ops import kernels as K
from ..weights.loader import TensorSpec
from .base import CacheNeed, Mixer, build_part
from .sink_attention import K_fits


class GatedWindowAttention(Mixer):
    """params: num_heads, num_kv_heads, key_dim, value_dim, scale (float), window (int, 0: all keys),
    keep_first (int, default 0), taps (int, 0 or 1..8: the filter's length, 0: none), rotary (``PartSpec`` of
    a position part that rotates, or None), gate ("sigmoid", "silu" or None), out_scale (float, default 1: a
    factor on the result)."""

    raw_output_ok = True

    def __init__(self, spec, hidden_size, dtype):
        super().__init__(spec, hidden_size, dtype)
        self.num_heads = int(self.param("num_heads"))
        self.num_kv_heads = int(self.param("num_kv_heads", self.num_heads))
        self.key_dim = int(self.param("key_dim"))
        self.value_dim = int(self.param("value_dim", self.key_dim))
        self.scale = float(self.param("scale"))
        self.window = int(spec.params.get("window", 0) or 0)
        self.keep_first = int(spec.params.get("keep_first", 0) or 0) if self.window > 0 else 0
        self.taps = int(spec.params.get("taps", 0) or 0)
        self.gate = spec.params.get("gate", "sigmoid")
        self.out_scale = float(spec.params.get("out_scale", 1.0))
        if self.num_heads % self.num_kv_heads:
            raise ValueError(f"{self.num_heads} heads do not divide into {self.num_kv_heads} key heads")
        if self.taps > 8:
            raise ValueError(f"the convolution kernel takes 1 to 8 taps, not {self.taps}")
        if self.gate not in (None, "sigmoid", "silu"):
            raise ValueError(f"the gate on the heads' outputs is sigmoid, silu or None, not {self.gate!r}")
        if not K_fits(self.num_heads, self.key_dim, self.value_dim, False):
            raise ValueError(f"the attention kernel holds a row's queries and a block's scores in 64 KB of LDS and "
                             f"up to 8192 output coordinates a row: {self.num_heads} heads of {self.key_dim} / "
                             f"{self.value_dim} do not fit")
        rot = spec.params.get("rotary")
        self.rotary = build_part("position", rot, hidden_size, dtype) if rot is not None else None
        self.q_size = self.num_heads * self.key_dim
        self.k_size = self.num_kv_heads * self.key_dim
        self.v_size = self.num_kv_heads * self.value_dim
        self.o_size = self.num_heads * self.value_dim
        self.qkv_size = self.q_size + self.k_size + self.v_size

    def tensor_specs(self) -> List[TensorSpec]:
        H = self.hidden_size
        specs = [TensorSpec(self.name("q"), (self.q_size, H), "matrix"),
                 TensorSpec(self.name("k"), (self.k_size, H), "matrix"),
                 TensorSpec(self.name("v"), (self.v_size, H), "matrix"),
                 TensorSpec(self.name("out"), (H, self.o_size), "matrix")]
        if self.gate is not None:
            specs.append(TensorSpec(self.name("gate"), (self.o_size, H), "matrix"))
        if self.taps > 0:
            specs += [TensorSpec(self.name("q_conv"), (self.q_size, self.taps), "vector"),
                      TensorSpec(self.name("k_conv"), (self.k_size, self.taps), "vector"),
                      TensorSpec(self.name("v_conv"), (self.v_size, self.taps), "vector")]
        return specs

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        t = lambda n: tensors[self.name(n)]
        # q | k | v | gate stacked along the output dimension: one product makes all four
        rows = [t("q"), t("k"), t("v")] + ([t("gate")] if self.gate is not None else [])
        self.w_in = torch.cat(rows, dim=0).contiguous()
        self.w_conv = (torch.cat([t("q_conv"), t("k_conv"), t("v_conv")], dim=0).contiguous()
                       if self.taps > 0 else None)
        self.w_out = t("out")
        if self.rotary is not None:
            self.rotary.bind(tensors)

    def cache_parts(self) -> Dict[str, CacheNeed]:
        parts = {"kv": CacheNeed("paged_kv", num_kv_heads=self.num_kv_heads, head_dim=self.key_dim,
                                 window=self.window, keep_first=self.keep_first,
                                 value_dim=self.value_dim if self.value_dim != self.key_dim else 0)}
        if self.taps > 1:
            parts["conv"] = CacheNeed("state", state_shape=(self.taps - 1, self.qkv_size), state_dtype=torch.float32)
        return parts

    def _splits(self, ctx, rows: int) -> int:
        """Workgroups a row (see ``SinkAttention._splits``): a function of the rows and, for recorded
        steps, of nothing else."""
        span = ctx.max_kv_len if self.window <= 0 else min(ctx.max_kv_len, self.window + self.keep_first)
        blocks = max(1, -(-span // 64))
        return max(1, min(256 // max(rows, 1), blocks, 16))

    def forward(self, x_t: torch.Tensor, residual32: Optional[torch.Tensor], ctx, cache, write: bool = True) -> torch.Tensor:
        if not write:
            raise ValueError("this attention keeps a filter state that moves with every token: no read-only run")
        kv = cache["kv"]
        proj = K.gemm(x_t, self.w_in)                                  # q | k | v | gate
        qkv = proj[:, :self.qkv_size]
        if self.taps > 0:
            items = (ctx.token_item, ctx.item_len, ctx.item_tok_off, ctx.item_slot)
            state = cache["conv"].state if self.taps > 1 else proj[:0]
            qkv = K.token_conv(qkv, self.w_conv, state, items, self.dtype, add_input=False)
        q = qkv[:, :self.q_size]
        k = qkv[:, self.q_size:self.q_size + self.k_size]
        v = qkv[:, self.q_size + self.k_size:]
        if self.rotary is not None:
            self.rotary.rotate(q, k, ctx)
        bt = ctx.block_tables[kv.group]
        K.paged_write(kv.k, k, ctx.token_item, ctx.positions, bt)
        K.paged_write(kv.v, v, ctx.token_item, ctx.positions, bt)
        o = K.sink_attention(q, kv.k, kv.v, ctx.token_item, ctx.positions, bt, self.num_heads, self.scale,
                             window=self.window, keep_first=self.keep_first, sink=False, head_mix=None,
                             num_splits=self._splits(ctx, proj.shape[0]))
        if self.gate is not None:
            o = K.activation_multiply(proj[:, self.qkv_size:], o, self.gate)
        return K.gemm(o, self.w_out, residual=residual32, out_f32=True, out_scale=self.out_scale)
