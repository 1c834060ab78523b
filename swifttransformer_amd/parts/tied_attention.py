"""Grouped softmax attention whose values are its keys, with a norm over the whole query and key projections,
capped scores and, optionally, a mask of chunks.

    q = Wq x, k = Wk x                               (heads x head_dim, kv_heads x head_dim; no biases)
    q' = q * rsqrt(mean(q^2) + eps) * gq             (the mean over all heads' coordinates at once; the same for k')
    v = k                                            (the keys as projected, before their norm; there is no Wv)
    s = (q'_h . k'_g) * scale;  s <- cap * tanh(s / cap)
    position i sees j <= i with floor(i / chunk) = floor(j / chunk) (chunks counted from the sequence's start;
    chunk 0: every j <= i; or a sliding ``window``);  softmax;  y = Wo [o_1 .. o_H]

Positions do not enter the scores.  One product makes q and k as floats; one kernel normalises both, rounds
the queries to the storage type and writes the normalised keys into the key pool and the raw keys into the
value pool; the paged attention kernels of ``PagedAttention`` (rows and tiles) then run with a cap on the
scores and the chunk's first position as each row's lower bound.  Heads of a size that is no multiple of 16
are padded with zeros in queries and pools, and the output matrix gets zero columns there.  Pages of chunks
that no later row reads are kept until the request ends.  The reference has no such mixer."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..ops import kernels as K
from ..weights.loader import TensorSpec
from .attention import PagedAttention
from .base import CacheNeed
from .spec import PartSpec


class TiedKeyValueAttention(PagedAttention):
    """params: num_heads, num_kv_heads, head_dim, scale (float), eps (float, of the two norms), softcap (float,
    default 0 = none), chunk (int, default 0 = none), window (int, default 0; not together with chunk),
    tile_min_len (as ``PagedAttention``).  names: q, k, q_norm, k_norm, out."""

    raw_output_ok = True
    accepts_norm = False

    def __init__(self, spec, hidden_size, dtype):
        p = spec.params
        self.dim = int(p["head_dim"])
        self.pad = -(-self.dim // 16) * 16
        super().__init__(PartSpec(spec.kind, dict(p, head_dim=self.pad, bias=False), spec.names), hidden_size, dtype)
        self.spec = spec
        self.eps = float(p["eps"])
        self.softcap = float(p.get("softcap", 0.0) or 0.0)
        self.chunk = int(p.get("chunk", 0) or 0)
        if self.chunk and self.window:
            raise ValueError("an attention has chunks or a window, not both")
        if self.softcap < 0 or self.chunk < 0:
            raise ValueError(f"softcap {self.softcap} and chunk {self.chunk} must not be negative")
        # the kernels' one mask parameter: a window as it is, chunks as a negative number
        self.mask = -self.chunk if self.chunk else self.window

    def tensor_specs(self) -> List[TensorSpec]:
        H, nq, nk = self.hidden_size, self.num_heads * self.dim, self.num_kv_heads * self.dim
        return [TensorSpec(self.name("q"), (nq, H), "matrix"), TensorSpec(self.name("k"), (nk, H), "matrix"),
                TensorSpec(self.name("q_norm"), (nq,), "vector", init="gain"),
                TensorSpec(self.name("k_norm"), (nk,), "vector", init="gain"),
                TensorSpec(self.name("out"), (H, nq), "matrix")]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        t = lambda n: tensors[self.name(n)]
        self.w_qk = torch.cat([t("q"), t("k")], dim=0).contiguous()
        self.gain_q, self.gain_k = t("q_norm"), t("k_norm")
        w_out = t("out")
        if self.pad != self.dim:       # zero columns where the heads are padded
            H = self.hidden_size
            wide = torch.zeros((H, self.num_heads, self.pad), dtype=w_out.dtype, device=w_out.device)
            wide[:, :, :self.dim] = w_out.view(H, self.num_heads, self.dim)
            w_out = wide.view(H, self.num_heads * self.pad).contiguous()
        self.w_out = w_out

    def cache_need(self) -> CacheNeed:
        # (with chunks every page stays: only a window gives pages back)
        return CacheNeed("paged_kv", num_kv_heads=self.num_kv_heads, head_dim=self.pad, window=self.window)

    def plan_key(self):
        return ("attention_tiles", self.tile_min_len, self.num_heads, self.pad, self.dtype, True)

    def step_planner(self):
        n = self.tile_min_len

        def planner(items, info):
            from .attention import plan_tiles
            return plan_tiles(items, n, K.PREFILL_TILE, bucketed=info.bucketed)     # (capped scores: tiles of 64 rows)
        return self.plan_key(), planner

    def forward(self, x_t: torch.Tensor, residual32: Optional[torch.Tensor], ctx, cache, write: bool = True,
                norm=None) -> torch.Tensor:
        qk = K.gemm(x_t, self.w_qk, out_f32=True)
        bt = ctx.block_tables[cache.group]
        q = K.qk_norm_write(qk, self.gain_q, self.gain_k, self.eps, self.num_heads, self.num_kv_heads, self.dim,
                            cache.k, cache.v, ctx.token_item, ctx.positions, bt, write=write)
        T = q.shape[0]
        out = K.empty((T, self.q_size), self.dtype, q.device)
        plan = ctx.plans.get(self.plan_key())
        if plan is not None and K.prefill_available():
            K.attention_prefill(q, cache.k, cache.v, plan.arrays["tile_item"], plan.arrays["tile_q0"],
                                ctx.item_tok_off, ctx.item_start, ctx.item_len, bt, self.num_heads, self.scale,
                                window=self.mask, out=out, tile_rows=plan.host["tile_rows"], softcap=self.softcap)
            if plan.host["num_short_rows"] > 0:
                splits, waves = self._shape_row_kernel(ctx, plan.host["num_short_rows"])
                K.attention_rows(q, cache.k, cache.v, ctx.token_item, ctx.positions, bt, self.num_heads, self.scale,
                                 window=self.mask, row_ids=plan.arrays["short_rows"], num_splits=splits,
                                 num_waves=waves, out=out, softcap=self.softcap)
        else:
            splits, waves = self._shape_row_kernel(ctx, T)
            K.attention_rows(q, cache.k, cache.v, ctx.token_item, ctx.positions, bt, self.num_heads, self.scale,
                             window=self.mask, num_splits=splits, num_waves=waves, out=out, softcap=self.softcap)
        return K.gemm(out, self.w_out, residual=residual32, out_f32=True)

    def key_span(self, ctx) -> int:
        return min(ctx.max_kv_len, self.chunk) if self.chunk else super().key_span(ctx)
