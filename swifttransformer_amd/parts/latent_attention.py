"""Attention whose keys and values are linear functions of one cached latent vector per token.

    q = Wq x                                   (heads x key_dim)
    c = rmsnorm(Wdkv x) * gain                 (rank; the only thing that is cached)
    k_h = Wuk_h c, v_h = Wuv_h c;  score = (q_h . k_h) * scale;  causal softmax;  y = Wo [o_1 .. o_H]

Because k and v are linear in c, the two up-projections are folded into the neighbouring
products when the weights are bound: q'_h = Wuk_h^T Wq_h x scores against c itself, the
weighted sum of the c's is what Wo_h Wuv_h then maps to the output.  What is left is attention
with one shared key/value head whose keys and values are the same vectors, which the paged
attention kernels of ``PagedAttention`` run as they are: the pool has no second half
(``CacheNeed(values=False)``), and a layer may read the latent cache of an earlier layer
(``ScheduleEntry(cache=j, write=False)``) with up-projections of its own.  The latent's norm is
float, straight from the product's float result, and is written to its page by the same kernel.

Optionally (``rot_dim`` > 0) a query head is [key_dim plain | rot_dim turned] and the down-projection
has rot_dim more rows, one small key part that all heads share; both are turned by the token's
position (pairs 2i, 2i + 1) and score = (q_plain . k_h + q_turned . k_shared) * scale.  The shared
part is cached behind the latent in the same entry, so the folded query is [Wuk_h^T q_plain | q_turned]
against [c | k_shared], and the folded output matrix has zero columns where the shared part lies:
still one shared head whose keys are its values.  ``window`` > 0: a row sees itself and the window - 1
tokens before it; pages behind the window are given back.  The reference has no such mixer."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..ops import kernels as K
from ..weights.loader import TensorSpec
from .attention import PagedAttention
from .base import CacheNeed
from .position import rotary_frequencies


class LatentAttention(PagedAttention):
    """params: num_heads, key_dim, value_dim, rank, scale (float), eps (float, of the latent's norm),
    own_latent (bool, default True; False: the layer reads another layer's cache and has no
    down-projection), residual_scale (float, default 1), tile_min_len (as ``PagedAttention``), rot_dim
    (int, default 0: the turned part of a query head and the shared turned key part), rot_dims (int, default
    rot_dim: how many of its coordinates turn, the first ones), rot_base (float), rot_scaling (None or a rule of ``rotary_frequencies``), window (int, default 0: all keys)."""

    raw_output_ok = True     # forward(..., residual32=None) returns the mixer's result alone

    def __init__(self, spec, hidden_size, dtype):
        p = spec.params
        self.rank = int(p["rank"])
        self.rot_dim = int(p.get("rot_dim", 0) or 0)
        if self.rot_dim % 2:
            raise ValueError(f"the turned part of a head has an even size, not {self.rot_dim}")
        self.entry = -(-(self.rank + self.rot_dim) // 16) * 16     # the attention kernels take multiples of 16
        if self.entry > 256:
            raise ValueError(f"the attention kernels take cached vectors of up to 256 numbers, not "
                             f"{self.rank} + {self.rot_dim}")
        from .spec import PartSpec
        as_paged = PartSpec(spec.kind, dict(p, num_kv_heads=1, head_dim=self.entry, bias=False,
                                            window=int(p.get("window", 0) or 0)), spec.names)
        super().__init__(as_paged, hidden_size, dtype)
        self.spec = spec
        self.key_dim = int(p["key_dim"])
        self.value_dim = int(p["value_dim"])
        self.eps = float(p["eps"])
        self.own_latent = bool(p.get("own_latent", True))
        self.residual_scale = float(p.get("residual_scale", 1.0))
        if self.rot_dim and not self.own_latent:
            raise ValueError("a latent attention with a turned key part caches it with its own latent")
        self._freq_host = self.freq = None
        self.rot_mult = 1.0
        if self.rot_dim:
            dims = int(p.get("rot_dims", self.rot_dim) or self.rot_dim)
            if dims % 2 or not 0 < dims <= self.rot_dim:
                raise ValueError(f"{dims} turning coordinates in a part of {self.rot_dim}")
            # (a rule that also scales cosine and sine scales the turned parts of queries and keys alike)
            freq, self.rot_mult = rotary_frequencies(dims, float(p["rot_base"]), p.get("rot_scaling"))
            freq = list(freq) + [0.0] * ((self.rot_dim - dims) // 2)      # an angle of zero leaves a pair as it is
            self._freq_host = torch.tensor(freq, dtype=torch.float64).to(torch.float32)

    def tensor_specs(self) -> List[TensorSpec]:
        H, nh = self.hidden_size, self.num_heads
        specs = [TensorSpec(self.name("q"), (nh * (self.key_dim + self.rot_dim), H), "matrix"),
                 TensorSpec(self.name("up_k"), (nh * self.key_dim, self.rank), "matrix"),
                 TensorSpec(self.name("up_v"), (nh * self.value_dim, self.rank), "matrix"),
                 TensorSpec(self.name("out"), (H, nh * self.value_dim), "matrix")]
        if self.own_latent:
            specs += [TensorSpec(self.name("down"), (self.rank + self.rot_dim, H), "matrix"),
                      TensorSpec(self.name("down_norm"), (self.rank,), "vector", init="gain")]
        return specs

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        t = lambda n: tensors[self.name(n)]
        H, nh, R, E = self.hidden_size, self.num_heads, self.rank, self.entry
        wide = torch.float64
        wq_all = t("q").to(wide).view(nh, self.key_dim + self.rot_dim, H)
        wq = wq_all[:, :self.key_dim]
        uk = t("up_k").to(wide).view(nh, self.key_dim, R)
        uv = t("up_v").to(wide).view(nh, self.value_dim, R)
        wo = t("out").to(wide).view(H, nh, self.value_dim)
        # queries against the latent itself: per head Wuk^T Wq, [heads * entry, hidden]
        w_q = torch.zeros((nh, E, H), dtype=wide, device=wq.device)
        w_q[:, :R] = torch.einsum("hdr,hdk->hrk", uk, wq)
        if self.rot_dim:           # the turned part of a query meets the shared key part behind the latent
            w_q[:, R:R + self.rot_dim] = wq_all[:, self.key_dim:]
            self.freq = self._freq_host.to(wq.device)
        # the weighted latents to the output: per head Wo_h Wuv_h, [hidden, heads * entry]
        w_o = torch.zeros((H, nh, E), dtype=wide, device=wq.device)
        w_o[:, :, :R] = torch.einsum("khv,hvr->khr", wo, uv)
        self.w_q = w_q.view(nh * E, H).to(self.dtype).contiguous()
        self.w_out = w_o.view(H, nh * E).to(self.dtype).contiguous()
        if self.own_latent:
            self.w_down, self.gain = t("down"), t("down_norm")

    def cache_need(self) -> Optional[CacheNeed]:
        return CacheNeed("paged_kv", num_kv_heads=1, head_dim=self.entry, window=self.window, values=False)

    accepts_norm = False

    def forward(self, x_t: torch.Tensor, residual32: Optional[torch.Tensor], ctx, cache, write: bool = True,
                norm=None) -> torch.Tensor:
        if write != self.own_latent:
            raise ValueError("a latent attention writes the cache it owns and only reads a borrowed one")
        if write:
            raw = K.gemm(x_t, self.w_down, out_f32=True)
            K.latent_write(cache.k, raw, self.gain, self.eps, ctx.token_item, ctx.positions,
                           ctx.block_tables[cache.group], tail=self.rot_dim, tail_freq=self.freq, tail_mult=self.rot_mult)
        q = K.gemm(x_t, self.w_q)
        if self.rot_dim:
            K.rotary(q, None, self.entry, self.freq, self.rot_mult, ctx.positions, offset=self.rank, interleaved=True)
        o = self.attend(q, ctx, cache, unmerged_ok=True)
        return K.gemm(o, self.w_out, residual=residual32, out_f32=True, out_scale=self.residual_scale)
