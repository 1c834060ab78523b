"""Position encodings.

``LearnedPositions``: a table of position vectors added to the token embedding;
the row for position p is ``p + offset``.  The reference strips the first
``offset`` = 2 rows of OPT's table when converting (scripts/lib/converter_lib.py:271)
and indexes by p (src/csrc/kernel/embedding.cu:25-35); the table stays whole here.
``NoPositions``: nothing is added (the reference passes a null table for rotary
models, src/csrc/model/gpt/gpt.cc:138).
``RotaryPositions``: queries and keys are turned by an angle that grows with the position
(the reference's rotary kernel turns neighbouring pairs, src/csrc/kernel/rotary_posi_embedding.cu;
here coordinate i pairs with i + dims/2, only the first ``dims`` coordinates of a head turn, and
the frequencies may be rescaled for contexts longer than the model was trained on)."""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

from ..ops import kernels as K

from ..weights.loader import TensorSpec
from .base import PositionEncoding


class LearnedPositions(PositionEncoding):
    """params: max_positions (int), offset (int)."""

    def __init__(self, spec, hidden_size, dtype):
        super().__init__(spec, hidden_size, dtype)
        self.max_positions = int(self.param("max_positions"))
        self.offset = int(spec.params.get("offset", 0))
        self.table = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec(self.name("weight"), (self.max_positions + self.offset, self.hidden_size),
                           "table")]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.table = tensors[self.name("weight")]

    def embedding_addend(self, ctx):
        """(table, row index tensor, constant added to the index)."""
        return self.table, ctx.positions, self.offset


class NoPositions(PositionEncoding):
    pass


def rotary_frequencies(dims: int, base: float, scaling: Optional[dict] = None):
    """(angles a position step for the dims / 2 pairs as float64 list, factor on cosine and sine).

    Plain: f_i = base^(-2i / dims).  With ``scaling`` = {factor, original, fast, slow} the frequencies
    are blended between f_i (pairs that turn more than ``fast`` times within ``original`` positions keep
    theirs) and f_i / factor (pairs that turn fewer than ``slow`` times), linearly in the pair's index
    between the two border indices d(fast) and d(slow), d(t) = dims ln(original / (2 pi t)) / (2 ln base);
    cosine and sine are then multiplied by 0.1 ln(factor) + 1.
    With ``scaling`` = {factor, original, low, high} the rule goes by a pair's wavelength l = 2 pi / f_i:
    l < original / high keeps f_i, l > original / low takes f_i / factor, and between the two
    s = (original / l - low) / (high - low) blends them, (1 - s) f_i / factor + s f_i; cosine and sine
    keep their size."""
    half = dims // 2
    f = [float(base) ** (-2.0 * i / dims) for i in range(half)]
    if not scaling:
        return f, 1.0
    if "low" in scaling and "high" in scaling:
        factor, orig = float(scaling["factor"]), float(scaling["original"])
        low, high = float(scaling["low"]), float(scaling["high"])
        out = []
        for fi in f:
            wave = 2.0 * math.pi / fi
            if wave < orig / high:
                out.append(fi)
            elif wave > orig / low:
                out.append(fi / factor)
            else:
                s = (orig / wave - low) / (high - low)
                out.append((1.0 - s) * fi / factor + s * fi)
        return out, 1.0
    factor, orig = float(scaling["factor"]), float(scaling["original"])
    border = lambda turns: dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(border(float(scaling["fast"]))), 0)
    hi = min(math.ceil(border(float(scaling["slow"]))), dims - 1)
    out = []
    for i in range(half):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f[i] / factor * ramp + f[i] * (1.0 - ramp))
    return out, 0.1 * math.log(factor) + 1.0


class RotaryPositions(PositionEncoding):
    """params: head_dim (int), dims (int, even, <= head_dim: the coordinates of a head that turn), base
    (float), scaling (None, {factor, original, fast, slow} or {factor, original, low, high}: see
    ``rotary_frequencies``), interleaved (bool, default False: pairs are 2i, 2i + 1 instead of i, i + dims / 2).  It adds nothing to the embedding; mixers
    call ``rotate`` on their queries and keys.  Positions, angles, cosine and sine are float."""
    rotates = True

    def __init__(self, spec, hidden_size, dtype):
        super().__init__(spec, hidden_size, dtype)
        self.head_dim = int(self.param("head_dim"))
        self.dims = int(self.param("dims"))
        if self.dims % 2 or not 0 < self.dims <= self.head_dim:
            raise ValueError(f"rotary dims must be even and at most the head size {self.head_dim}, got {self.dims}")
        self.interleaved = bool(spec.params.get("interleaved", False))
        freq, self.mult = rotary_frequencies(self.dims, float(self.param("base")), spec.params.get("scaling"))
        self._freq_host = torch.tensor(freq, dtype=torch.float64).to(torch.float32)
        self.freq: Optional[torch.Tensor] = None

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        for t in tensors.values():
            self.freq = self._freq_host.to(t.device)
            break

    def rotate(self, q, k, ctx) -> None:
        if self.freq is None or self.freq.device != q.device:
            self.freq = self._freq_host.to(q.device)
        K.rotary(q, k, self.head_dim, self.freq, self.mult, ctx.positions, interleaved=self.interleaved)
