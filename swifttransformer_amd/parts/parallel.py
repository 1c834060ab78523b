"""Two mixers side by side: both read the same input, and their results are added.

    y = left(x) + right(x)          (a factor on either result is that mixer's own ``out_scale``)

Each branch is a mixer part of its own kind with caches of its own; the pair reports them under the
names "left" and "right" (a branch that keeps several caches itself: "left.<its name>").  The second
branch adds its result onto the first's in its output product's epilogue, so the sum costs no kernel.
The reference has no such mixer."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..weights.loader import TensorSpec
from .base import CacheNeed, Mixer, build_part


class ParallelMixers(Mixer):
    """params: left, right (``PartSpec`` of a mixer each)."""

    raw_output_ok = True

    def __init__(self, spec, hidden_size, dtype):
        super().__init__(spec, hidden_size, dtype)
        self.branches = {side: build_part("mixer", self.param(side), hidden_size, dtype) for side in ("left", "right")}
        for side, m in self.branches.items():
            if not getattr(m, "raw_output_ok", False):
                raise ValueError(f"the {side} mixer cannot give its result without the residual stream")

    def use_position(self, position) -> None:
        super().use_position(position)
        for m in self.branches.values():
            if hasattr(m, "use_position"):
                m.use_position(position)

    @property
    def graph_safe(self) -> bool:
        return all(getattr(m, "graph_safe", False) for m in self.branches.values())

    def tensor_specs(self) -> List[TensorSpec]:
        return [s for m in self.branches.values() for s in m.tensor_specs()]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        for m in self.branches.values():
            m.bind(tensors)

    def cache_parts(self) -> Dict[str, CacheNeed]:
        parts: Dict[str, CacheNeed] = {}
        for side, m in self.branches.items():
            if hasattr(m, "cache_parts"):
                parts.update({f"{side}.{name}": need for name, need in m.cache_parts().items()})
            else:
                need = m.cache_need()
                if need is not None:
                    parts[side] = need
        return parts

    def _cache_of(self, side: str, cache):
        m = self.branches[side]
        if hasattr(m, "cache_parts"):
            return {name: cache[f"{side}.{name}"] for name in m.cache_parts()}
        return cache.get(side)

    def forward(self, x_t: torch.Tensor, residual32: Optional[torch.Tensor], ctx, cache, write: bool = True) -> torch.Tensor:
        y32 = self.branches["left"].forward(x_t, residual32, ctx, self._cache_of("left", cache), write)
        return self.branches["right"].forward(x_t, y32, ctx, self._cache_of("right", cache), write)
