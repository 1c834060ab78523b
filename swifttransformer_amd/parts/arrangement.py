"""How a layer's norms, mixer and feed-forward are wired around the residual stream.

pre-norm (reference src/csrc/model/gpt/gpt.cc:325-335, :347-391, :423-436, :467-501):
    a = N1(x); r = x + Mix(a); d = N2(r); x' = r + FFN(d)
    (optionally a = C(N1(x)) with C a short filter over time, and optionally without the second
    half; a factor on the branches is the mixer's and the feed-forward's own parameter)
post-norm (the reference refuses it, gpt.cc:238-240):
    r = N1(x + Mix(x)); x' = N2(r + FFN(r))
sandwich (norms before and after each sublayer; the reference has no such block):
    r = x + N1b(Mix(N1(x))); s = r + N2b(FFN(N2(r))); x' = s + Side(s, token)
    (the feed-forward and the side input are optional)
hyper-connections (several copies of the stream; the reference has no such block):
    u = sum_s a1[s] x_s;  y = Mix(N1(u));  x_t <- sum_s M1[s, t] x_s + b1[t] y   (all t at once)
    and the same with a2, M2, b2 around the feed-forward, which is optional
The residual stream is float; parts that multiply matrices take the storage type."""
from __future__ import annotations

import torch

from typing import Dict, List

from ..ops import kernels as K
from ..weights.loader import TensorSpec
from .base import Part


def _fuses(part, norm, rows: int) -> bool:
    """A part that accepts a norm and a norm that can be a product's prologue at this size."""
    return (getattr(part, "accepts_norm", False) and hasattr(norm, "fusable")
            and norm.fusable(rows, part.hidden_size))


class PreNorm(Part):
    """params: feed_forward (bool, default True; False: the block ends after the mixer).  A layer
    with a ``mixer_conv`` part has its mixer read conv(N1(x)) instead of N1(x)."""

    def __init__(self, spec, hidden_size, dtype):
        super().__init__(spec, hidden_size, dtype)
        self.has_ffn = bool(spec.params.get("feed_forward", True))
        # layer slots that must be filled
        self.needs = ("mixer_norm", "ffn_norm", "feed_forward") if self.has_ffn else ("mixer_norm",)

    def forward(self, x32: torch.Tensor, layer, ctx, cache, write: bool = True, conv_cache=None) -> torch.Tensor:
        rows = x32.shape[0]
        if layer.mixer_conv is not None:
            # the filter reads the float norm and makes the mixer's input in the storage type
            _, n32 = layer.mixer_norm.forward(x32, out_t=False, out_f32=True)
            a = layer.mixer_conv.forward(n32, ctx, conv_cache)
            r32 = layer.mixer.forward(a, x32, ctx, cache, write)
        elif _fuses(layer.mixer, layer.mixer_norm, rows):
            r32 = layer.mixer.forward(None, x32, ctx, cache, write, norm=layer.mixer_norm)
        else:
            a, _ = layer.mixer_norm.forward(x32, out_t=True)
            r32 = layer.mixer.forward(a, x32, ctx, cache, write)
        if not self.has_ffn:
            return r32
        if _fuses(layer.feed_forward, layer.ffn_norm, rows):
            return layer.feed_forward.forward(None, r32, ctx, norm=layer.ffn_norm)
        d, _ = layer.ffn_norm.forward(r32, out_t=True)
        return layer.feed_forward.forward(d, r32, ctx)


class PostNorm(Part):
    needs = ("mixer_norm", "ffn_norm", "feed_forward")

    def forward(self, x32: torch.Tensor, layer, ctx, cache, write: bool = True) -> torch.Tensor:
        x_t = x32 if self.dtype == torch.float32 else K.cast(x32, self.dtype)
        s32 = layer.mixer.forward(x_t, x32, ctx, cache, write)
        r_t, r32 = layer.mixer_norm.forward(s32, out_t=True, out_f32=True)
        u32 = layer.feed_forward.forward(r_t, r32, ctx)
        _, y32 = layer.ffn_norm.forward(u32, out_t=False, out_f32=True)
        return y32


class Sandwich(Part):
    """params: feed_forward (bool, default True).  The mixer and the feed-forward are asked for their
    results alone (``residual32`` None, which they must allow: ``raw_output_ok``); the norm after each adds
    its result to the stream (``forward_onto``).  A ``side_input`` part of the layer acts on the stream last."""

    def __init__(self, spec, hidden_size, dtype):
        super().__init__(spec, hidden_size, dtype)
        self.has_ffn = bool(spec.params.get("feed_forward", True))
        self.needs = (("mixer_norm", "mixer_out_norm", "ffn_norm", "feed_forward", "ffn_out_norm") if self.has_ffn
                      else ("mixer_norm", "mixer_out_norm"))

    def forward(self, x32: torch.Tensor, layer, ctx, cache, write: bool = True) -> torch.Tensor:
        for part in (layer.mixer, layer.feed_forward if self.has_ffn else None):
            if part is not None and not getattr(part, "raw_output_ok", False):
                raise ValueError(f"{type(part).__name__} cannot give its result without the residual stream")
        a, _ = layer.mixer_norm.forward(x32, out_t=True)
        m32 = layer.mixer.forward(a, None, ctx, cache, write)
        side = layer.side_input
        x_t = None                                  # the stream in the storage type, where a pass has made it
        if self.has_ffn:
            # norm after the mixer, the sum into the stream and the norm before the feed-forward: one pass where
            # the two norms can do that
            if _chains(layer.mixer_out_norm, layer.ffn_norm):
                x32, d = layer.mixer_out_norm.forward_onto(m32, x32, then=layer.ffn_norm)
            else:
                x32 = layer.mixer_out_norm.forward_onto(m32, x32)
                d, _ = layer.ffn_norm.forward(x32, out_t=True)
            f32 = layer.feed_forward.forward(d, None, ctx)
            last = layer.ffn_out_norm
        else:
            f32, last = m32, layer.mixer_out_norm
        if side is not None and not getattr(side, "fused", False) and _chains(last, None):
            x32, x_t = last.forward_onto(f32, x32, cast=True)
        else:
            x32 = last.forward_onto(f32, x32)
        if side is not None:
            x32 = side.forward(x32, ctx, x_t=x_t)
        return x32


def _chains(norm, then) -> bool:
    """Whether ``norm.forward_onto`` can make a second result in the same pass (``then``: another norm of its
    kind, or None for the plain sum in the storage type)."""
    return getattr(norm, "chains_onto", False) and (then is None or type(then) is type(norm))


class HyperConnections(Part):
    """params: streams (int), feed_forward (bool, default True).  names: ``mixer_in``, ``mixer_out`` (float
    [streams]), ``mixer_mix`` ([streams, streams], indexed [from, to]) and ``ffn_in``, ``ffn_out``, ``ffn_mix``.

    The stream it is handed is float [T, streams * hidden]: the model makes the copies after the embedding
    and sums them before the final norm (``ModelSpec.streams``).  It is updated in place.  The sublayers are
    asked for their results alone (``raw_output_ok``).  Where a norm is the root-mean-square form with a gain,
    the weighted sum of the streams and the norm are one kernel, and the write after the mixer makes the
    feed-forward's input in the same pass.  ``forward(..., then=layer)``: the layer that runs next; where it
    is of this kind, the layer's last write also makes that layer's mixer input (``reads_ahead``) and leaves
    it with the step's context, where the next run finds it."""

    reads_ahead = True

    def __init__(self, spec, hidden_size, dtype):
        super().__init__(spec, hidden_size, dtype)
        self.streams = int(self.param("streams"))
        if not 1 <= self.streams <= 16:
            raise ValueError(f"1 to 16 streams, not {self.streams}")
        self.has_ffn = bool(spec.params.get("feed_forward", True))
        self.needs = ("mixer_norm", "ffn_norm", "feed_forward") if self.has_ffn else ("mixer_norm",)
        self.w = {}

    def _sides(self):
        return ("mixer", "ffn") if self.has_ffn else ("mixer",)

    def tensor_specs(self) -> List[TensorSpec]:
        S = self.streams
        specs = []
        for side in self._sides():
            specs += [TensorSpec(self.name(side + "_in"), (S,), "vector", init="gain"),
                      TensorSpec(self.name(side + "_out"), (S,), "vector", init="gain"),
                      TensorSpec(self.name(side + "_mix"), (S, S), "vector", init="mix")]
        if not self.has_ffn:
            # a layer without feed-forward: a file may still hold the second sublayer's weights; they are not read
            for what, shape in (("ffn_in", (S,)), ("ffn_out", (S,)), ("ffn_mix", (S, S)), ("unused_norm", (self.hidden_size,))):
                if what in self.spec.names:
                    specs.append(TensorSpec(self.name(what), shape, "vector", optional=True))
        return specs

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        for side in self._sides():
            for what in ("in", "out", "mix"):
                self.w[side, what] = tensors[self.name(f"{side}_{what}")].contiguous()

    @staticmethod
    def _plain_rms(norm):
        """(gain, eps) of a norm that the stream kernels can apply themselves, else None."""
        if (type(norm).__name__ == "LayerNorm" and not norm.center and norm.beta is None and norm.affine):
            return norm.gamma, norm.eps
        return None

    def _read(self, x32, side: str, norm):
        fused = self._plain_rms(norm)
        if fused is not None:
            return K.streams_read(x32, self.w[side, "in"], fused[0], fused[1], self.dtype)
        u32 = K.streams_read(x32, self.w[side, "in"], None, 0.0, torch.float32)
        return norm.forward(u32, out_t=True)[0]

    def _ahead(self, then):
        """What the last write of this layer can make for the layer ``then``: (weights, gain, eps), or None."""
        if then is None or type(then.arrangement) is not type(self) or then.arrangement.streams != self.streams:
            return None
        fused = self._plain_rms(then.mixer_norm)
        return None if fused is None else (then.arrangement.w["mixer", "in"], fused[0], fused[1])

    def _last_write(self, x32, y32, side: str, then, ctx) -> None:
        ahead = self._ahead(then)
        made = K.streams_write(x32, y32, self.w[side, "mix"], self.w[side, "out"], then=ahead,
                               out_dtype=self.dtype if ahead is not None else None)
        ctx.read_ahead = (made, x32.data_ptr()) if ahead is not None else None

    def forward(self, x32: torch.Tensor, layer, ctx, cache, write: bool = True, then=None) -> torch.Tensor:
        for part in (layer.mixer, layer.feed_forward if self.has_ffn else None):
            if part is not None and not getattr(part, "raw_output_ok", False):
                raise ValueError(f"{type(part).__name__} cannot give its result without the residual stream")
        if x32.shape[1] != self.streams * self.hidden_size:
            raise ValueError(f"{self.streams} streams of {self.hidden_size} make no row of {x32.shape[1]}")
        ahead, ctx.read_ahead = getattr(ctx, "read_ahead", None), None
        if ahead is not None and ahead[1] == x32.data_ptr():
            a = ahead[0]                     # the run before this one has made it with its last write
        else:
            a = self._read(x32, "mixer", layer.mixer_norm)
        m32 = layer.mixer.forward(a, None, ctx, cache, write)
        if not self.has_ffn:
            self._last_write(x32, m32, "mixer", then, ctx)
            return x32
        fused = self._plain_rms(layer.ffn_norm)
        if fused is not None:
            d = K.streams_write(x32, m32, self.w["mixer", "mix"], self.w["mixer", "out"],
                                then=(self.w["ffn", "in"], fused[0], fused[1]), out_dtype=self.dtype)
        else:
            K.streams_write(x32, m32, self.w["mixer", "mix"], self.w["mixer", "out"])
            d = self._read(x32, "ffn", layer.ffn_norm)
        f32 = layer.feed_forward.forward(d, None, ctx)
        self._last_write(x32, f32, "ffn", then, ctx)
        return x32
