"""Typed hyper-parameters of the Gisedra architecture, read from its config.json.

A Gisedra model is a list of layers, each a "sandwich" (a dynamic-tanh norm before and after the mixer
and before and after the feed-forward).  A layer's mixer is either a *latent attention* with a sliding
window and a small rotated key part that all heads share, or a *parallel* pair: grouped softmax attention
(short filter over time on q, k, v, partial rotary positions with rescaled frequencies, a window that
keeps the first tokens, a sigmoid gate on the heads) beside a retention (linear attention with a fixed
decay a head).  Feed-forwards are routed experts or absent.  After the feed-forward a layer may add a
gated projection of a per-layer token embedding at unit root mean square.  A group of consecutive layers
may run several times in a row with the same weights, every pass with caches and states of its own.

config.json:
    {"architecture": "Gisedra", "vocab": V, "width": W, "norm": {"eps": e},
     "token_side": {"dim": d} | absent, "loop": {"start": a, "stop": b, "times": n} | absent,
     "layers": [
       {"type": "latent_attention", "mixer": {"heads", "dim", "rot_dim", "vdim", "kv_rank", "scale",
                                              "mask": {"size"}?, "rot": {"base", "dims"}}, "mlp": ...},
       {"type": "parallel", "mixer": {"left_scale", "right_scale",
            "left": {"heads", "kv_heads", "dim", "vdim", "scale", "conv"?, "mask": {"size", "keep_first"?}?,
                     "rot": {"base", "dims", "scaling": {"factor", "low", "high", "original"}?}?},
            "right": {"heads", "dim", "vdim", "decay": [one a head]}}, "mlp": ...}]}
    mlp: null | {"kind": "moe", "router": {"experts", "top"}, "expert": {"ff"}}
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from .hyper_param import ConfigError

ARCHITECTURE = "Gisedra"
MIXER_TYPES = ("latent_attention", "parallel")
_NUM = (int, float)


def _need(d, key: str, where: str, kind=(int,), minimum=None):
    if not isinstance(d, dict) or key not in d:
        raise ConfigError(f"config.json: {where} lacks the key {key!r}")
    v = d[key]
    if isinstance(v, bool) or not isinstance(v, kind):
        raise ConfigError(f"config.json: {where}.{key} must be {'/'.join(k.__name__ for k in kind)}, got {v!r}")
    if minimum is not None and v < minimum:
        raise ConfigError(f"config.json: {where}.{key} must be >= {minimum}, got {v}")
    return v


def _check_rot(rot, where: str, limit: int, scaling_ok: bool) -> None:
    dims = _need(rot, "dims", where, (int,), 2)
    if dims % 2 or dims > limit:
        raise ConfigError(f"config.json: {where}.dims must be even and at most {limit}, got {dims}")
    if _need(rot, "base", where, _NUM) <= 1:
        raise ConfigError(f"config.json: {where}.base must be above 1")
    sc = rot.get("scaling")
    if sc is not None:
        if not scaling_ok:
            raise ConfigError(f"config.json: {where}.scaling is not part of this mixer")
        for key in ("factor", "low", "high", "original"):
            if _need(sc, key, f"{where}.scaling", _NUM) <= 0:
                raise ConfigError(f"config.json: {where}.scaling.{key} must be positive")
        if sc["high"] <= sc["low"]:
            raise ConfigError(f"config.json: {where}.scaling.high must be above low")


@dataclass(frozen=True)
class GisedraHyperParam:
    vocab: int
    width: int
    layers: List[Dict[str, Any]]                 # as in config.json
    loop: Optional[Dict[str, int]] = None        # {"start", "stop", "times"}: layers [start, stop) run `times` times
    token_side_dim: int = 0                      # 0: no per-layer token input
    norm_eps: float = 1e-5
    max_positions: int = 65536                   # the design has no limit of its own; tables are sized by this
    eos_token_id: Optional[int] = None
    torch_dtype: str = "bfloat16"
    architecture: str = ARCHITECTURE
    extra: Dict[str, Any] = field(default_factory=dict, compare=False)

    # ------------------------------------------------------------- validation
    def validate(self) -> "GisedraHyperParam":
        if self.norm_eps <= 0:
            raise ConfigError(f"norm.eps must be positive, got {self.norm_eps}")
        if self.token_side_dim < 0:
            raise ConfigError(f"token_side.dim must not be negative, got {self.token_side_dim}")
        if not self.layers:
            raise ConfigError("config.json: 'layers' is empty")
        for i, L in enumerate(self.layers):
            w = f"layers[{i}]"
            kind = L.get("type") if isinstance(L, dict) else None
            if kind not in MIXER_TYPES:
                raise ConfigError(f"config.json: {w}.type must be one of {MIXER_TYPES}, got {kind!r}")
            m = L.get("mixer")
            if kind == "latent_attention":
                self._check_latent(m, f"{w}.mixer")
            else:
                for key in ("left_scale", "right_scale"):
                    _need(m, key, f"{w}.mixer", _NUM)
                self._check_left(m.get("left"), f"{w}.mixer.left")
                self._check_right(m.get("right"), f"{w}.mixer.right")
            mlp = L.get("mlp")
            if mlp is not None:
                if mlp.get("kind") != "moe":
                    raise ConfigError(f"config.json: {w}.mlp.kind must be 'moe', got {mlp.get('kind')!r}")
                experts = _need(mlp.get("router"), "experts", f"{w}.mlp.router", (int,), 1)
                top = _need(mlp.get("router"), "top", f"{w}.mlp.router", (int,), 1)
                if top > min(experts, 16):
                    raise ConfigError(f"config.json: {w}.mlp.router.top must be at most the experts and 16, got {top}")
                _need(mlp.get("expert"), "ff", f"{w}.mlp.expert", (int,), 1)
        if self.loop is not None:
            a = _need(self.loop, "start", "loop", (int,), 0)
            b = _need(self.loop, "stop", "loop", (int,), 0)
            _need(self.loop, "times", "loop", (int,), 1)
            if not a < b <= len(self.layers):
                raise ConfigError(f"config.json: loop must name layers start < stop <= {len(self.layers)}, "
                                  f"got {a} and {b}")
        return self

    @staticmethod
    def _check_latent(m, w: str) -> None:
        _need(m, "heads", w, (int,), 1)
        _need(m, "dim", w, (int,), 1)
        _need(m, "vdim", w, (int,), 1)
        rank = _need(m, "kv_rank", w, (int,), 1)
        r = _need(m, "rot_dim", w, (int,), 0)
        _need(m, "scale", w, _NUM)
        if r % 2 or rank + r > 256:
            raise ConfigError(f"config.json: {w}.rot_dim must be even and kv_rank + rot_dim at most 256, got "
                              f"{rank} + {r}")
        if r:
            _check_rot(m.get("rot"), f"{w}.rot", r, scaling_ok=True)
        if m.get("mask") is not None:
            _need(m["mask"], "size", f"{w}.mask", (int,), 1)

    @staticmethod
    def _check_left(m, w: str) -> None:
        heads = _need(m, "heads", w, (int,), 1)
        if heads % _need(m, "kv_heads", w, (int,), 1):
            raise ConfigError(f"config.json: {w}.heads must be a multiple of kv_heads")
        dim = _need(m, "dim", w, (int,), 1)
        _need(m, "vdim", w, (int,), 1)
        _need(m, "scale", w, _NUM)
        if m.get("conv") is not None and not 1 <= _need(m, "conv", w, (int,), 1) <= 8:
            raise ConfigError(f"config.json: {w}.conv must be 1 to 8 taps")
        mask = m.get("mask")
        if mask is not None:
            _need(mask, "size", f"{w}.mask", (int,), 1)
            if mask.get("keep_first") is not None:
                _need(mask, "keep_first", f"{w}.mask", (int,), 0)
        if m.get("rot") is not None:
            _check_rot(m["rot"], f"{w}.rot", dim, scaling_ok=True)

    @staticmethod
    def _check_right(m, w: str) -> None:
        heads = _need(m, "heads", w, (int,), 1)
        if _need(m, "dim", w, (int,), 1) > 256:
            raise ConfigError(f"config.json: {w}.dim: up to 256 key channels a head, got {m['dim']}")
        _need(m, "vdim", w, (int,), 1)
        decay = m.get("decay")
        if not isinstance(decay, list) or len(decay) != heads or not all(isinstance(d, _NUM) and not isinstance(d, bool)
                                                                         for d in decay):
            raise ConfigError(f"config.json: {w}.decay must list one number a head ({heads})")

    def run_order(self) -> List[tuple]:
        """[(layer, pass number or None)] in the order the layers run; a pass number is given for the first
        layer of each pass over the repeated group."""
        n = len(self.layers)
        if self.loop is None:
            return [(i, None) for i in range(n)]
        a, b, times = int(self.loop["start"]), int(self.loop["stop"]), int(self.loop["times"])
        order = [(i, None) for i in range(a)]
        for r in range(times):
            order += [(i, r if i == a else None) for i in range(a, b)]
        return order + [(i, None) for i in range(b, n)]

    # --------------------------------------------------------------- factories
    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "GisedraHyperParam":
        layers = copy.deepcopy(d.get("layers"))
        if not isinstance(layers, list):
            raise ConfigError("config.json lacks the list 'layers'")
        side = d.get("token_side")
        known = {"architecture", "architectures", "vocab", "width", "layers", "loop", "norm", "token_side",
                 "max_positions", "eos_token_id", "torch_dtype", "dtype"}
        return cls(
            vocab=_need(d, "vocab", "the top level", (int,), 1),
            width=_need(d, "width", "the top level", (int,), 1),
            layers=layers,
            loop=copy.deepcopy(d.get("loop")) or None,
            token_side_dim=int(_need(side, "dim", "token_side", (int,), 1)) if side else 0,
            norm_eps=float(_need(d.get("norm"), "eps", "norm", _NUM)),
            max_positions=int(d.get("max_positions", 65536)),
            eos_token_id=d.get("eos_token_id"),
            torch_dtype=str(d.get("torch_dtype", d.get("dtype", "bfloat16"))).replace("torch.", ""),
            architecture=ARCHITECTURE,
            extra={k: v for k, v in d.items() if k not in known},
        ).validate()

    def to_config_dict(self) -> Dict[str, Any]:
        cfg: Dict[str, Any] = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                               "norm": {"eps": self.norm_eps}, "layers": copy.deepcopy(self.layers),
                               "torch_dtype": self.torch_dtype}
        if self.token_side_dim:
            cfg["token_side"] = {"dim": self.token_side_dim}
        if self.loop is not None:
            cfg["loop"] = dict(self.loop)
        if self.max_positions != 65536:
            cfg["max_positions"] = self.max_positions
        if self.eos_token_id is not None:
            cfg["eos_token_id"] = self.eos_token_id
        return cfg

    def __str__(self) -> str:
        kinds = ", ".join(f"{L['type']}/{(L.get('mlp') or {}).get('kind', 'none')}" for L in self.layers)
        return (f"GisedraHyperParam {{\n\tvocab = {self.vocab}\n\twidth = {self.width}\n\tnorm_eps = {self.norm_eps}\n\t"
                f"token_side_dim = {self.token_side_dim}\n\tloop = {self.loop}\n\tlayers = [{kinds}]\n}}")
