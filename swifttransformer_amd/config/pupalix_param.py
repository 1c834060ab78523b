"""Typed hyper-parameters of the Pupalix architecture, read from its config.json.

A Pupalix model embeds a token as its table row times a factor plus a row of a second table chosen by a hash
of the token and the one before it.  Its layers are pre-norm blocks (root-mean-square norms) around one of
three mixers, in any order: *latent attention* (one small normalised latent a token that every head's keys and
values are products of, and one small rotated key part that all heads share; interleaved pairs, frequencies and
amplitude rescaled for long contexts), grouped *attention* whose values are its keys (a norm over the whole
query and key projections, no positions, capped scores, a mask of chunks), or *lightning* attention (a linear
recurrence with one fixed decay a head, read out through a norm over all heads and a sigmoid gate).  The
feed-forward is a dense gated unit, routed experts chosen within the best groups and weighted by their shares
of the softmax over all experts, or absent.  The residual stream may run as several copies that every
sublayer reads as a weighted sum and writes through a mixing matrix.  A group of consecutive layers may run
several times in a row with the same weights, every pass with caches and states of its own.  The head is the
embedding table; logits are multiplied by a factor and limited smoothly.

config.json:
    {"architecture": "Pupalix", "vocab": V, "width": W, "norm": {"eps": e}, "streams": S | absent,
     "embedding": {"scale": f, "bigram": {"buckets", "mul_prev", "mul_cur"} | absent},
     "logit_scale": f, "logit_softcap": c | absent, "loop": {"start", "stop", "times"} | absent,
     "layers": [
       {"type": "latent_attention", "mixer": {"heads", "dim", "rot_dim", "vdim", "kv_rank", "scale",
            "rot": {"base", "dims", "scaling": {"factor", "original", "fast", "slow"}?}}, "mlp": ...},
       {"type": "attention", "mixer": {"heads", "kv_heads", "dim", "vdim", "scale", "softcap"?,
            "mask": {"size"}?}, "mlp": ...},
       {"type": "lightning", "mixer": {"heads", "dim", "vdim", "decay": [one a head]}, "mlp": ...}]}
    mlp: null | {"kind": "dense", "ff"} |
         {"kind": "moe", "router": {"experts", "top", "groups": {"count", "keep"}?}, "expert": {"ff"}}
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from .gisedra_param import _need, _NUM
from .hyper_param import ConfigError

ARCHITECTURE = "Pupalix"
MIXER_TYPES = ("latent_attention", "attention", "lightning")


@dataclass(frozen=True)
class PupalixHyperParam:
    vocab: int
    width: int
    layers: List[Dict[str, Any]]                 # as in config.json
    streams: int = 0                             # 0: one residual stream and the plain sum
    embedding_scale: float = 1.0
    bigram: Optional[Dict[str, int]] = None      # {"buckets", "mul_prev", "mul_cur"}
    logit_scale: float = 1.0
    logit_softcap: float = 0.0                   # 0: none
    loop: Optional[Dict[str, int]] = None        # {"start", "stop", "times"}
    norm_eps: float = 1e-5
    max_positions: int = 65536                   # the design has no limit of its own
    eos_token_id: Optional[int] = None
    torch_dtype: str = "bfloat16"
    architecture: str = ARCHITECTURE
    extra: Dict[str, Any] = field(default_factory=dict, compare=False)

    # ------------------------------------------------------------- validation
    def validate(self) -> "PupalixHyperParam":
        if self.norm_eps <= 0:
            raise ConfigError(f"norm.eps must be positive, got {self.norm_eps}")
        if not 0 <= self.streams <= 16:
            raise ConfigError(f"streams must be 1 to 16 (or absent), got {self.streams}")
        if self.logit_softcap < 0:
            raise ConfigError(f"logit_softcap must not be negative, got {self.logit_softcap}")
        if self.bigram is not None:
            _need(self.bigram, "buckets", "embedding.bigram", (int,), 1)
            _need(self.bigram, "mul_prev", "embedding.bigram", (int,))
            _need(self.bigram, "mul_cur", "embedding.bigram", (int,))
        if not self.layers:
            raise ConfigError("config.json: 'layers' is empty")
        for i, L in enumerate(self.layers):
            w = f"layers[{i}]"
            kind = L.get("type") if isinstance(L, dict) else None
            if kind not in MIXER_TYPES:
                raise ConfigError(f"config.json: {w}.type must be one of {MIXER_TYPES}, got {kind!r}")
            m = L.get("mixer")
            getattr(self, "_check_" + kind)(m, f"{w}.mixer")
            self._check_mlp(L.get("mlp"), f"{w}.mlp")
        if self.loop is not None:
            a = _need(self.loop, "start", "loop", (int,), 0)
            b = _need(self.loop, "stop", "loop", (int,), 0)
            _need(self.loop, "times", "loop", (int,), 1)
            if not a < b <= len(self.layers):
                raise ConfigError(f"config.json: loop must name layers start < stop <= {len(self.layers)}, "
                                  f"got {a} and {b}")
        return self

    @staticmethod
    def _check_latent_attention(m, w: str) -> None:
        for key in ("heads", "dim", "vdim"):
            _need(m, key, w, (int,), 1)
        rank = _need(m, "kv_rank", w, (int,), 1)
        r = _need(m, "rot_dim", w, (int,), 0)
        _need(m, "scale", w, _NUM)
        if r % 2 or rank + r > 256:
            raise ConfigError(f"config.json: {w}.rot_dim must be even and kv_rank + rot_dim at most 256, got "
                              f"{rank} + {r}")
        if r:
            rot = m.get("rot")
            dims = _need(rot, "dims", f"{w}.rot", (int,), 2)
            if dims % 2 or dims > r:
                raise ConfigError(f"config.json: {w}.rot.dims must be even and at most rot_dim, got {dims}")
            if _need(rot, "base", f"{w}.rot", _NUM) <= 1:
                raise ConfigError(f"config.json: {w}.rot.base must be above 1")
            sc = rot.get("scaling")
            if sc is not None:
                for key in ("factor", "original", "fast", "slow"):
                    if _need(sc, key, f"{w}.rot.scaling", _NUM) <= 0:
                        raise ConfigError(f"config.json: {w}.rot.scaling.{key} must be positive")

    @staticmethod
    def _check_attention(m, w: str) -> None:
        heads = _need(m, "heads", w, (int,), 1)
        if heads % _need(m, "kv_heads", w, (int,), 1):
            raise ConfigError(f"config.json: {w}.heads must be a multiple of kv_heads")
        dim = _need(m, "dim", w, (int,), 1)
        if dim > 256:
            raise ConfigError(f"config.json: {w}.dim: heads of up to 256, got {dim}")
        if "vdim" in m and m["vdim"] != dim:
            raise ConfigError(f"config.json: {w}.vdim: the values are the keys, so it equals dim ({dim}), got {m['vdim']}")
        _need(m, "scale", w, _NUM)
        if m.get("softcap") is not None and _need(m, "softcap", w, _NUM) < 0:
            raise ConfigError(f"config.json: {w}.softcap must not be negative")
        if m.get("mask") is not None:
            _need(m["mask"], "size", f"{w}.mask", (int,), 1)

    @staticmethod
    def _check_lightning(m, w: str) -> None:
        heads = _need(m, "heads", w, (int,), 1)
        if _need(m, "dim", w, (int,), 1) > 256:
            raise ConfigError(f"config.json: {w}.dim: up to 256 key channels a head, got {m['dim']}")
        _need(m, "vdim", w, (int,), 1)
        decay = m.get("decay")
        if not isinstance(decay, list) or len(decay) != heads or not all(isinstance(d, _NUM) and not isinstance(d, bool)
                                                                         for d in decay):
            raise ConfigError(f"config.json: {w}.decay must list one number a head ({heads})")

    @staticmethod
    def _check_mlp(mlp, w: str) -> None:
        if mlp is None:
            return
        kind = mlp.get("kind") if isinstance(mlp, dict) else None
        if kind == "dense":
            _need(mlp, "ff", w, (int,), 1)
        elif kind == "moe":
            r = mlp.get("router")
            experts = _need(r, "experts", f"{w}.router", (int,), 1)
            top = _need(r, "top", f"{w}.router", (int,), 1)
            count, keep = 1, 1
            if r.get("groups") is not None:
                count = _need(r["groups"], "count", f"{w}.router.groups", (int,), 1)
                keep = _need(r["groups"], "keep", f"{w}.router.groups", (int,), 1)
            if experts % count or keep > count or count > 64:
                raise ConfigError(f"config.json: {w}.router.groups: {experts} experts in {count} equal groups (up to 64) "
                                  f"of which {keep} are kept")
            if top > min(keep * (experts // count), 16):
                raise ConfigError(f"config.json: {w}.router.top must be at most the experts of the kept groups and "
                                  f"16, got {top}")
            _need(mlp.get("expert"), "ff", f"{w}.expert", (int,), 1)
        else:
            raise ConfigError(f"config.json: {w}.kind must be 'dense' or 'moe', got {kind!r}")

    def run_order(self) -> List[int]:
        """The layers in the order they run: the repeated group ``times`` times in a row."""
        n = len(self.layers)
        if self.loop is None:
            return list(range(n))
        a, b, times = int(self.loop["start"]), int(self.loop["stop"]), int(self.loop["times"])
        return list(range(a)) + list(range(a, b)) * times + list(range(b, n))

    # --------------------------------------------------------------- factories
    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "PupalixHyperParam":
        layers = copy.deepcopy(d.get("layers"))
        if not isinstance(layers, list):
            raise ConfigError("config.json lacks the list 'layers'")
        emb = d.get("embedding") or {}
        known = {"architecture", "architectures", "vocab", "width", "layers", "loop", "norm", "streams", "embedding",
                 "logit_scale", "logit_softcap", "max_positions", "eos_token_id", "torch_dtype", "dtype"}
        return cls(
            vocab=_need(d, "vocab", "the top level", (int,), 1),
            width=_need(d, "width", "the top level", (int,), 1),
            layers=layers,
            streams=int(_need(d, "streams", "the top level", (int,), 1)) if d.get("streams") is not None else 0,
            embedding_scale=float(emb["scale"]) if emb.get("scale") is not None else 1.0,
            bigram=copy.deepcopy(emb.get("bigram")) or None,
            logit_scale=float(d["logit_scale"]) if d.get("logit_scale") is not None else 1.0,
            logit_softcap=float(d.get("logit_softcap") or 0.0),
            loop=copy.deepcopy(d.get("loop")) or None,
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
                               "embedding": {"scale": self.embedding_scale}, "logit_scale": self.logit_scale,
                               "torch_dtype": self.torch_dtype}
        if self.bigram is not None:
            cfg["embedding"]["bigram"] = dict(self.bigram)
        if self.streams:
            cfg["streams"] = self.streams
        if self.logit_softcap:
            cfg["logit_softcap"] = self.logit_softcap
        if self.loop is not None:
            cfg["loop"] = dict(self.loop)
        if self.max_positions != 65536:
            cfg["max_positions"] = self.max_positions
        if self.eos_token_id is not None:
            cfg["eos_token_id"] = self.eos_token_id
        return cfg

    def __str__(self) -> str:
        kinds = ", ".join(f"{L['type']}/{(L.get('mlp') or {}).get('kind', 'none')}" for L in self.layers)
        return (f"PupalixHyperParam {{\n\tvocab = {self.vocab}\n\twidth = {self.width}\n\tnorm_eps = {self.norm_eps}\n\t"
                f"streams = {self.streams}\n\tloop = {self.loop}\n\tlayers = [{kinds}]\n}}")
