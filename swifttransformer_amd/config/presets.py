"""Named sizes of the OPT family, for runs with random weights where no config.json exists.

Counterpart of the reference's table of hyper-parameters by name
(src/examples/lib/common_gpt_hyper_params.h:9-68, looked up by ``str2hyperparam``
:105-130).  The numbers are those of the published OPT configurations; a model folder's
config.json always takes precedence over a name."""
from __future__ import annotations

from typing import Dict

from .hyper_param import OptHyperParam

#          name        layers hidden heads  ffn
_SIZES = {"opt_125m": (12, 768, 12, 3072),
          "opt_1.3b": (24, 2048, 32, 8192),
          "opt_2.7b": (32, 2560, 32, 10240),
          "opt_6.7b": (32, 4096, 32, 16384),
          "opt_13b": (40, 5120, 40, 20480),
          "opt_30b": (48, 7168, 56, 28672)}


def preset_names():
    return list(_SIZES)


def preset(name: str, **overrides) -> OptHyperParam:
    """Hyper-parameters of ``name`` (``opt_125m`` ... ``opt_30b``); keyword arguments replace fields."""
    key = name.lower().replace("-", "_")
    if key not in _SIZES:
        raise KeyError(f"invalid model name {name!r}; valid names: {' '.join(_SIZES)}")
    layers, hidden, heads, ffn = _SIZES[key]
    fields: Dict = dict(vocab_size=50272, max_position_embeddings=2048, hidden_size=hidden,
                        num_hidden_layers=layers, num_attention_heads=heads, ffn_dim=ffn,
                        word_embed_proj_dim=hidden)
    fields.update(overrides)
    return OptHyperParam(**fields).validate()


# ---- named sizes of the Zitupel family, for runs with random weights: the layer sizes of the
# OPT model of the same name (width, heads, feed-forward width), so that the two can be set side
# by side.  Of every four layers three are gated linear attention and one is latent attention;
# every second latent layer borrows the latent of the one before it; the first layer's
# feed-forward is dense, the others route every token to 2 of 16 experts of a quarter of the
# dense width each.
def zitupel_preset(name: str, **overrides):
    from .zitupel_param import ZitupelHyperParam
    key = name.lower().replace("-", "_")
    size = key.split("_", 1)[1] if "_" in key else ""
    if "opt_" + size not in _SIZES:
        raise KeyError(f"invalid model name {name!r}; valid names: " +
                       " ".join("zitupel_" + k.split("_", 1)[1] for k in _SIZES))
    n_layers, hidden, heads, ffn = _SIZES["opt_" + size]
    n_layers = int(overrides.pop("num_layers", n_layers))
    dense_only = bool(overrides.pop("dense_only", False))
    hd = hidden // heads
    layers, last_owner = [], None
    for i in range(n_layers):
        if i % 4 == 3:
            mixer = {"heads": heads, "dim": hd, "vdim": hd, "kv_rank": 128, "scale": float(hd) ** -0.5}
            if last_owner is not None:
                mixer["kv_from"], last_owner = last_owner, None
            else:
                last_owner = i
            kind = "latent_attention"
        else:
            mixer, kind = {"heads": heads, "dim": hd, "vdim": hd, "tau": 16.0, "decay_rank": 16}, "gla"
        if i == 0 or dense_only:
            mlp = {"kind": "dense", "ff": ffn}
        else:
            mlp = {"kind": "moe", "router": {"experts": 16, "top": 2}, "expert": {"ff": ffn // 4, "limit": 7.0}}
        layers.append({"type": kind, "mixer": mixer, "mlp": mlp})
    fields: Dict = dict(vocab=50272, width=hidden, layers=layers, residual_mult=0.5, norm_eps=1e-5, canon_taps=4,
                        max_positions=2048)
    fields.update(overrides)
    return ZitupelHyperParam(**fields).validate()


# ---- named sizes of the Zimorax family, for runs with random weights: the layer sizes of the OPT
# model of the same name (width, heads, feed-forward width).  Of every four layers the first is a gated
# delta rule, the second windowed attention (a quarter of the heads as key heads, a window of 1,024,
# rotary positions on half of each head, scaled fourfold), the last two state-space mixers; the first
# two layers run twice.
def zimorax_preset(name: str, **overrides):
    from .zimorax_param import ZimoraxHyperParam
    key = name.lower().replace("-", "_")
    size = key.split("_", 1)[1] if "_" in key else ""
    if "opt_" + size not in _SIZES:
        raise KeyError(f"invalid model name {name!r}; valid names: " +
                       " ".join("zimorax_" + k.split("_", 1)[1] for k in _SIZES))
    n_layers, hidden, heads, ffn = _SIZES["opt_" + size]
    n_layers = int(overrides.pop("num_layers", n_layers))
    only = overrides.pop("only", None)            # one mixer type for every layer (measurements)
    window = int(overrides.pop("window", 1024))
    loop_times = int(overrides.pop("loop_times", 2))
    hd = hidden // heads
    layers = []
    for i in range(n_layers):
        kind = only or ("delta", "attention", "mamba2", "mamba2")[i % 4]
        if kind == "attention":
            mixer = {"heads": heads, "kv_heads": max(1, heads // 4), "dim": hd, "vdim": hd, "scale": float(hd) ** -0.5,
                     "mask": {"size": window},
                     "rot": {"dims": hd // 2, "base": 10000.0,
                             "scaling": {"factor": 4.0, "original": 2048, "fast": 32.0, "slow": 1.0}}}
        elif kind == "mamba2":
            mixer = {"heads": heads, "vdim": hd, "state": 64, "groups": max(1, heads // 8), "norm_groups": 1, "conv": 4}
        else:
            mixer = {"heads": heads, "kv_heads": heads, "dim": hd, "vdim": hd, "conv": 4}
        layers.append({"type": kind, "mixer": mixer, "mlp": {"kind": "dense", "ff": ffn}})
    loop = {"start": 0, "stop": min(2, n_layers), "times": loop_times} if loop_times > 0 else None
    fields: Dict = dict(vocab=50272, width=hidden, layers=layers, loop=loop, norm_eps=1e-5, max_positions=4096)
    fields.update(overrides)
    return ZimoraxHyperParam(**fields).validate()


# ---- named sizes of the Gisedra family, for runs with random weights: the layer sizes of the OPT model of
# the same name (width, heads).  Of every four layers the third is a parallel pair (window attention with a
# quarter of the heads as key heads, a window of 1,024 that keeps the first 16 tokens, rotary positions on
# half of each head; beside it a retention of an eighth of the heads), the others latent attention (rank
# 128, a rotated part of 32, a window of 1,024); every layer has 16 experts of a quarter of the OPT
# feed-forward's width, 2 a token, and a token input of 16; the first two layers run twice.
def gisedra_preset(name: str, **overrides):
    from .gisedra_param import GisedraHyperParam
    key = name.lower().replace("-", "_")
    size = key.split("_", 1)[1] if "_" in key else ""
    if "opt_" + size not in _SIZES:
        raise KeyError(f"invalid model name {name!r}; valid names: " +
                       " ".join("gisedra_" + k.split("_", 1)[1] for k in _SIZES))
    n_layers, hidden, heads, ffn = _SIZES["opt_" + size]
    n_layers = int(overrides.pop("num_layers", n_layers))
    only = overrides.pop("only", None)            # one mixer type for every layer (measurements)
    window = int(overrides.pop("window", 1024))
    loop_times = int(overrides.pop("loop_times", 2))
    hd = hidden // heads
    layers = []
    for i in range(n_layers):
        kind = only or ("latent_attention", "latent_attention", "parallel", "latent_attention")[i % 4]
        if kind == "latent_attention":
            mixer = {"heads": heads, "dim": hd, "rot_dim": 32, "vdim": hd, "kv_rank": 128,
                     "scale": float(hd + 32) ** -0.5, "mask": {"size": window}, "rot": {"base": 10000.0, "dims": 32}}
        else:
            rh = max(1, heads // 8)
            mixer = {"left_scale": 1.0, "right_scale": 1.0,
                     "left": {"heads": heads, "kv_heads": max(1, heads // 4), "dim": hd, "vdim": hd,
                              "scale": float(hd) ** -0.5, "conv": 4, "mask": {"size": window, "keep_first": 16},
                              "rot": {"dims": hd // 2, "base": 10000.0,
                                      "scaling": {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 2048}}},
                     "right": {"heads": rh, "dim": hd, "vdim": 2 * hd,
                               "decay": [1.0 - 2.0 ** (-5 - (j % 4)) for j in range(rh)]}}
        mlp = {"kind": "moe", "router": {"experts": 16, "top": 2}, "expert": {"ff": ffn // 4}}
        layers.append({"type": kind, "mixer": mixer, "mlp": mlp})
    loop = {"start": 0, "stop": min(2, n_layers), "times": loop_times} if loop_times > 0 else None
    fields: Dict = dict(vocab=50272, width=hidden, layers=layers, loop=loop, token_side_dim=16, norm_eps=1e-5,
                        max_positions=4096)
    fields.update(overrides)
    return GisedraHyperParam(**fields).validate()


# ---- named sizes of the Pupalix family, for runs with random weights: the layer sizes of the OPT model of the
# same name.  Of every four layers the first is latent attention (dense gated feed-forward), the second grouped
# attention whose values are its keys (chunks of 1,024 positions, a quarter of the heads as key heads, routed
# experts), the third and fourth lightning attention (dense, then routed); four streams; the first two layers
# run twice.
def pupalix_preset(name: str, **overrides):
    from .pupalix_param import PupalixHyperParam
    key = name.lower().replace("-", "_")
    size = key.split("_", 1)[1] if "_" in key else ""
    if "opt_" + size not in _SIZES:
        raise KeyError(f"invalid model name {name!r}; valid names: " +
                       " ".join("pupalix_" + k.split("_", 1)[1] for k in _SIZES))
    n_layers, hidden, heads, ffn = _SIZES["opt_" + size]
    n_layers = int(overrides.pop("num_layers", n_layers))
    only = overrides.pop("only", None)            # one mixer type for every layer (measurements)
    chunk = int(overrides.pop("chunk", 1024))
    loop_times = int(overrides.pop("loop_times", 2))
    hd = hidden // heads
    layers = []
    for i in range(n_layers):
        kind = only or ("latent_attention", "attention", "lightning", "lightning")[i % 4]
        if kind == "latent_attention":
            mixer = {"heads": heads, "dim": hd, "rot_dim": 32, "vdim": hd, "kv_rank": 128, "scale": float(hd + 32) ** -0.5,
                     "rot": {"base": 10000.0, "dims": 32,
                             "scaling": {"factor": 8.0, "original": 1024, "fast": 16.0, "slow": 2.0}}}
        elif kind == "attention":
            mixer = {"heads": heads, "kv_heads": max(1, heads // 4), "dim": hd, "vdim": hd, "scale": float(hd) ** -0.5,
                     "softcap": 50.0, "mask": {"size": chunk}}
        else:
            lh = max(1, heads // 8)
            mixer = {"heads": lh, "dim": hd, "vdim": 2 * hd, "decay": [1.0 - 2.0 ** (-5 - (j % 4)) for j in range(lh)]}
        if i % 2 == 0:
            mlp = {"kind": "dense", "ff": ffn // 2}
        else:
            mlp = {"kind": "moe", "router": {"experts": 16, "top": 2, "groups": {"count": 4, "keep": 2}},
                   "expert": {"ff": ffn // 4}}
        layers.append({"type": kind, "mixer": mixer, "mlp": mlp})
    loop = {"start": 0, "stop": min(2, n_layers), "times": loop_times} if loop_times > 0 else None
    fields: Dict = dict(vocab=50272, width=hidden, layers=layers, loop=loop, streams=4, embedding_scale=float(hidden) ** 0.5,
                        bigram={"buckets": 65521, "mul_prev": 36313, "mul_cur": 27191}, logit_scale=1.0,
                        logit_softcap=30.0, norm_eps=1e-5, max_positions=4096)
    fields.update(overrides)
    return PupalixHyperParam(**fields).validate()
