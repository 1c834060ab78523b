"""Small Gisedra configurations for the tests, with weights made here, large enough that every mechanism
moves the logits, a router whose choices rest on no close call, and retention keys that lean towards the
queries (a first token's read-out is then no matter of a sign that rounding decides).

A: a latent layer (rank 20 and a turned part of 8: an entry padded to 32; keys of 24, values of 16, a window
   of 9), a parallel layer (4 heads on 2 key heads, keys of 16 and values of 24, 3 taps, a window of 12 that
   keeps the first 3 tokens, half of each head turned with rescaled frequencies; a retention of 2 heads),
   a latent layer without window and without feed-forward; layers 1 and 2 run three times; a token input of 8.
B: sizes that no vector load divides (width 72, heads of 10 and 6, a retention head of 5 x 18, experts of 20
   and 50), no filter, a window longer than most prompts and no kept tokens, full rotation without rescaling,
   all experts a token and one expert a token, no repeated group, no token input.
C: 8 heads on one key head, a filter of one tap, more kept tokens (70) than the window holds (64), a retention
   with wide keys (64), no feed-forward in the first layer; a latent layer whose turned part is as large as
   its keys; the whole model is one group that runs once; a token input of 4.
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict

import torch


def _latent(heads, dim, rot_dim, vdim, rank, scale, window=None, base=100.0):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank, "scale": scale,
         "rot": {"base": base, "dims": rot_dim}}
    if window is not None:
        m["mask"] = {"size": window}
    return {"type": "latent_attention", "mixer": m}


def _parallel(left, right, ls, rs):
    return {"type": "parallel", "mixer": {"left": left, "right": right, "left_scale": ls, "right_scale": rs}}


def _left(heads, kv, dim, vdim, scale, conv=None, mask=None, rot=None):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale}
    if conv is not None:
        m["conv"] = conv
    if mask is not None:
        m["mask"] = mask
    if rot is not None:
        m["rot"] = rot
    return m


def _moe(experts, top, ff):
    return {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}


def _with(layer, mlp):
    return dict(layer, mlp=mlp)


CONFIGS = {
    "A": {"architecture": "Gisedra", "vocab": 97, "width": 64, "max_positions": 512, "norm": {"eps": 1e-6}, "token_side": {"dim": 8},
          "loop": {"start": 1, "stop": 3, "times": 3},
          "layers": [_with(_latent(2, 24, 8, 16, 20, 0.3, window=9), _moe(4, 2, 24)),
                     _with(_parallel(_left(4, 2, 16, 24, 0.35, conv=3, mask={"size": 12, "keep_first": 3},
                                           rot={"dims": 8, "base": 100.0,
                                                "scaling": {"factor": 2.0, "low": 1.0, "high": 4.0, "original": 16}}),
                                     {"heads": 2, "dim": 12, "vdim": 20, "decay": [0.9, 0.995]}, 1.3, 0.6),
                           _moe(6, 3, 16)),
                     _with(_latent(4, 8, 4, 24, 33, 0.4), None)]},
    "B": {"architecture": "Gisedra", "vocab": 131, "width": 72, "max_positions": 512, "norm": {"eps": 1e-4},
          "layers": [_with(_parallel(_left(3, 3, 10, 6, 0.4, mask={"size": 130}, rot={"dims": 10, "base": 50.0}),
                                     {"heads": 1, "dim": 5, "vdim": 18, "decay": [0.75]}, 0.7, 1.5), _moe(3, 3, 20)),
                     _with(_latent(3, 10, 6, 14, 30, 0.35, window=5), _moe(5, 1, 50))]},
    "C": {"architecture": "Gisedra", "vocab": 61, "width": 128, "max_positions": 512, "norm": {"eps": 1e-5}, "token_side": {"dim": 4},
          "loop": {"start": 0, "stop": 2, "times": 1},
          "layers": [_with(_parallel(_left(8, 1, 32, 32, 0.2, conv=1, mask={"size": 64, "keep_first": 70},
                                           rot={"dims": 32, "base": 1000.0,
                                                "scaling": {"factor": 8.0, "low": 0.5, "high": 2.0, "original": 32}}),
                                     {"heads": 4, "dim": 64, "vdim": 16, "decay": [0.5, 0.9, 0.99, 1.0]}, 1.0, 1.0), None),
                     _with(_latent(8, 16, 16, 32, 64, 0.2, window=100, base=1000.0), _moe(8, 2, 40))]},
}
PAGE_SIZE = {"A": 4, "B": 2, "C": 16}


def reserved(cfg: dict) -> int:
    """The first coordinates of the stream hold a code of the token that only the routers read."""
    return max([L["mlp"]["router"]["experts"] for L in cfg["layers"] if L.get("mlp")] or [0])


def make_weights(cfg: dict, seed: int) -> Dict[str, torch.Tensor]:
    """float32 tensors by name.  The embedding's first ``reserved`` coordinates are a code of the token's id
    (levels from 1 down to -1, the highest at id % experts), no layer writes there, and a router reads nothing
    else: a token's experts follow from its id by a wide margin in every pass."""
    g = torch.Generator().manual_seed(seed)
    W, V, n = cfg["width"], cfg["vocab"], len(cfg["layers"])
    R = reserved(cfg)
    rnd = lambda *shape, std=1.0: torch.randn(*shape, generator=g) * std
    mat = lambda out, inp, gain=1.0: rnd(out, inp, std=gain / math.sqrt(inp))

    def clear(t):                 # rows (or entries) of the reserved coordinates
        t[:R] = 0.0
        return t

    def norm(name, width, w_out=False):
        gain, bias = 1.0 + rnd(width, std=0.2), rnd(width, std=0.1)
        if w_out:
            clear(gain), clear(bias)
        else:
            gain[:R] = 1.0
            bias[:R] = 0.0
        return {name: gain, name + ".b": bias, name + ".alpha": torch.tensor(0.7 + 0.3 * float(torch.rand((), generator=g)))}

    emb = rnd(V, W)
    for t in range(V):
        for e in range(R):
            emb[t, e] = 1.0 - 2.0 * ((e - t) % R) / max(R - 1, 1)
    w = {"embed": emb, "head": mat(V, W, 2.0)}
    w.update(norm("final.norm", W))
    if cfg.get("loop"):
        w["loop.step"] = clear(rnd(cfg["loop"]["times"], W, std=0.3).T.contiguous()).T.contiguous()
    side = (cfg.get("token_side") or {}).get("dim", 0)
    if side:
        w["side.embed"] = rnd(V, n * side)
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        w.update(norm(p + "norm1", W))
        w.update(norm(p + "norm1b", W, w_out=True))
        if L["type"] == "latent_attention":
            H, d, r, dv, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
            w.update({p + "mix.q": mat(H * (d + r), W, 1.5), p + "mix.dkv": mat(rank + r, W, 1.5),
                      p + "mix.dkv.norm": 1.0 + rnd(rank, std=0.2), p + "mix.uk": mat(H * d, rank, 1.5),
                      p + "mix.uv": mat(H * dv, rank, 1.2), p + "mix.o": mat(W, H * dv, 1.0)})
        else:
            le, ri = m["left"], m["right"]
            H, G, d, dv = le["heads"], le["kv_heads"], le["dim"], le["vdim"]
            w.update({p + "mix.left.q": mat(H * d, W, 1.5), p + "mix.left.k": mat(G * d, W, 1.5),
                      p + "mix.left.v": mat(G * dv, W, 1.2), p + "mix.left.g": mat(H * dv, W, 1.5),
                      p + "mix.left.o": mat(W, H * dv, 1.0)})
            if le.get("conv"):
                for nme, c in (("q", H * d), ("k", G * d), ("v", G * dv)):
                    f = rnd(c, le["conv"], std=0.4)
                    f[:, -1] += 1.0
                    w[p + f"mix.left.{nme}.conv"] = f
            H, d, dv = ri["heads"], ri["dim"], ri["vdim"]
            # a retention's first tokens read out v (k . q) and are then brought to unit size: where k . q is
            # near zero, rounding decides its sign.  Keys that lean towards the queries keep it positive.
            rq = mat(H * d, W, 1.5)
            w.update({p + "mix.right.q": rq, p + "mix.right.k": 0.8 * rq + mat(H * d, W, 0.5),
                      p + "mix.right.v": mat(H * dv, W, 1.2), p + "mix.right.g": mat(H * dv, W, 1.5),
                      p + "mix.right.o": mat(W, H * dv, 1.0)})
        mlp = L.get("mlp")
        if mlp:
            E, F = mlp["router"]["experts"], mlp["expert"]["ff"]
            w.update(norm(p + "norm2", W))
            w.update(norm(p + "norm2b", W, w_out=True))
            router = torch.zeros(E, W)
            for e in range(E):
                router[e, e] = 2.0
            w[p + "mlp.router"] = router
            w[p + "mlp.router.b"] = rnd(E, std=0.01)
            for e in range(E):
                w[p + f"mlp.e{e}.gate"] = mat(F, W, 1.2)
                w[p + f"mlp.e{e}.up"] = mat(F, W, 1.2)
                w[p + f"mlp.e{e}.down"] = mat(W, F, 1.0)
        if side:
            w.update({p + "side.gate": mat(side, W, 1.5), p + "side.proj": mat(W, side, 1.0),
                      p + "side.norm": clear(0.5 + rnd(W, std=0.1))})
    return w


def write_folder(cfg: dict, folder: str, seed: int, weights: Dict[str, torch.Tensor] = None) -> str:
    """config.json and model.safetensors (bfloat16) of ``cfg`` in ``folder``."""
    from swifttransformer_amd.weights.safetensors_io import save_safetensors
    os.makedirs(folder, exist_ok=True)
    w = weights if weights is not None else make_weights(cfg, seed)
    save_safetensors(os.path.join(folder, "model.safetensors"),
                     {k: v.to(torch.bfloat16).contiguous() for k, v in w.items()}, {"format": "pt"})
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f, indent=1)
    return folder


def prompt(length: int, vocab: int, seed: int):
    g = torch.Generator().manual_seed(9100 + seed)
    return torch.randint(0, vocab, (length,), generator=g).tolist()
