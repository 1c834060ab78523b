"""Small Pupalix configurations for the tests, with weights made here, large enough that every mechanism moves
the logits, and a router whose choices rest on no close call.

A: three streams; a hashed pair table; a latent layer (rank 20 and a turned part of 8, frequencies and amplitude
   rescaled; a dense feed-forward), an attention layer (4 heads on 2 key heads, chunks of 12, capped scores;
   6 experts in 3 groups of which 2 are kept, 2 a token) and a lightning layer without feed-forward; layers 1
   and 2 run twice; logits with a factor and a limit.
B: one stream (still read and written through its weights); sizes that no vector load divides (width 72, heads
   of 10 and 6, a lightning head of 5 x 18, experts of 20, a dense width of 50); an attention without chunks
   and without a cap; all experts a token, no groups; no repeated group; no limit on the logits.
C: no streams at all (the plain residual sum) and no pair table; 8 heads on one key head with chunks of 64; a
   lightning layer with wide keys and a decay of 1; a latent layer whose turned part is as large as its keys;
   one expert a token from the one kept group of four; the whole model is one group that runs once.
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict

import torch


def _latent(heads, dim, rot_dim, vdim, rank, scale, base=100.0, scaling=None):
    rot = {"base": base, "dims": rot_dim}
    if scaling is not None:
        rot["scaling"] = scaling
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank, "scale": scale, "rot": rot}}


def _attention(heads, kv, dim, scale, softcap=None, chunk=None):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": dim, "scale": scale}
    if softcap is not None:
        m["softcap"] = softcap
    if chunk is not None:
        m["mask"] = {"size": chunk}
    return {"type": "attention", "mixer": m}


def _lightning(heads, dim, vdim, decay):
    return {"type": "lightning", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": decay}}


def _moe(experts, top, ff, groups=None):
    r = {"experts": experts, "top": top}
    if groups is not None:
        r["groups"] = {"count": groups[0], "keep": groups[1]}
    return {"kind": "moe", "router": r, "expert": {"ff": ff}}


def _dense(ff):
    return {"kind": "dense", "ff": ff}


def _with(layer, mlp):
    return dict(layer, mlp=mlp)


CONFIGS = {
    "A": {"architecture": "Pupalix", "vocab": 97, "width": 64, "max_positions": 512, "norm": {"eps": 1e-6}, "streams": 3,
          "embedding": {"scale": 3.0, "bigram": {"buckets": 53, "mul_prev": 5, "mul_cur": 11}},
          "logit_scale": 1.5, "logit_softcap": 8.0, "loop": {"start": 1, "stop": 3, "times": 2},
          "layers": [_with(_latent(2, 24, 8, 16, 20, 0.3, scaling={"factor": 2.0, "original": 16, "fast": 4.0, "slow": 1.0}),
                           _dense(48)),
                     _with(_attention(4, 2, 16, 0.4, softcap=5.0, chunk=12), _moe(6, 2, 24, groups=(3, 2))),
                     _with(_lightning(2, 12, 20, [0.9, 0.995]), None)]},
    "B": {"architecture": "Pupalix", "vocab": 131, "width": 72, "max_positions": 512, "norm": {"eps": 1e-4}, "streams": 1,
          "embedding": {"scale": 0.5, "bigram": {"buckets": 7, "mul_prev": 1, "mul_cur": 1}}, "logit_scale": 1.0,
          "layers": [_with(_attention(3, 3, 10, 0.5), _moe(5, 5, 20)),
                     _with(_lightning(1, 5, 18, [0.75]), _dense(50)),
                     _with(_latent(3, 10, 6, 14, 30, 0.35, base=50.0), _moe(4, 1, 20, groups=(2, 2)))]},
    "C": {"architecture": "Pupalix", "vocab": 61, "width": 128, "max_positions": 512, "norm": {"eps": 1e-5},
          "embedding": {"scale": 2.0}, "logit_scale": 0.7, "logit_softcap": 20.0, "loop": {"start": 0, "stop": 3, "times": 1},
          "layers": [_with(_attention(8, 1, 32, 0.25, softcap=25.0, chunk=64), _moe(8, 1, 40, groups=(4, 1))),
                     _with(_lightning(4, 64, 16, [0.5, 0.9, 0.99, 1.0]), _dense(96)),
                     _with(_latent(8, 16, 16, 32, 64, 0.2, base=1000.0,
                                   scaling={"factor": 8.0, "original": 32, "fast": 8.0, "slow": 0.5}), None)]},
}
PAGE_SIZE = {"A": 4, "B": 2, "C": 16}


def reserved(cfg: dict) -> int:
    """The first coordinates of the stream hold a code of the token that only the routers read."""
    return max([L["mlp"]["router"]["experts"] for L in cfg["layers"] if (L.get("mlp") or {}).get("kind") == "moe"] or [0])


def make_weights(cfg: dict, seed: int) -> Dict[str, torch.Tensor]:
    """float32 tensors by name.  The embedding's first ``reserved`` coordinates are a code of the token's id
    (levels from 1 down to -1, the highest at id % experts); the pair table and every matrix that writes into
    the stream are zero there, the streams' weights are positive, and a router reads nothing else: a token's
    experts follow from its id by a wide margin in every pass."""
    g = torch.Generator().manual_seed(seed)
    W, V = cfg["width"], cfg["vocab"]
    R = reserved(cfg)
    S = cfg.get("streams")
    rnd = lambda *shape, std=1.0: torch.randn(*shape, generator=g) * std
    mat = lambda out, inp, gain=1.0: rnd(out, inp, std=gain / math.sqrt(inp))

    def writes(t):                # a matrix whose result enters the stream: nothing into the reserved coordinates
        t[:R] = 0.0
        return t

    def gain(width):
        w = 1.0 + rnd(width, std=0.2)
        w[:R] = 1.0
        return w

    scale = cfg["embedding"].get("scale", 1.0)
    emb = rnd(V, W) * (1.0 / max(scale, 1.0))
    for t in range(V):
        for e in range(R):
            emb[t, e] = (1.0 - 2.0 * ((e - t) % R) / max(R - 1, 1)) / scale
    w = {"embed": emb, "final.norm": gain(W)}
    big = cfg["embedding"].get("bigram")
    if big:
        table = rnd(big["buckets"] + 1, W, std=0.7)
        table[:, :R] = 0.0
        w["bigram"] = table
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        w[p + "norm1"] = gain(W)
        if L["type"] == "latent_attention":
            H, d, r, dv, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
            w.update({p + "mix.q": mat(H * (d + r), W, 1.5), p + "mix.dkv": mat(rank + r, W, 1.5),
                      p + "mix.dkv.norm": 1.0 + rnd(rank, std=0.2), p + "mix.uk": mat(H * d, rank, 1.5),
                      p + "mix.uv": mat(H * dv, rank, 1.2), p + "mix.o": writes(mat(W, H * dv, 1.0))})
        elif L["type"] == "attention":
            H, G, d = m["heads"], m["kv_heads"], m["dim"]
            w.update({p + "mix.q": mat(H * d, W, 1.5), p + "mix.k": mat(G * d, W, 1.5),
                      p + "mix.q.norm": 1.0 + rnd(H * d, std=0.3), p + "mix.k.norm": 1.0 + rnd(G * d, std=0.3),
                      p + "mix.o": writes(mat(W, H * d, 1.0))})
        else:
            H, d, dv = m["heads"], m["dim"], m["vdim"]
            # a read-out is a sum of v (k . q) and is then normalised: where the k . q of the few tokens that a fast
            # decay leaves cancel, rounding decides the direction.  Keys that lean towards the queries keep them positive.
            rq = mat(H * d, W, 1.5)
            w.update({p + "mix.q": rq, p + "mix.k": 0.8 * rq + mat(H * d, W, 0.5), p + "mix.v": mat(H * dv, W, 1.2),
                      p + "mix.g": mat(H * dv, W, 1.5), p + "mix.norm": 1.0 + rnd(H * dv, std=0.2),
                      p + "mix.o": writes(mat(W, H * dv, 1.0))})
        mlp = L.get("mlp")
        if mlp:
            w[p + "norm2"] = gain(W)
            if mlp["kind"] == "dense":
                F = mlp["ff"]
                w.update({p + "mlp.gate": mat(F, W, 1.2), p + "mlp.up": mat(F, W, 1.2), p + "mlp.down": writes(mat(W, F, 1.0))})
            else:
                E, F = mlp["router"]["experts"], mlp["expert"]["ff"]
                router = torch.zeros(E, W)
                for e in range(E):
                    router[e, e] = 2.0
                w[p + "mlp.router"] = router
                for e in range(E):
                    w[p + f"mlp.e{e}.gate"] = mat(F, W, 1.2)
                    w[p + f"mlp.e{e}.up"] = mat(F, W, 1.2)
                    w[p + f"mlp.e{e}.down"] = writes(mat(W, F, 1.5))
        if S:
            for hc in ("hc1", "hc2") if mlp else ("hc1",):
                w[p + hc + ".in"] = 1.0 / S + torch.rand(S, generator=g) * 0.5
                w[p + hc + ".out"] = 0.6 + torch.rand(S, generator=g) * 0.8 - (torch.arange(S) % 2) * 0.5
                w[p + hc + ".mix"] = torch.eye(S) * 0.8 + torch.rand(S, S, generator=g) * 0.3
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
    g = torch.Generator().manual_seed(7300 + seed)
    return torch.randint(0, vocab, (length,), generator=g).tolist()
