"""A plain, slow Pupalix in float64 on the CPU, one function a mechanism, written from the design's
equations and sharing no code with the engine.  ``PlainPupalix(config, tensors)`` runs whole sequences;
``layers=True`` also returns the sum of the streams after every run of a layer."""
from __future__ import annotations

import math
from typing import Dict, List

import torch

F = torch.float64


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def bigram_rows(tokens: List[int], buckets: int, mul_prev: int, mul_cur: int) -> List[int]:
    """Row of the bigram table for every token: the last row for a sequence's first token."""
    return [buckets if i == 0 else (tokens[i - 1] * mul_prev + t * mul_cur) % buckets for i, t in enumerate(tokens)]


def embed(tokens, table, scale, bigram=None, rule=None):
    x = table[tokens] * scale
    if bigram is not None:
        x = x + bigram[bigram_rows(tokens, rule["buckets"], rule["mul_prev"], rule["mul_cur"])]
    return x


def yarn_frequencies(dims, base, scaling):
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    if not scaling:
        return f, 1.0
    factor, orig = scaling["factor"], scaling["original"]
    d = lambda t: dims * math.log(orig / (2 * math.pi * t)) / (2 * math.log(base))
    lo = max(math.floor(d(scaling["fast"])), 0)
    hi = min(math.ceil(d(scaling["slow"])), dims - 1)
    out = []
    for i, fi in enumerate(f):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(fi / factor * ramp + fi * (1 - ramp))
    return out, 0.1 * math.log(factor) + 1.0


def turn_pairs(x, positions, freq, mult):
    """x [..., T, n]: the first 2 len(freq) coordinates in pairs (2i, 2i + 1) by position * freq[i]."""
    n = 2 * len(freq)
    a = torch.tensor(positions, dtype=F)[:, None] * torch.tensor(freq, dtype=F)[None, :]
    c, s = torch.cos(a) * mult, torch.sin(a) * mult
    u, v = x[..., 0:n:2], x[..., 1:n:2]
    out = x.clone()
    out[..., 0:n:2] = u * c - v * s
    out[..., 1:n:2] = v * c + u * s
    return out


def softmax_rows(scores, visible):
    scores = scores.masked_fill(~visible, float("-inf"))
    return torch.softmax(scores, dim=-1)


def latent_attention(h, w, m, eps, positions):
    T = h.shape[0]
    H, d, r, vd, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    q = (h @ w["q"].T).view(T, H, d + r)
    dkv = h @ w["dkv"].T
    c = rms(dkv[:, :R], eps) * w["dkv.norm"]
    k_rot = dkv[:, R:]
    if r:
        rot = m["rot"]
        freq, mult = yarn_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
        k_rot = turn_pairs(k_rot, positions, freq, mult)
        q_rot = turn_pairs(q[:, :, d:].transpose(0, 1), positions, freq, mult).transpose(0, 1)
    k = (c @ w["uk"].T).view(T, H, d)
    v = (c @ w["uv"].T).view(T, H, vd)
    s = torch.einsum("ihd,jhd->hij", q[:, :, :d], k)
    if r:
        s = s + torch.einsum("ihd,jd->hij", q_rot, k_rot)
    s = s * m["scale"]
    i, j = torch.arange(T)[:, None], torch.arange(T)[None, :]
    p = softmax_rows(s, (j <= i)[None])
    o = torch.einsum("hij,jhv->ihv", p, v).reshape(T, H * vd)
    return o @ w["o"].T


def tied_attention(h, w, m, eps):
    T = h.shape[0]
    H, G, d = m["heads"], m["kv_heads"], m["dim"]
    q_raw, k_raw = h @ w["q"].T, h @ w["k"].T
    q = (rms(q_raw, eps) * w["q.norm"]).view(T, H, d)
    k = (rms(k_raw, eps) * w["k.norm"]).view(T, G, d)
    v = k_raw.view(T, G, d)
    rep = H // G
    k, v = k.repeat_interleave(rep, dim=1), v.repeat_interleave(rep, dim=1)
    s = torch.einsum("ihd,jhd->hij", q, k) * m["scale"]
    cap = m.get("softcap")
    if cap:
        s = cap * torch.tanh(s / cap)
    i, j = torch.arange(T)[:, None], torch.arange(T)[None, :]
    visible = j <= i
    size = (m.get("mask") or {}).get("size")
    if size:
        visible = visible & (i // size == j // size)
    p = softmax_rows(s, visible[None])
    o = torch.einsum("hij,jhv->ihv", p, v).reshape(T, H * d)
    return o @ w["o"].T


def lightning(h, w, m, eps):
    T = h.shape[0]
    H, d, vd = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ w["q"].T).view(T, H, d)
    k = silu(h @ w["k"].T).view(T, H, d)
    v = silu(h @ w["v"].T).view(T, H, vd)
    decay = torch.tensor(m["decay"], dtype=F)
    S = torch.zeros(H, d, vd, dtype=F)
    out = torch.zeros(T, H, vd, dtype=F)
    for t in range(T):
        S = decay[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hdv,hd->hv", S, q[t])
    y = rms(out.reshape(T, H * vd), eps) * w["norm"] * torch.sigmoid(h @ w["g"].T)
    return y @ w["o"].T


def dense_ff(h, w):
    return (gelu_tanh(h @ w["gate"].T) * (h @ w["up"].T)) @ w["down"].T


def route(scores, top, groups, keep):
    """scores [experts] -> the chosen experts: the ``top`` largest among the experts of the ``keep`` groups
    whose largest score is largest."""
    E = scores.shape[0]
    per = E // groups
    best = scores.view(groups, per).max(dim=1).values
    kept = torch.topk(best, keep).indices.tolist()
    allowed = torch.full((E,), float("-inf"), dtype=F)
    for g in kept:
        allowed[g * per:(g + 1) * per] = scores[g * per:(g + 1) * per]
    return torch.topk(allowed, top).indices.tolist()


def moe_ff(h, w, mlp):
    r = mlp["router"]
    E, top = r["experts"], r["top"]
    grp = r.get("groups") or {"count": 1, "keep": 1}
    z = h @ w["router"].T
    s = torch.softmax(z, dim=-1)
    out = torch.zeros(h.shape[0], w["e0.down"].shape[0], dtype=F)
    for t in range(h.shape[0]):
        for e in route(s[t], top, grp["count"], grp["keep"]):
            y = (silu(h[t] @ w[f"e{e}.gate"].T) * (h[t] @ w[f"e{e}.up"].T)) @ w[f"e{e}.down"].T
            out[t] += s[t, e] * y
    return out


def hyper_step(xs, hc, sublayer, norm_w, eps):
    """xs [S, T, W]: one sublayer under hyper-connections."""
    u = torch.einsum("s,stw->tw", hc["in"], xs)
    y = sublayer(rms(u, eps) * norm_w)
    return torch.einsum("sr,stw->rtw", hc["mix"], xs) + hc["out"][:, None, None] * y[None]


def head(x, table, norm_w, eps, logit_scale, cap):
    z = (rms(x, eps) * norm_w) @ table.T * logit_scale
    return cap * torch.tanh(z / cap) if cap else z


def run_order(cfg):
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return list(range(n))
    a, b, times = loop["start"], loop["stop"], loop["times"]
    return list(range(a)) + list(range(a, b)) * times + list(range(b, n))


class PlainPupalix:
    def __init__(self, cfg: dict, tensors: Dict[str, torch.Tensor]):
        self.cfg = cfg
        self.t = {k: (v.to(F) if v.is_floating_point() else v) for k, v in tensors.items()}

    def sub(self, prefix):
        n = len(prefix)
        return {k[n:]: v for k, v in self.t.items() if k.startswith(prefix)}

    def forward(self, tokens: List[int], layers: bool = False):
        cfg, t = self.cfg, self.t
        eps = cfg["norm"]["eps"]
        T = len(tokens)
        positions = list(range(T))
        emb = cfg["embedding"]
        x = embed(tokens, t["embed"], emb.get("scale", 1.0), t.get("bigram"), emb.get("bigram"))
        S = cfg.get("streams")
        xs = torch.stack([x] * S) if S else None
        after = []
        for i in run_order(cfg):
            L = cfg["layers"][i]
            m, mlp = L["mixer"], L.get("mlp")
            wm, wf = self.sub(f"l{i}.mix."), self.sub(f"l{i}.mlp.")
            if L["type"] == "latent_attention":
                mixer = lambda h: latent_attention(h, wm, m, eps, positions)
            elif L["type"] == "attention":
                mixer = lambda h: tied_attention(h, wm, m, eps)
            elif L["type"] == "lightning":
                mixer = lambda h: lightning(h, wm, m, eps)
            else:
                raise ValueError(L["type"])
            ff = None
            if mlp is not None:
                ff = (lambda h: dense_ff(h, wf)) if mlp["kind"] == "dense" else (lambda h: moe_ff(h, wf, mlp))
            if S:
                xs = hyper_step(xs, self.sub(f"l{i}.hc1."), mixer, t[f"l{i}.norm1"], eps)
                if ff is not None:
                    xs = hyper_step(xs, self.sub(f"l{i}.hc2."), ff, t[f"l{i}.norm2"], eps)
                x = xs.sum(0)
            else:
                x = x + mixer(rms(x, eps) * t[f"l{i}.norm1"])
                if ff is not None:
                    x = x + ff(rms(x, eps) * t[f"l{i}.norm2"])
            after.append(x.clone())
        logits = head(x, t["embed"], t["final.norm"], eps, cfg.get("logit_scale", 1.0), cfg.get("logit_softcap"))
        return (logits, torch.stack(after)) if layers else logits


def load_folder(folder: str):
    """(config, float64 tensors by name) of a model folder, through this file's own reader."""
    import json
    import os
    import struct
    import numpy as np
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    with open(os.path.join(folder, "model.safetensors"), "rb") as f:
        n = struct.unpack("<Q", f.read(8))[0]
        meta = json.loads(f.read(n))
        data = f.read()
    out = {}
    for name, m in meta.items():
        if name == "__metadata__":
            continue
        a, b = m["data_offsets"]
        raw = np.frombuffer(data[a:b], dtype=np.uint8)
        if m["dtype"] == "BF16":
            u = raw.view("<u2").astype(np.uint32) << 16
            t = torch.from_numpy(u.view(np.float32).copy())
        elif m["dtype"] == "F32":
            t = torch.from_numpy(raw.view("<f4").copy())
        else:
            raise ValueError(m["dtype"])
        out[name] = t.reshape(m["shape"]).to(F)
    return cfg, out


def logits(cfg, w, tokens):
    with torch.no_grad():
        return PlainPupalix(cfg, w).forward(list(tokens))


def residual_streams(cfg, w, tokens):
    with torch.no_grad():
        return PlainPupalix(cfg, w).forward(list(tokens), layers=True)[1]


def generate(cfg, w, prompt, n):
    seq, out = list(prompt), []
    for _ in range(n):
        tok = int(logits(cfg, w, seq)[-1].argmax())
        out.append(tok)
        seq.append(tok)
    return out
