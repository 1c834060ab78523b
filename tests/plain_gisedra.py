"""A plain float64 Gisedra: one function a mechanism, written from the design's equations, slow and
literal.  It shares nothing with the engine: tensors come in as a dict name -> torch tensor, the
configuration as the dict that config.json holds.

Notation: T tokens of one sequence, positions 0 .. T-1; h [T, width] is what a sublayer reads.

    dynamic tanh            n(x) = tanh(alpha x) * w + b                       (no mean, no variance)
    layer                   x += n1b(mix(n1(x)));  x += n2b(ffn(n2(x)));  x += side(x, token)
    side input              e = E[token, i*d:(i+1)*d];  y = P (gelu(G x) * e);  side = y / rms(y) * s
    passes                  layers a..b-1 run `times` times; before pass t: x += embedding (t > 0), x += step[t]
"""
from __future__ import annotations

import json
import math
import os
import struct
from typing import Dict, List, Optional

import numpy as np
import torch

F64 = torch.float64


# ----------------------------------------------------------------------------- files
def read_safetensors(path: str) -> Dict[str, torch.Tensor]:
    """8-byte little-endian header length, JSON header, raw data: name -> float64 (or int64) tensor."""
    with open(path, "rb") as f:
        (n,) = struct.unpack("<Q", f.read(8))
        header = json.loads(f.read(n))
        blob = f.read()
    out = {}
    for name, info in header.items():
        if name == "__metadata__":
            continue
        lo, hi = info["data_offsets"]
        raw = np.frombuffer(blob[lo:hi], dtype=np.uint8)
        if info["dtype"] == "BF16":
            t = torch.from_numpy((raw.view("<u2").astype(np.uint32) << 16).view(np.float32).astype(np.float64))
        elif info["dtype"] == "F32":
            t = torch.from_numpy(raw.view("<f4").astype(np.float64))
        elif info["dtype"] == "I32":
            t = torch.from_numpy(raw.view("<i4").astype(np.int64))
        else:
            raise ValueError(f"{name}: dtype {info['dtype']}")
        out[name] = t.reshape(info["shape"])
    return out


def load_folder(folder: str):
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    return cfg, read_safetensors(os.path.join(folder, "model.safetensors"))


# ----------------------------------------------------------------------------- small functions
def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def unit_rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def dynamic_tanh(x, w, b, alpha):
    return torch.tanh(alpha * x) * w + b


def causal_filter(u, w):
    """u [T, C], w [C, taps]: y_t = sum_j w[:, j] u_(t - taps + 1 + j), zeros before the start."""
    T, C = u.shape
    taps = w.shape[1]
    y = torch.zeros_like(u)
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] += w[:, j] * u[s]
    return y


# ----------------------------------------------------------------------------- rotation
def rotary_frequencies(dims: int, base: float, scaling: Optional[dict] = None) -> List[float]:
    """f_i = base^(-2i/dims); with ``scaling`` {factor, low, high, original}: by wavelength l = 2 pi / f,
    short waves (l < original / high) keep f, long ones (l > original / low) get f / factor, and those
    between are blended by s = (original / l - low) / (high - low)."""
    out = []
    for i in range(dims // 2):
        f = float(base) ** (-2.0 * i / dims)
        if scaling:
            factor, low, high = float(scaling["factor"]), float(scaling["low"]), float(scaling["high"])
            orig = float(scaling["original"])
            l = 2.0 * math.pi / f
            if l < orig / high:
                pass
            elif l > orig / low:
                f = f / factor
            else:
                s = (orig / l - low) / (high - low)
                f = (1.0 - s) * f / factor + s * f
        out.append(f)
    return out


def rotate(x, positions, freqs, interleaved: bool):
    """x [T, heads, n]: the first 2 len(freqs) coordinates of each head are turned by positions * freqs.
    Pairs are (i, i + half) or, ``interleaved``, (2i, 2i + 1)."""
    half = len(freqs)
    a = positions.to(F64)[:, None] * torch.tensor(freqs, dtype=F64)[None, :]      # [T, half]
    c, s = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
    y = x.clone()
    if interleaved:
        u, v = x[..., 0:2 * half:2], x[..., 1:2 * half:2]
        y[..., 0:2 * half:2] = u * c - v * s
        y[..., 1:2 * half:2] = v * c + u * s
    else:
        u, v = x[..., :half], x[..., half:2 * half]
        y[..., :half] = u * c - v * s
        y[..., half:2 * half] = v * c + u * s
    return y


# ----------------------------------------------------------------------------- attention
def visible(T: int, size: int, keep_first: int = 0):
    """[T, T] bool: i sees j when j <= i and (i - j < size or j < keep_first); size 0: every j <= i."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    near = (i - j < size) if size > 0 else torch.ones(T, T, dtype=torch.bool)
    return (j <= i) & (near | (j < keep_first))


def softmax_attention(q, k, v, scale, mask):
    """q [T, H, d], k [T, G, d], v [T, G, dv]; query head h reads key head h // (H / G)."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=F64)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        s = s.masked_fill(~mask, float("-inf"))
        out[:, h] = torch.softmax(s, dim=-1) @ v[:, g]
    return out


def gated_window_attention(h, W: Dict[str, torch.Tensor], p: str, c: dict):
    """Grouped softmax attention with a short filter over time on q, k and v, partial rotation, a sliding
    window that keeps the first tokens, and a sigmoid gate on the heads' outputs."""
    T = h.shape[0]
    H, G, d, dv = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
    q, k, v = h @ W[p + ".q"].T, h @ W[p + ".k"].T, h @ W[p + ".v"].T
    if c.get("conv"):
        q, k, v = (causal_filter(u, W[f"{p}.{n}.conv"]) for u, n in ((q, "q"), (k, "k"), (v, "v")))
    q, k, v = q.view(T, H, d), k.view(T, G, d), v.view(T, G, dv)
    rot = c.get("rot")
    if rot:
        f = rotary_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
        pos = torch.arange(T)
        q, k = rotate(q, pos, f, False), rotate(k, pos, f, False)
    mask = c.get("mask") or {}
    o = softmax_attention(q, k, v, c["scale"], visible(T, mask.get("size", 0), mask.get("keep_first", 0)))
    o = o.reshape(T, H * dv) * torch.sigmoid(h @ W[p + ".g"].T)
    return o @ W[p + ".o"].T


def retention(h, W: Dict[str, torch.Tensor], p: str, c: dict, eps: float):
    """S_t = decay S_(t-1) + k_t v_t^T, o_t = S_t^T q_t per head; no softmax, no denominator."""
    T = h.shape[0]
    H, d, dv = c["heads"], c["dim"], c["vdim"]
    q = (h @ W[p + ".q"].T).view(T, H, d)
    k = (h @ W[p + ".k"].T).view(T, H, d) * d ** -0.5
    v = (h @ W[p + ".v"].T).view(T, H, dv)
    o = torch.zeros(T, H, dv, dtype=F64)
    for n in range(H):
        S = torch.zeros(d, dv, dtype=F64)
        for t in range(T):
            S = float(c["decay"][n]) * S + torch.outer(k[t, n], v[t, n])
            o[t, n] = S.T @ q[t, n]
    o = unit_rms(o, eps).reshape(T, H * dv) * silu(h @ W[p + ".g"].T)
    return o @ W[p + ".o"].T


def parallel_mixer(h, W, p: str, c: dict, eps: float):
    return (c["left_scale"] * gated_window_attention(h, W, p + ".left", c["left"]) +
            c["right_scale"] * retention(h, W, p + ".right", c["right"], eps))


def latent_attention(h, W: Dict[str, torch.Tensor], p: str, c: dict, eps: float):
    """Keys and values of all heads come from one normed latent a token; one small rotated key part is
    shared by the heads.  A query head is [dim plain | rot_dim turned]."""
    T = h.shape[0]
    H, d, r, dv, R = c["heads"], c["dim"], c["rot_dim"], c["vdim"], c["kv_rank"]
    q = (h @ W[p + ".q"].T).view(T, H, d + r)
    down = h @ W[p + ".dkv"].T
    lat = unit_rms(down[:, :R], eps) * W[p + ".dkv.norm"]
    f = rotary_frequencies(c["rot"]["dims"], c["rot"]["base"], c["rot"].get("scaling"))
    pos = torch.arange(T)
    k_rot = rotate(down[:, R:].view(T, 1, r), pos, f, True)
    q_rot = rotate(q[..., d:], pos, f, True)
    k_plain = (lat @ W[p + ".uk"].T).view(T, H, d)
    v = (lat @ W[p + ".uv"].T).view(T, H, dv)
    mask = visible(T, (c.get("mask") or {}).get("size", 0))
    out = torch.zeros(T, H, dv, dtype=F64)
    for n in range(H):
        s = (q[:, n, :d] @ k_plain[:, n].T + q_rot[:, n] @ k_rot[:, 0].T) * c["scale"]
        s = s.masked_fill(~mask, float("-inf"))
        out[:, n] = torch.softmax(s, dim=-1) @ v[:, n]
    return out.reshape(T, H * dv) @ W[p + ".o"].T


# ----------------------------------------------------------------------------- feed-forward, side input
def routed_experts(h, W: Dict[str, torch.Tensor], p: str, c: dict):
    """The ``top`` largest router logits choose a token's experts; their weights are the softmax over
    those logits alone; an expert is down(silu(gate h) * (up h))."""
    E, top = c["router"]["experts"], c["router"]["top"]
    z = h @ W[p + ".router"].T + W[p + ".router.b"]
    out = torch.zeros(h.shape[0], W[f"{p}.e0.down"].shape[0], dtype=F64)
    for t in range(h.shape[0]):
        best = sorted(range(E), key=lambda e: (-float(z[t, e]), e))[:top]
        w = torch.softmax(z[t, best], dim=0)
        for wi, e in zip(w, best):
            y = silu(W[f"{p}.e{e}.gate"] @ h[t]) * (W[f"{p}.e{e}.up"] @ h[t])
            out[t] += wi * (W[f"{p}.e{e}.down"] @ y)
    return out


def side_input(x, tokens, W, i: int, dim: int, eps: float):
    e = W["side.embed"][tokens][:, i * dim:(i + 1) * dim]
    g = gelu_tanh(x @ W[f"l{i}.side.gate"].T) * e
    y = g @ W[f"l{i}.side.proj"].T
    return unit_rms(y, eps) * W[f"l{i}.side.norm"]


# ----------------------------------------------------------------------------- the model
def _norm(x, W, name):
    return dynamic_tanh(x, W[name], W[name + ".b"], W[name + ".alpha"])


def run_order(cfg: dict):
    """[(layer, pass number or None)]: a pass number at the first layer of each pass."""
    n, loop = len(cfg["layers"]), cfg.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    a, b, times = loop["start"], loop["stop"], loop["times"]
    order = [(i, None) for i in range(a)]
    for t in range(times):
        order += [(i, t if i == a else None) for i in range(a, b)]
    return order + [(i, None) for i in range(b, n)]


def layer(x, tokens, W, cfg: dict, i: int):
    L, eps, p = cfg["layers"][i], cfg["norm"]["eps"], f"l{i}"
    h = _norm(x, W, p + ".norm1")
    if L["type"] == "parallel":
        m = parallel_mixer(h, W, p + ".mix", L["mixer"], eps)
    else:
        m = latent_attention(h, W, p + ".mix", L["mixer"], eps)
    x = x + _norm(m, W, p + ".norm1b")
    if L.get("mlp") is not None:
        x = x + _norm(routed_experts(_norm(x, W, p + ".norm2"), W, p + ".mlp", L["mlp"]), W, p + ".norm2b")
    side = cfg.get("token_side")
    if side:
        x = x + side_input(x, tokens, W, i, side["dim"], eps)
    return x


def forward(tokens, weights: Dict[str, torch.Tensor], cfg: dict, streams: Optional[list] = None):
    """float64 logits [T, vocab] of one sequence; ``streams`` collects the residual stream after every
    run of a layer."""
    W = {k: (v.to(F64) if v.is_floating_point() else v) for k, v in weights.items()}
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    first = x = W["embed"][tokens]
    for i, pass_no in run_order(cfg):
        if pass_no is not None:
            if pass_no > 0:
                x = x + first
            x = x + W["loop.step"][pass_no]
        x = layer(x, tokens, W, cfg, i)
        if streams is not None:
            streams.append(x.clone())
    return _norm(x, W, "final.norm") @ W["head"].T


def logits(cfg: dict, w: Dict[str, torch.Tensor], tokens) -> torch.Tensor:
    return forward(tokens, w, cfg)


def residual_streams(cfg: dict, w: Dict[str, torch.Tensor], tokens) -> List[torch.Tensor]:
    out: List[torch.Tensor] = []
    forward(tokens, w, cfg, out)
    return out


def generate(cfg: dict, w: Dict[str, torch.Tensor], prompt, n: int) -> List[int]:
    """Greedy continuation of ``prompt`` by ``n`` tokens (the lowest id on ties)."""
    seq, out = list(prompt), []
    for _ in range(n):
        nxt = int(torch.argmax(logits(cfg, w, seq)[-1]))
        out.append(nxt)
        seq.append(nxt)
    return out
