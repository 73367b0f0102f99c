"""Plain, slow model of the Nopunex design, written from its equations: one function per
mechanism, one whole sequence at a time, no cache, no batching, double precision.
The tests compare the framework with it; it shares no code with the package.

Notation: a sequence is ``x[t, :]`` for t = 0..n-1 (positions count from 0), ``W`` are [out, in]
matrices applied as ``W @ v``.  ``cfg`` is the parsed config.json, ``w`` a dict name -> tensor.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

DT = torch.float64


def layer_norm(x: torch.Tensor, g: torch.Tensor, b: torch.Tensor, eps: float) -> torch.Tensor:
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * g + b


def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def softplus(z: torch.Tensor) -> torch.Tensor:
    return torch.log1p(torch.exp(-z.abs())) + z.clamp(min=0)


# ------------------------------------------------------------------ rotations
def rotary_frequencies(rot: dict):
    """Per pair i of ``dims`` / 2: the angle per position, and the factor on cos / sin."""
    dims, base = int(rot["dims"]), float(rot["base"])
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    sc = rot.get("scaling")
    if not sc:
        return torch.tensor(f, dtype=DT), 1.0
    factor, orig = float(sc["factor"]), float(sc["original"])
    at = lambda turns: dims * math.log(orig / (2 * math.pi * turns)) / (2 * math.log(base))
    lo = max(math.floor(at(float(sc["fast"]))), 0)
    hi = min(math.ceil(at(float(sc["slow"]))), dims - 1)
    out = []
    for i in range(dims // 2):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f[i] / factor * ramp + f[i] * (1 - ramp))
    return torch.tensor(out, dtype=DT), 0.1 * math.log(factor) + 1.0


def rotate_halves(x: torch.Tensor, pos: torch.Tensor, freq: torch.Tensor, mag: float) -> torch.Tensor:
    """x[..., i] and x[..., i + n2] (n2 = len(freq)) of the first 2 n2 coordinates turn by
    pos * freq[i]; the rest pass.  x: [n, heads, d], pos: [n]."""
    n2 = freq.numel()
    ang = pos.to(DT)[:, None] * freq[None, :]
    c, s = (torch.cos(ang) * mag)[:, None, :], (torch.sin(ang) * mag)[:, None, :]
    out = x.clone()
    u, v = x[..., :n2], x[..., n2:2 * n2]
    out[..., :n2] = u * c - v * s
    out[..., n2:2 * n2] = v * c + u * s
    return out


# --------------------------------------------------------------------- mixers
def short_conv(x: torch.Tensor, taps: torch.Tensor) -> torch.Tensor:
    """Causal per-channel filter over time: y[t, c] = sum_j taps[c, j] x[t - (K - 1) + j, c], zeros
    before the start."""
    n, K = x.shape[0], taps.shape[1]
    y = torch.zeros_like(x)
    for j in range(K):
        back = K - 1 - j
        if back < n:
            y[back:] += x[:n - back] * taps[:, j]
    return y


def delta(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    """Gated delta rule: per head a [dim, vdim] memory that decays, is corrected towards the new
    value along the new key, and is read with the query."""
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    n = h.shape[0]
    q = silu(short_conv(h @ w[p + "q"].T, w[p + "q.conv"])).view(n, G, D)
    k = silu(short_conv(h @ w[p + "k"].T, w[p + "k.conv"])).view(n, G, D)
    v = silu(short_conv(h @ w[p + "v"].T, w[p + "v.conv"])).view(n, H, V)
    unit = lambda x: x / torch.sqrt((x * x).sum(-1, keepdim=True) + 1e-6)
    q, k = unit(q) * D ** -0.5, unit(k)
    beta = torch.sigmoid(h @ w[p + "b"].T)                                           # [n, H]
    g = torch.exp(-torch.exp(w[p + "A_log"]) * softplus(h @ w[p + "a"].T + w[p + "dt_bias"]))
    out = torch.zeros(n, H, V, dtype=DT)
    for a in range(H):
        kv = a // (H // G)
        S = torch.zeros(D, V, dtype=DT)
        for t in range(n):
            S = g[t, a] * S
            u = beta[t, a] * (v[t, a] - S.T @ k[t, kv])
            S = S + torch.outer(k[t, kv], u)
            out[t, a] = S.T @ q[t, kv]
    o = unit_rms(out, eps) * w[p + "norm"] * silu(h @ w[p + "g"].T).view(n, H, V)
    return o.reshape(n, H * V) @ w[p + "o"].T


def latent_attention(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    """Queries through a normed latent; keys and values expanded from a normed latent of the token
    plus one rotated key part shared by the heads; sliding window; a per-head sink in the softmax."""
    H, D, Dr, V, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    n = h.shape[0]
    pos = torch.arange(n)
    cq = unit_rms(h @ w[p + "dq"].T, eps) * w[p + "dq.norm"]
    q = (cq @ w[p + "uq"].T).view(n, H, D + Dr)
    dkv = h @ w[p + "dkv"].T
    c = unit_rms(dkv[:, :R], eps) * w[p + "dkv.norm"]
    kr = dkv[:, R:].view(n, 1, Dr)
    f, mag = rotary_frequencies(m["rot"])
    qr = rotate_halves(q[..., D:], pos, f, mag)
    kr = rotate_halves(kr, pos, f, mag)[:, 0]
    kn = (c @ w[p + "uk"].T).view(n, H, D)
    v = (c @ w[p + "uv"].T).view(n, H, V)
    size = int(m["mask"]["size"]) if m.get("mask") else n + 1
    out = torch.zeros(n, H, V, dtype=DT)
    for a in range(H):
        for i in range(n):
            lo = max(0, i - size + 1)
            s = (kn[lo:i + 1, a] @ q[i, a, :D] + kr[lo:i + 1] @ qr[i, a]) * m["scale"]
            e = torch.exp(s)
            out[i, a] = (e / (e.sum() + torch.exp(w[p + "sink"][a]))) @ v[lo:i + 1, a]
    return out.reshape(n, H * V) @ w[p + "o"].T


def diff_attention(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    """Two softmax maps per head over the same values, the second subtracted with one learned
    factor; keys visible inside the query's block of mask.size positions only; gated output."""
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    n = h.shape[0]
    pos = torch.arange(n)
    q = (h @ w[p + "q"].T).view(n, H * 2, D)
    k = (h @ w[p + "k"].T).view(n, G * 2, D)
    v = (h @ w[p + "v"].T).view(n, G, V)
    if m.get("rot"):
        f, mag = rotary_frequencies(m["rot"])
        q, k = rotate_halves(q, pos, f, mag), rotate_halves(k, pos, f, mag)
    diff = float(m["diff"])
    lam = torch.exp((w[p + "lq1"] * w[p + "lk1"]).sum()) - torch.exp((w[p + "lq2"] * w[p + "lk2"]).sum()) + diff
    size = int(m["mask"]["size"]) if m.get("mask") else n + 1
    out = torch.zeros(n, H, V, dtype=DT)
    for a in range(H):
        g = a // (H // G)
        for i in range(n):
            lo = (i // size) * size
            maps = []
            for mp in range(2):
                s = (k[lo:i + 1, 2 * g + mp] @ q[i, 2 * a + mp]) * m["scale"]
                maps.append(torch.softmax(s, 0) @ v[lo:i + 1, g])
            out[i, a] = maps[0] - lam * maps[1]
    o = unit_rms(out, eps) * (1 - diff)
    o = o.reshape(n, H * V) * torch.sigmoid(h @ w[p + "g"].T)
    return o @ w[p + "o"].T


MIXERS = {"delta": delta, "latent_attention": latent_attention, "attention": diff_attention}


def dense_ff(h, w, p):
    return (silu(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


# ---------------------------------------------------------------------- model
def run_order(cfg: dict) -> List[tuple]:
    """(layer, pass number or None, first of its pass) per layer run."""
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    if not lp:
        return [(i, None, False) for i in range(n)]
    a, b, times = int(lp["start"]), int(lp["stop"]), int(lp["times"])
    out = [(i, None, False) for i in range(a)]
    for t in range(times):
        out += [(i, t, i == a) for i in range(a, b)]
    return out + [(i, None, False) for i in range(b, n)]


def forward(cfg: dict, w: Dict[str, torch.Tensor], tokens, layers_out: Optional[list] = None) -> torch.Tensor:
    """Logits [n, vocab] of one sequence; ``layers_out`` collects the stream after every layer run."""
    w = {k: v.to(DT) for k, v in w.items()}
    eps = float(cfg["norm"]["eps"])
    x0 = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    x = x0
    for i, t, first in run_order(cfg):
        l, p = cfg["layers"][i], f"l{i}."
        if first:
            x = torch.cat([x, x0], -1) @ w["loop.in"].T + w["loop.step"][t]
        norm = lambda name, z: layer_norm(z, w[p + name], w[p + name + ".b"], eps)
        y = MIXERS[l["type"]](norm("norm1", x), w, p + "mix.", l["mixer"], eps)
        x = x + norm("norm1b", y)
        if l.get("mlp") is not None:
            x = x + norm("norm2b", dense_ff(norm("norm2", x), w, p + "mlp."))
        if layers_out is not None:
            layers_out.append(x)
    x = layer_norm(x, w["final.norm"], w["final.norm.b"], eps)
    return (x @ w["head"].T) * float(cfg.get("logit_scale", 1.0))


# ------------------------------------------------------- configurations and weights for tests
def make_config(vocab=80, width=48, pattern="AdMA", heads=4, kv_heads=2, dim=8, vdim=12, rot_dims=6, ff=40, chunk=16,
                window=24, kv_rank=20, q_rank=28, rot_dim=6, conv=3, loop=None, diff=0.3, scaling=(4.0, 64, 8.0, 1.0),
                logit_scale=1.5, eps=1e-5) -> dict:
    """``pattern``: A differential attention / M latent attention / D delta rule per layer, lower
    case without a feed-forward."""
    layers = []
    for ch in pattern:
        up = ch.upper()
        if up == "A":
            m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": dim ** -0.5, "diff": diff,
                 "mask": {"size": chunk}, "rot": {"dims": rot_dims, "base": 10000.0}}
            if not rot_dims:
                del m["rot"]
        elif up == "M":
            rot = {"dims": rot_dim, "base": 5000.0}
            if scaling:
                rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
            m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
                 "scale": (dim + rot_dim) ** -0.5, "mask": {"size": window}, "rot": rot}
        else:
            m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}
        layers.append({"type": {"A": "attention", "M": "latent_attention", "D": "delta"}[up], "mixer": m,
                       "mlp": {"kind": "dense", "ff": ff} if ch.isupper() else None})
    cfg = {"architecture": "Nopunex", "vocab": vocab, "width": width, "layers": layers, "norm": {"eps": eps},
           "logit_scale": logit_scale}
    if loop:
        cfg["loop"] = dict(zip(("start", "stop", "times"), loop))
    return cfg


def random_model(cfg: dict, seed: int = 0, std: float = 0.25) -> Dict[str, torch.Tensor]:
    """bf16-representable random tensors under the checkpoint names."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]
    r = lambda *shape, s=std: (torch.randn(*shape, generator=g) * s).bfloat16().double()
    w = {"embed": r(cfg["vocab"], W, s=1.0), "head": r(cfg["vocab"], W)}

    def norm(name):
        w[name], w[name + ".b"] = (1 + r(W, s=0.1)).bfloat16().double(), r(W, s=0.1)
    norm("final.norm")
    if cfg.get("loop"):
        w["loop.in"] = r(W, 2 * W, s=(2 * W) ** -0.5)
        w["loop.step"] = r(cfg["loop"]["times"], W, s=0.2)
    for i, l in enumerate(cfg["layers"]):
        p, m = f"l{i}.", l["mixer"]
        for q in ["1", "1b"] + (["2", "2b"] if l["mlp"] else []):
            norm(p + "norm" + q)
        p += "mix."
        if l["type"] == "attention":
            H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            w.update({p + "q": r(2 * H * D, W), p + "k": r(2 * G * D, W), p + "v": r(G * V, W), p + "g": r(H * V, W),
                      p + "o": r(W, H * V)})
            for n in ("lq1", "lk1", "lq2", "lk2"):
                w[p + n] = r(D, s=0.3)
        elif l["type"] == "latent_attention":
            H, D, Dr, V, R, Q = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
            w.update({p + "dq": r(Q, W), p + "dq.norm": (1 + r(Q, s=0.1)).bfloat16().double(), p + "uq": r(H * (D + Dr), Q),
                      p + "dkv": r(R + Dr, W), p + "dkv.norm": (1 + r(R, s=0.1)).bfloat16().double(),
                      p + "uk": r(H * D, R), p + "uv": r(H * V, R), p + "sink": r(H, s=1.0), p + "o": r(W, H * V)})
        else:
            H, G, D, V, K = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"]
            w.update({p + "q": r(G * D, W), p + "k": r(G * D, W), p + "v": r(H * V, W), p + "a": r(H, W), p + "b": r(H, W),
                      p + "g": r(H * V, W), p + "o": r(W, H * V), p + "q.conv": r(G * D, K, s=0.6),
                      p + "k.conv": r(G * D, K, s=0.6), p + "v.conv": r(H * V, K, s=0.6), p + "A_log": r(H, s=0.7),
                      p + "dt_bias": r(H, s=0.7), p + "norm": (1 + r(V, s=0.1)).bfloat16().double()})
        if l["mlp"]:
            F = l["mlp"]["ff"]
            w.update({f"l{i}.mlp.gate": r(F, W), f"l{i}.mlp.up": r(F, W), f"l{i}.mlp.down": r(W, F)})
    return w
