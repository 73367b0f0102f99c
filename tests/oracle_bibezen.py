"""Plain per-sequence model of the Bibezen design in double precision: one function per mechanism,
written from the equations below, sharing no code with the package.

Notation: U(u) = u / sqrt(mean(u^2) + eps); N_w(u) = U(u) (1 + w); F_c(u)_t = sum_j c[:, j] u_(t - K + 1 + j)
(a causal filter of K taps per channel, zeros before the sequence); sp(z) = log(1 + e^z).

    streams X_1..X_S (all = embed[token] * scale);  sublayer q with coefficients a[S], M[S, S], b[S]:
        u = sum_s a[s] X_s;  y = sublayer(N(u));  X_t <- sum_s M[s, t] X_s + m b[t] y
    the mixer reads h + F_canon(h) instead of h = N(u)
    logits = embed N_final(sum_s X_s)
"""
from __future__ import annotations

import torch

D64 = torch.float64


def unit(u, eps):
    return u / torch.sqrt((u * u).mean(-1, keepdim=True) + eps)


def norm_one_plus(u, w, eps):
    return unit(u, eps) * (1.0 + w)


def causal_filter(u, c, bias=None):
    """u [T, C], c [C, K]: y_t = sum_j c[:, j] u_(t - K + 1 + j)."""
    T, C = u.shape
    K = c.shape[1]
    pad = torch.cat([torch.zeros((K - 1, C), dtype=D64), u], 0)
    y = torch.zeros((T, C), dtype=D64)
    for j in range(K):
        y = y + pad[j:j + T] * c[:, j]
    return y if bias is None else y + bias


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30))))


def rotate_halves(x, dims, base):
    """x [T, heads, d]: coordinate i < dims/2 pairs with i + dims/2, angle = position * base^(-2i/dims)."""
    T = x.shape[0]
    n = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(n)], dtype=D64)
    ang = torch.arange(T, dtype=D64)[:, None] * f[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    out = x.clone()
    a, b = x[..., :n], x[..., n:2 * n]
    out[..., :n] = a * c - b * s
    out[..., n:2 * n] = b * c + a * s
    return out


def pooled_softmax(q, k, v, scale, cap=0.0, size=0, P=0, sink=None, talk=None):
    """q [T, H, D], k [T, G, D], v [T, G, V] of one sequence from position 0.  Query i sees keys
    max(0, i - size + 1) .. i (size 0: all) and the mean key / value of every block b of P positions with
    b P + P - 1 <= i - size; s = cap tanh(q . k scale / cap); the denominator also holds exp(sink_h);
    the weights of all heads are mixed by talk [H, H] before they meet head h's own values.  -> [T, H, V]"""
    T, H, D = q.shape
    G, V = k.shape[1], v.shape[2]
    nb = T // P if (P and size) else 0
    if nb:
        kb, vb = k[:nb * P].view(nb, P, G, D).mean(1), v[:nb * P].view(nb, P, G, V).mean(1)
    rep = H // G
    wts = torch.zeros((H, T, T + nb), dtype=D64)      # softmax weights over single keys then blocks
    for i in range(T):
        seen = torch.zeros(T + nb, dtype=torch.bool)
        seen[(max(0, i - size + 1) if size else 0):i + 1] = True
        for b in range(nb):
            if b * P + P - 1 <= i - size:
                seen[T + b] = True
        for hh in range(H):
            g = hh // rep
            sc = torch.cat([k[:, g] @ q[i, hh], kb[:, g] @ q[i, hh]] if nb else [k[:, g] @ q[i, hh]]) * scale
            if cap:
                sc = cap * torch.tanh(sc / cap)
            sc = sc[seen]
            m = sc.max()
            if sink is not None:
                m = torch.maximum(m, sink[hh])
            e = torch.exp(sc - m)
            den = e.sum() + (torch.exp(sink[hh] - m) if sink is not None else 0.0)
            wts[hh, i, seen] = e / den
    if talk is not None:
        wts = torch.einsum("hg,gij->hij", talk, wts)
    o = torch.zeros((T, H, V), dtype=D64)
    for hh in range(H):
        g = hh // rep
        o[:, hh] = wts[hh] @ (torch.cat([v[:, g], vb[:, g]], 0) if nb else v[:, g])
    return o


def pooled_window_attention(h, t, s, eps):
    """The softmax attention branch: biased projections, filters, weighted unit RMS per head,
    rotation, then :func:`pooled_softmax` and the output projection."""
    T = h.shape[0]
    H, G, D, V = s["heads"], s["kv_heads"], s["dim"], s["vdim"]

    def proj(n):
        y = h @ t[n].T
        if n + ".b" in t:
            y = y + t[n + ".b"]
        if n + ".conv" in t:
            y = causal_filter(y, t[n + ".conv"])
        return y
    q, k, v = proj("q").view(T, H, D), proj("k").view(T, G, D), proj("v").view(T, G, V)
    if "q.norm" in t:
        q = unit(q, eps) * t["q.norm"]
    if "k.norm" in t:
        k = unit(k, eps) * t["k.norm"]
    rot = s.get("rot")
    if rot:
        q, k = rotate_halves(q, rot["dims"], rot["base"]), rotate_halves(k, rot["dims"], rot["base"])
    mask = s.get("mask") or {}
    o = pooled_softmax(q, k, v, s["scale"], s.get("softcap", 0.0), mask.get("size", 0), mask.get("pool", 0),
                       t.get("sink"), t.get("talk"))
    return o.reshape(T, H * V) @ t["o"].T


def wkv(h, t, s, eps):
    """Time mixing with per-channel decays: token-shift mixes, low-rank decay, bonus for the current
    token, matrix state per head, unit RMS per head, weight, SiLU gate."""
    T, W = h.shape
    H, D = s["heads"], s["dim"]
    prev = torch.cat([torch.zeros((1, W), dtype=D64), h[:-1]], 0)
    mix = lambda n: h + (prev - h) * t["mu." + n]
    r, k, v = (mix(n) @ t[n].T for n in "rkv")
    gate = silu(mix("g") @ t["g"].T)
    dec = torch.exp(-torch.exp(torch.tanh(mix("w") @ t["w1"].T) @ t["w2"].T + t["w0"]))
    r, k, v, dec = r.view(T, H, D), k.view(T, H, D), v.view(T, H, D), dec.view(T, H, D)
    u = t["u"].view(H, D)
    S = torch.zeros((H, D, D), dtype=D64)
    o = torch.zeros((T, H, D), dtype=D64)
    for i in range(T):
        kv = k[i][:, :, None] * v[i][:, None, :]
        o[i] = torch.einsum("hd,hdv->hv", r[i], S + u[:, :, None] * kv)
        S = dec[i][:, :, None] * S + kv
    o = unit(o, eps).reshape(T, H * D) * t["norm"] * gate
    return o @ t["o"].T


def selective_scan(h, t, s):
    """Input-dependent state-space mixer: filter + SiLU, step sizes by softplus, diagonal state per channel."""
    T = h.shape[0]
    I, N, R = s["inner"], s["state"], s["dt_rank"]
    xz = h @ t["in"].T
    x, z = xz[:, :I], xz[:, I:]
    x = silu(causal_filter(x, t["conv"], t.get("conv.b")))
    low = x @ t["x"].T
    dt = softplus(low[:, :R] @ t["dt"].T + t["dt.b"])
    B, C = low[:, R:R + N], low[:, R + N:]
    A = -torch.exp(t["A_log"])
    S = torch.zeros((I, N), dtype=D64)
    y = torch.zeros((T, I), dtype=D64)
    for i in range(T):
        S = torch.exp(dt[i][:, None] * A) * S + (dt[i] * x[i])[:, None] * B[i][None, :]
        y[i] = S @ C[i] + t["D"] * x[i]
    return (y * silu(z)) @ t["o"].T


def parallel(h, t, s, eps):
    sub = lambda side: {k[len(side) + 1:]: v for k, v in t.items() if k.startswith(side + ".")}
    return s["left_scale"] * pooled_window_attention(h, sub("left"), s["left"], eps) + \
        s["right_scale"] * wkv(h, sub("right"), s["right"], eps)


def dense_ff(h, t, f):
    L = f["limit"]
    g = torch.clamp(h @ t["gate"].T, max=L)
    u = torch.clamp(h @ t["up"].T, -L, L)
    return (g * torch.sigmoid(1.702 * g) * (u + 1)) @ t["down"].T


def gated_expert(h, t, p):
    return (silu(h @ t[p + "gate"].T) * (h @ t[p + "up"].T)) @ t[p + "down"].T


def moe_ff(h, t, f):
    E, top = f["router"]["experts"], f["router"]["top"]
    z = h @ t["router"].T
    out = torch.zeros((h.shape[0], t["e0.down"].shape[0]), dtype=D64)
    for i in range(h.shape[0]):
        order = sorted(range(E), key=lambda e: (-float(z[i, e]), e))[:top]
        w = torch.softmax(z[i, order], 0)
        for j, e in enumerate(order):
            out[i] += w[j] * gated_expert(h[i:i + 1], t, f"e{e}.")[0]
    if f.get("shared"):
        out = out + gated_expert(h, t, "shared.")
    return out


MIXERS = {"wkv": lambda h, t, s, eps: wkv(h, t, s, eps), "mamba1": lambda h, t, s, eps: selective_scan(h, t, s),
          "parallel": parallel}


def forward(cfg: dict, tensors: dict, tokens):
    """Logits [T, vocab] and the streams' sum after every layer [layers, T, W] of one sequence."""
    t64 = {k: v.to(D64) for k, v in tensors.items()}
    eps = cfg["norm"]["eps"]
    m = cfg.get("residual_mult", 1.0)
    S = cfg.get("streams", 0)
    W = cfg["width"]
    x0 = t64["embed"][torch.as_tensor(tokens, dtype=torch.long)] * cfg.get("embedding", {}).get("scale", 1.0)
    xs = [x0.clone() for _ in range(max(S, 1))]
    taps = (cfg.get("canon") or {}).get("taps", 0)
    after = []
    for i, l in enumerate(cfg["layers"]):
        p = f"l{i}."
        sub = lambda pre: {k[len(p + pre):]: v for k, v in t64.items() if k.startswith(p + pre)}
        for q in (1, 2):
            if q == 2 and l.get("mlp") is None:
                continue
            if S:
                a, M, b = t64[p + f"hc{q}.in"], t64[p + f"hc{q}.mix"], t64[p + f"hc{q}.out"]
            else:
                a, M, b = torch.ones(1, dtype=D64), torch.ones((1, 1), dtype=D64), torch.ones(1, dtype=D64)
            u = sum(a[s] * xs[s] for s in range(len(xs)))
            h = norm_one_plus(u, t64[p + f"norm{q}"], eps)
            if q == 1:
                if taps and p + "canon1" in t64:
                    h = h + causal_filter(h, t64[p + "canon1"])
                y = MIXERS[l["type"]](h, sub("mix."), l["mixer"], eps)
            else:
                y = dense_ff(h, sub("mlp."), l["mlp"]) if l["mlp"]["kind"] == "dense" else moe_ff(h, sub("mlp."), l["mlp"])
            xs = [sum(M[s, tt] * xs[s] for s in range(len(xs))) + m * b[tt] * y for tt in range(len(xs))]
        after.append(sum(xs))
    x = norm_one_plus(sum(xs), t64["final.norm"], eps)
    return x @ t64["embed"].T, torch.stack(after)



# ------------------------------------------------------------------ small configurations and random weights
def make_config(pattern=("wkv:dense", "parallel:moe", "mamba1:moe", "parallel:none"), vocab=96, width=48, streams=2,
                heads=4, kv_heads=2, dim=16, vdim=8, rot_dims=8, window=24, pool=5, conv=3, softcap=15.0, wheads=3,
                wdim=12, inner=40, state=6, dt_rank=5, mconv=4, ff=56, experts=5, top=2, eff=24, shared=32, taps=3,
                mult=0.5, scale=None):
    """A config.json dict: ``pattern`` lists "mixer:feed-forward" per layer."""
    layers = []
    for item in pattern:
        kind, ffk = item.split(":")
        if kind == "wkv":
            mixer = {"heads": wheads, "dim": wdim}
        elif kind == "mamba1":
            mixer = {"inner": inner, "state": state, "dt_rank": dt_rank, "conv": mconv}
        else:
            left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv, "scale": dim ** -0.5,
                    "softcap": softcap, "mask": {"size": window, "pool": pool}}
            if rot_dims:
                left["rot"] = {"dims": rot_dims, "base": 1000.0}
            mixer = {"left": left, "right": {"heads": wheads, "dim": wdim}, "left_scale": 0.7, "right_scale": 1.2}
        mlp = None
        if ffk == "dense":
            mlp = {"kind": "dense", "ff": ff, "limit": 1.5}
        elif ffk == "moe":
            mlp = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": eff}}
            if shared:
                mlp["shared"] = {"ff": shared}
        layers.append({"type": kind, "mixer": mixer, "mlp": mlp})
    cfg = {"architecture": "Bibezen", "vocab": vocab, "width": width, "norm": {"eps": 1e-5}, "residual_mult": mult,
           "embedding": {"scale": scale if scale is not None else float(width) ** 0.5}, "layers": layers}
    if streams:
        cfg["streams"] = streams
    if taps:
        cfg["canon"] = {"taps": taps}
    return cfg


def random_model(cfg, seed=0, std=None):
    """Random bf16-representable tensors under the checkpoint names."""
    g = torch.Generator().manual_seed(seed)
    W, S = cfg["width"], cfg.get("streams", 0)
    out = {}

    def r(name, shape, s, mean=0.0):
        out[name] = (mean + torch.randn(shape, generator=g) * s).to(torch.bfloat16).float()
    fan = lambda n: std if std is not None else n ** -0.5

    def wkv_weights(p, m):
        n = m["heads"] * m["dim"]
        for x in "rkvgw":
            r(p + "mu." + x, (W,), 0.25, 0.5)
        for x in "rkvg":
            r(p + x, (n, W), fan(W))
        r(p + "w1", (7, W), fan(W)), r(p + "w2", (n, 7), 0.4), r(p + "w0", (n,), 1.5, -1.0)
        r(p + "u", (m["heads"], m["dim"]), 0.5), r(p + "norm", (n,), 0.1, 1.0), r(p + "o", (W, n), fan(n))

    r("embed", (cfg["vocab"], W), W ** -0.5), r("final.norm", (W,), 0.1)
    for i, l in enumerate(cfg["layers"]):
        p, m = f"l{i}.", l["mixer"]
        for q in ["1"] + (["2"] if l["mlp"] is not None else []):
            r(p + "norm" + q, (W,), 0.1)
            if S:
                r(p + f"hc{q}.in", (S,), 0.15, 1.0 / S), r(p + f"hc{q}.out", (S,), 0.2, 1.0)
                r(p + f"hc{q}.mix", (S, S), 0.1)
                out[p + f"hc{q}.mix"] = (out[p + f"hc{q}.mix"] + torch.eye(S)).to(torch.bfloat16).float()
        if (cfg.get("canon") or {}).get("taps"):
            r(p + "canon1", (W, cfg["canon"]["taps"]), 0.25)
        if l["type"] == "wkv":
            wkv_weights(p + "mix.", m)
        elif l["type"] == "mamba1":
            I, N, R, K = m["inner"], m["state"], m["dt_rank"], m["conv"]
            r(p + "mix.in", (2 * I, W), fan(W)), r(p + "mix.conv", (I, K), 0.4), r(p + "mix.conv.b", (I,), 0.1)
            r(p + "mix.x", (R + 2 * N, I), fan(I)), r(p + "mix.dt", (I, R), fan(R)), r(p + "mix.dt.b", (I,), 1.0, -1.5)
            r(p + "mix.A_log", (I, N), 0.5, 0.3), r(p + "mix.D", (I,), 0.5), r(p + "mix.o", (W, I), fan(I))
        else:
            a, q = m["left"], p + "mix.left."
            H, G, D, V = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
            for n, rows in (("q", H * D), ("k", G * D), ("v", G * V)):
                r(q + n, (rows, W), fan(W)), r(q + n + ".b", (rows,), 0.1)
                if a.get("conv"):
                    r(q + n + ".conv", (rows, a["conv"]), 0.5)
            r(q + "q.norm", (D,), 0.1, 1.0), r(q + "k.norm", (D,), 0.1, 1.0), r(q + "sink", (H,), 1.0)
            r(q + "talk", (H, H), 0.2)
            out[q + "talk"] = (out[q + "talk"] + torch.eye(H)).to(torch.bfloat16).float()
            r(q + "o", (W, H * V), fan(H * V))
            wkv_weights(p + "mix.right.", m["right"])
        f = l["mlp"]
        if f is None:
            continue
        if f["kind"] == "dense":
            r(p + "mlp.gate", (f["ff"], W), fan(W)), r(p + "mlp.up", (f["ff"], W), fan(W)), r(p + "mlp.down", (W, f["ff"]), fan(f["ff"]))
        else:
            r(p + "mlp.router", (f["router"]["experts"], W), 0.6)
            names = [(f"e{e}", f["expert"]["ff"]) for e in range(f["router"]["experts"])]
            if f.get("shared"):
                names.append(("shared", f["shared"]["ff"]))
            for n, ffn in names:
                r(p + f"mlp.{n}.gate", (ffn, W), fan(W)), r(p + f"mlp.{n}.up", (ffn, W), fan(W))
                r(p + f"mlp.{n}.down", (W, ffn), fan(ffn))
    return out
