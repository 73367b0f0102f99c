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


def pooled_window_attention(h, t, s, eps):
    """The softmax attention branch: biased projections, filters, head norms, rotation, capped scores,
    a window of single keys plus block means behind it, a sink in the denominator, head mixing."""
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
    size, P = mask.get("size", 0), mask.get("pool", 0)
    cap = s.get("softcap", 0.0)
    nb = T // P if P else 0
    if nb:
        kb, vb = k[:nb * P].view(nb, P, G, D).mean(1), v[:nb * P].view(nb, P, G, V).mean(1)
    rep = H // G
    wts = torch.zeros((H, T, T + nb), dtype=D64)      # softmax weights over single keys then blocks
    for i in range(T):
        seen = torch.zeros(T + nb, dtype=torch.bool)
        lo = max(0, i - size + 1) if size else 0
        seen[lo:i + 1] = True
        if size:
            for b in range(nb):
                if b * P + P - 1 <= i - size:
                    seen[T + b] = True
        for hh in range(H):
            g = hh // rep
            sc = torch.cat([k[:, g] @ q[i, hh], kb[:, g] @ q[i, hh]] if nb else [k[:, g] @ q[i, hh]]) * s["scale"]
            if cap:
                sc = cap * torch.tanh(sc / cap)
            sc = sc[seen]
            m = sc.max()
            sink = t["sink"][hh] if "sink" in t else None
            if sink is not None:
                m = torch.maximum(m, sink)
            e = torch.exp(sc - m)
            den = e.sum() + (torch.exp(sink - m) if sink is not None else 0.0)
            wts[hh, i, seen] = e / den
    if "talk" in t:
        wts = torch.einsum("hg,gij->hij", t["talk"], wts)
    o = torch.zeros((T, H, V), dtype=D64)
    for hh in range(H):
        g = hh // rep
        vals = torch.cat([v[:, g], vb[:, g]], 0) if nb else v[:, g]
        o[:, hh] = wts[hh] @ vals
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

