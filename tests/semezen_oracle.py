"""Slow float64 definition of the Semezen decoder, one function per mechanism, written from the
design's equations: dense attention over whole sequences, token-by-token recurrences, no
paging, no batching, no state carried between calls.  It shares no code with the package; the
tests compare the engine (CPU tier and HIP kernels) with it.

A model is ``(cfg, st)``: the checkpoint's ``config.json`` as a dict and its tensors by name.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rms_norm(x, w, eps):
    return rms(x, eps) * w.to(F64)


def token_shift(h, mu):
    """h [T, W]: every row moves towards the row before it (zeros before the first) by ``mu``."""
    prev = torch.cat([torch.zeros_like(h[:1]), h[:-1]], 0)
    return h + (prev - h) * mu.to(F64)


def rotary_frequencies(dims, base, scaling=None):
    """f_i = base^(-2i / dims), i < dims / 2, with the wavelength-dependent slow-down of long
    waves: short waves keep f, long ones get f / factor, the band between is blended."""
    out = []
    for i in range(dims // 2):
        f = float(base) ** (-2.0 * i / dims)
        if scaling:
            fac, lo, hi, orig = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
            wave = 2.0 * math.pi / f
            if wave < orig / hi:
                pass
            elif wave > orig / lo:
                f = f / fac
            else:
                s = (orig / wave - lo) / (hi - lo)
                f = (1.0 - s) * f / fac + s * f
        out.append(f)
    return torch.tensor(out, dtype=F64)


def rotate(x, pos, freqs):
    """x [T, H, d]: channel i pairs with channel i + n (n = len(freqs)) among the first 2 n."""
    n = freqs.shape[0]
    ang = pos.to(F64)[:, None] * freqs[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    u, v = x[..., :n], x[..., n:2 * n]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., 2 * n:]], -1)


def window_softmax_attention(q, k, v, scale, window):
    """q [T, H, d], k [T, G, d], v [T, G, dv]; row i attends rows j with 0 <= i - j < window."""
    T, H, _ = q.shape
    G = k.shape[1]
    rep = H // G
    out = torch.zeros(T, H, v.shape[2], dtype=F64)
    for h in range(H):
        g = h // rep
        for i in range(T):
            lo = max(0, i - window + 1)
            sc = (k[lo:i + 1, g] @ q[i, h]) * scale
            w = torch.softmax(sc, 0)
            out[i, h] = w @ v[lo:i + 1, g]
    return out


def attention_mixer(h, m, st, p, eps, pos0=0):
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = (h @ st[p + "q"].to(F64).T + st[p + "q.b"].to(F64)).view(T, H, d)
    k = (h @ st[p + "k"].to(F64).T + st[p + "k.b"].to(F64)).view(T, G, d)
    v = k.clone()                                   # values: the keys as projected
    rot = m.get("rot")
    if rot:
        fr = rotary_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
        pos = torch.arange(pos0, pos0 + T)
        q, k = rotate(q, pos, fr), rotate(k, pos, fr)
    q, k = rms(q, eps), rms(k, eps)
    window = (m.get("mask") or {}).get("size") or (T + pos0 + 1)
    a = window_softmax_attention(q, k, v, m["scale"], window).reshape(T, H * dv)
    a = a * torch.sigmoid(h @ st[p + "g"].to(F64).T)
    return a @ st[p + "o"].to(F64).T


def mingru_mixer(h, m, st, p):
    T = h.shape[0]
    z = torch.sigmoid(h @ st[p + "z"].to(F64).T + st[p + "z.b"].to(F64))
    u = h @ st[p + "x"].to(F64).T + st[p + "x.b"].to(F64)
    cand = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    g = h @ st[p + "g"].to(F64).T
    S = torch.zeros(m["width"], dtype=F64)
    rows = []
    for t in range(T):
        S = (1.0 - z[t]) * S + z[t] * cand[t]
        rows.append(S * (g[t] * torch.sigmoid(g[t])))
    return torch.stack(rows) @ st[p + "o"].to(F64).T


def gelu_erf(z):
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def dense_ff(h, st, p):
    return gelu_erf(h @ st[p + "up"].to(F64).T) @ st[p + "down"].to(F64).T


def expert(x, st, p, limit):
    g = torch.clamp(x @ st[p + "gate"].to(F64).T, max=limit)
    u = torch.clamp(x @ st[p + "up"].to(F64).T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ st[p + "down"].to(F64).T


def moe_ff(h, mlp, st, p, margins=None):
    """Every token's ``top`` best experts by sigmoid score; the score scales the expert's INPUT.
    ``margins`` receives, per token, the gap between the last chosen and the first rejected
    score (a small gap is a close call that rounding may decide the other way)."""
    s = torch.sigmoid(h @ st[p + "router"].to(F64).T)
    top = mlp["router"]["top"]
    if margins is not None and top < s.shape[1]:
        v = s.sort(1, descending=True).values
        margins.append(v[:, top - 1] - v[:, top])
    out = torch.zeros(h.shape[0], st[p + "e0.down"].shape[0], dtype=F64)
    for t in range(h.shape[0]):
        for e in torch.topk(s[t], top).indices.tolist():
            out[t] += expert(s[t, e] * h[t], st, f"{p}e{e}.", mlp["expert"]["limit"])
    return out


def forward(cfg, st, tokens, layers_out=None, margins=None):
    """Logits [T, vocab] of one whole sequence; ``layers_out`` receives the sum of the streams
    after every layer, ``margins`` every routed layer's per-token routing margin."""
    eps = cfg["norm"]["eps"]
    x0 = st["embed"].to(F64)[torch.as_tensor(tokens).long()]
    ns = int(cfg.get("streams") or 1)
    hyper = "streams" in cfg
    xs = [x0.clone() for _ in range(ns)]
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        for q in (1, 2):
            if q == 2 and not L.get("mlp"):
                continue
            if hyper:
                w_in = st[f"{p}hc{q}.in"].to(F64)
                u = sum(w_in[s] * xs[s] for s in range(ns))
            else:
                u = xs[0]
            n = rms_norm(u, st[f"{p}norm{q}"], eps)
            if q == 1:
                n = token_shift(n, st[p + "shift"]) if (p + "shift") in st else n
                if L["type"] == "attention":
                    y = attention_mixer(n, L["mixer"], st, p + "mix.", eps)
                elif L["type"] == "mingru":
                    y = mingru_mixer(n, L["mixer"], st, p + "mix.")
                else:
                    raise ValueError(L["type"])
            elif L["mlp"]["kind"] == "dense":
                y = dense_ff(n, st, p + "mlp.")
            else:
                y = moe_ff(n, L["mlp"], st, p + "mlp.", margins)
            if hyper:
                mix, w_out = st[f"{p}hc{q}.mix"].to(F64), st[f"{p}hc{q}.out"].to(F64)
                xs = [sum(mix[s, t] * xs[s] for s in range(ns)) + w_out[t] * y for t in range(ns)]
            else:
                xs = [xs[0] + y]
        if layers_out is not None:
            layers_out.append(sum(xs))
    x = sum(xs)
    return rms_norm(x, st["final.norm"], eps) @ st["head"].to(F64).T
